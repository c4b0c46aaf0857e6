"""Seeded random collectives through the HCCL entry points: rank counts up to 64, every reduce type and op the
entry points take, every template, ragged counts, both execution modes, compared bit for bit with the oracle."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api

from gpu_util import DevBuf, assert_same_bits, payload

pytestmark = pytest.mark.gpu

SMALL_CCL = 1024 * 1024 + 64 * 1024
AR_ALGS = list(T.ALLREDUCE_TEMPLATES)
RS_ALGS = [a for a in T.REDUCE_SCATTER_TEMPLATES]
TYPES = [T.INT8, T.INT16, T.INT32, T.INT64, T.FP16, T.FP32, T.FP64, T.BFP16]


def draw(rng):
    dtype = TYPES[int(rng.integers(len(TYPES)))]
    ops = [T.SUM, T.MAX, T.MIN] + ([T.PROD] if dtype not in (T.INT16, T.BFP16) else [])   # HcclAllReduce takes no PROD there
    op = ops[int(rng.integers(len(ops)))]
    n = int([2, 3, 5, 8, 12, 16, 17, 24, 33, 48, 64][int(rng.integers(11))])
    mode = api.EXEC_FUSED if rng.integers(4) else api.EXEC_STEP
    return dtype, op, n, mode


def ccl_for(n):
    """A small scratch buffer forces several executor loops; among many ranks the default one keeps the number of
    recorded steps (loops x ranks^2 or ranks^3) reasonable."""
    return SMALL_CCL if n <= 24 else T.CCL_BYTES_DEFAULT


def wide_sum(dtype, op, fused):
    return fused and dtype in (T.FP16, T.BFP16) and op == T.SUM


@pytest.mark.parametrize("seed", range(24))
def test_random_allreduce(seed):
    rng = np.random.default_rng(1000 + seed)
    dtype, op, n, mode = draw(rng)
    alg = AR_ALGS[int(rng.integers(len(AR_ALGS)))]
    count = int(rng.integers(1, 60000))
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    xs = [payload(rng, dtype, count, kind) for _ in range(n)]
    esz = T.DTYPE_SIZE[dtype]
    s = torch.cuda.Stream()
    ccl = ccl_for(n)
    w = api.World(n, ccl_bytes=ccl)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        send = [DevBuf(x, offset=int(rng.integers(4)) * esz) for x in xs]
        recv = [DevBuf(nbytes=count * esz, offset=int(rng.integers(4)) * esz) for _ in range(n)]
        torch.cuda.synchronize()
        for r in rng.permutation(n):          # the ranks call in any order
            assert w.all_reduce(int(r), send[r].ptr, recv[r].ptr, count, dtype, op, s.cuda_stream) == 0
        s.synchronize()
        info = w.last_info()
        what = f"seed {seed}: {alg} n={n} dtype={dtype} op={op} count={count} fused={info.fused}"
        if wide_sum(dtype, op, info.fused):
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_allreduce(T.NumericElems(T.FP32, T.SUM), wide, count, esz, alg, ccl_bytes=ccl)]
        else:
            want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=ccl)
        for r in range(n):
            assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype, f"{what} rank {r}")
            assert recv[r].guard_intact() and send[r].guard_intact(), what
    finally:
        w.close()


@pytest.mark.parametrize("seed", range(16))
def test_random_reduce_scatter(seed):
    rng = np.random.default_rng(2000 + seed)
    dtype, op, n, mode = draw(rng)
    alg = RS_ALGS[int(rng.integers(len(RS_ALGS)))]
    rc = int(rng.integers(1, 9000))
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    xs = [payload(rng, dtype, n * rc, kind) for _ in range(n)]
    esz = T.DTYPE_SIZE[dtype]
    s = torch.cuda.Stream()
    ccl = ccl_for(n)
    w = api.World(n, ccl_bytes=ccl)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
        send = [DevBuf(x, offset=int(rng.integers(4)) * esz) for x in xs]
        recv = [DevBuf(nbytes=rc * esz, offset=int(rng.integers(4)) * esz) for _ in range(n)]
        torch.cuda.synchronize()
        for r in rng.permutation(n):
            assert w.reduce_scatter(int(r), send[r].ptr, recv[r].ptr, rc, dtype, op, s.cuda_stream) == 0
        s.synchronize()
        info = w.last_info()
        what = f"seed {seed}: {alg} n={n} dtype={dtype} op={op} recv={rc} fused={info.fused}"
        if wide_sum(dtype, op, info.fused):
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), wide, rc, esz, alg, ccl_bytes=ccl)]
        else:
            want = T.run_reduce_scatter(T.NumericElems(dtype, op), xs, rc, esz, alg, ccl_bytes=ccl)
        for r in range(n):
            assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype, f"{what} rank {r}")
            assert recv[r].guard_intact() and send[r].guard_intact(), what
    finally:
        w.close()


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("mode", [api.EXEC_FUSED, api.EXEC_STEP])
def test_random_buffers_in_one_world(alg, mode):
    """One world, a few shapes, buffers that keep changing (new ones with random alignment, old ones coming back, in
    place now and then): plans are made, moved to other buffers and replayed in whatever order that gives, and every
    result is the oracle's."""
    n = 12 if alg != "InsAllReduceMesh1DOneShot" else 20
    rng = np.random.default_rng(len(alg) * 10 + mode)
    s = torch.cuda.Stream()
    shapes = [(T.FP32, T.SUM, 4099), (T.BFP16, T.SUM, 30011), (T.INT32, T.MAX, 777), (T.FP32, T.MAX, 20000)]
    seen = {0: 0, 1: 0, 2: 0}
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        pool = []
        for it in range(20):
            dtype, op, count = shapes[int(rng.integers(len(shapes)))]
            esz = T.DTYPE_SIZE[dtype]
            known = [p for p in pool if p[0] == (dtype, op, count)]
            if known and rng.integers(3) == 0:
                _, send, recv = known[int(rng.integers(len(known)))]
            else:
                send = [DevBuf(nbytes=count * esz, offset=int(rng.integers(5)) * esz) for _ in range(n)]
                recv = send if rng.integers(4) == 0 else [DevBuf(nbytes=count * esz, offset=int(rng.integers(5)) * esz)
                                                          for _ in range(n)]
                pool = (pool + [((dtype, op, count), send, recv)])[-6:]
            xs = [payload(rng, dtype, count, "uniform" if dtype == T.FP32 else "normal") for _ in range(n)]
            for r in range(n):
                send[r].t[send[r].offset:send[r].offset + count * esz] = torch.from_numpy(
                    xs[r].view(np.uint8).reshape(-1).copy()).to("cuda:0")
            torch.cuda.synchronize()
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, s.cuda_stream) == 0
            s.synchronize()
            info = w.last_info()
            seen[info.planCacheHit] += 1
            if wide_sum(dtype, op, info.fused):
                outs = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), [T.widen16(x, dtype) for x in xs], count, esz, alg,
                                       ccl_bytes=SMALL_CCL)
                want = [T.narrow16(o, dtype) for o in outs]
            else:
                want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=SMALL_CCL)
            for r in range(n):
                assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype,
                                 f"{alg} call {it} rank {r} cache {info.planCacheHit}")
                assert recv[r].guard_intact()
        assert seen[0] >= 1 and seen[2] >= 1, seen     # planned at least once, moved at least once
    finally:
        w.close()


MOVE_TYPES = [(T.INT8, np.uint8), (T.FP16, np.uint16), (T.FP32, np.uint32), (T.INT64, np.uint64)]


def scattered(rng, counts):
    """Non-overlapping places for blocks of the given lengths, in a random order with random gaps: the
    displacement of each block and the length of the buffer that holds them all."""
    displs = [0] * len(counts)
    at = int(rng.integers(3))
    for i in rng.permutation(len(counts)):
        displs[i] = at
        at += counts[i] + int(rng.integers(4))
    return displs, at


def ragged(rng, k, top):
    """k counts of which about a quarter are zero and a few are long."""
    c = rng.integers(0, top, size=k)
    c[rng.random(k) < 0.25] = 0
    long_ones = rng.random(k) < 0.05
    c[long_ones] = rng.integers(top, 20 * top, size=int(long_ones.sum()))
    return [int(x) for x in c]


@pytest.mark.parametrize("seed", range(12))
def test_random_reduce_scatter_v(seed):
    """HcclReduceScatterV: random ragged parts at scattered places of the input, any type and op, both modes."""
    rng = np.random.default_rng(3000 + seed)
    dtype, op, n, mode = draw(rng)
    n = min(n, 33)
    counts = ragged(rng, n, 3000)
    if max(counts) == 0:
        counts[int(rng.integers(n))] = 17
    displs, total = scattered(rng, counts)
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    xs = [payload(rng, dtype, max(total, 1), kind) for _ in range(n)]
    esz = T.DTYPE_SIZE[dtype]
    s = torch.cuda.Stream()
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        send = [DevBuf(x, offset=int(rng.integers(4)) * esz) for x in xs]
        recv = [DevBuf(nbytes=max(counts[r], 1) * esz, offset=int(rng.integers(4)) * esz) for r in range(n)]
        torch.cuda.synchronize()
        # fp64 has no ReduceScatterV algorithm in the reference (reduce_scatter_v_auto_selector.cc:204-220)
        # (the collective is selected and launched when its last rank has called: that call reports it)
        rcs = [w.reduce_scatter_v(int(r), send[r].ptr, counts, displs, recv[r].ptr, counts[r], dtype, op, s.cuda_stream)
               for r in rng.permutation(n)]
        s.synchronize()
        assert rcs[:-1] == [0] * (n - 1)
        if dtype == T.FP64:
            assert rcs[-1] == 5     # HCCL_E_NOT_SUPPORT
            return
        assert rcs[-1] == 0
        info = w.last_info()
        what = f"seed {seed}: n={n} dtype={dtype} op={op} counts={counts} fused={info.fused}"
        if wide_sum(dtype, op, info.fused):
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_reduce_scatter_v(T.NumericElems(T.FP32, T.SUM), wide, counts, displs, esz, ccl_bytes=SMALL_CCL)]
        else:
            want = T.run_reduce_scatter_v(T.NumericElems(dtype, op), xs, counts, displs, esz, ccl_bytes=SMALL_CCL)
        for r in range(n):
            got = recv[r].get(T.NP_STORAGE[dtype])[:counts[r]]
            assert_same_bits(got, want[r], dtype, f"{what} rank {r}")
            if counts[r]:
                assert recv[r].guard_intact(), what
            assert send[r].guard_intact(), what
    finally:
        w.close()


@pytest.mark.parametrize("seed", range(16))
def test_random_allgather_family(seed):
    """HcclAllGather and HcclAllGatherV: random rank counts up to 64, ragged counts with zeros, parts at scattered
    places of the output; what lies between the parts keeps its bytes."""
    rng = np.random.default_rng(4000 + seed)
    n = int([2, 3, 5, 8, 12, 16, 17, 24, 33, 48, 64][int(rng.integers(11))])
    mode = api.EXEC_FUSED if rng.integers(4) else api.EXEC_STEP
    dtype, npd = MOVE_TYPES[int(rng.integers(len(MOVE_TYPES)))]
    esz = np.dtype(npd).itemsize
    top = np.iinfo(npd).max
    s = torch.cuda.Stream()
    w = api.World(n, ccl_bytes=ccl_for(n))
    try:
        w.set_mode(mode)
        if rng.integers(3) == 0:
            count = int(rng.integers(1, 40000))
            alg = ["InsAllGatherMesh1D", "InsAllGatherNHR"][int(rng.integers(2))]
            w.set_algorithm(api.CMD_ALLGATHER, alg)
            xs = [rng.integers(0, top, size=count, dtype=npd, endpoint=True) for _ in range(n)]
            send = [DevBuf(x, offset=int(rng.integers(4)) * esz) for x in xs]
            recv = [DevBuf(nbytes=n * count * esz, offset=int(rng.integers(4)) * esz) for _ in range(n)]
            torch.cuda.synchronize()
            for r in rng.permutation(n):
                assert w.all_gather(int(r), send[r].ptr, recv[r].ptr, count, dtype, s.cuda_stream) == 0
            s.synchronize()
            want = T.run_allgather(xs, count)
            what = f"seed {seed}: {alg} n={n} dtype={dtype} count={count} mode={mode}"
        else:
            counts = ragged(rng, n, 4000)
            displs, total = scattered(rng, counts)
            total = max(total, 1)
            xs = [rng.integers(0, top, size=c, dtype=npd, endpoint=True) for c in counts]
            before = [rng.integers(0, top, size=total, dtype=npd, endpoint=True) for _ in range(n)]
            send = [DevBuf(x if x.size else np.zeros(1, npd), offset=int(rng.integers(4)) * esz) for x in xs]
            recv = [DevBuf(b, offset=int(rng.integers(4)) * esz) for b in before]
            torch.cuda.synchronize()
            for r in rng.permutation(n):
                sp = send[r].ptr if counts[r] else None
                assert w.all_gather_v(int(r), sp, counts[r], recv[r].ptr, counts, displs, dtype, s.cuda_stream) == 0
            s.synchronize()
            want = [T.run_allgatherv(xs, counts, displs, total, before[j])[j] for j in range(n)]
            what = f"seed {seed}: AllGatherV n={n} dtype={dtype} counts={counts} mode={mode}"
        for r in range(n):
            assert np.array_equal(recv[r].get(npd), want[r]), f"{what} rank {r}"
            assert recv[r].guard_intact() and send[r].guard_intact(), what
    finally:
        w.close()


@pytest.mark.parametrize("seed", range(16))
def test_random_alltoall_family(seed):
    """HcclAlltoAll, HcclAlltoAllV and HcclAlltoAllVC: random count matrices with zeros and a few long blocks; for
    AlltoAllV the blocks lie at scattered places of both buffers, in any order."""
    rng = np.random.default_rng(5000 + seed)
    n = int([2, 3, 5, 8, 12, 16, 17, 24, 33, 48, 64][int(rng.integers(11))])
    mode = api.EXEC_FUSED if rng.integers(4) else api.EXEC_STEP
    dtype, npd = MOVE_TYPES[int(rng.integers(len(MOVE_TYPES)))]
    esz = np.dtype(npd).itemsize
    top = np.iinfo(npd).max
    kind = ["v", "vc", "uniform"][int(rng.integers(3))]
    s = torch.cuda.Stream()
    w = api.World(n, ccl_bytes=ccl_for(n))
    try:
        w.set_mode(mode)
        if kind == "uniform":
            c = int(rng.integers(1, 3000))
            m = [[c] * n for _ in range(n)]
        else:
            m = [ragged(rng, n, 1500 if n <= 24 else 300) for _ in range(n)]
        if kind == "v":
            sd, send_len, rd, recv_len = [], [], [], []
            for r in range(n):
                d, total = scattered(rng, m[r])
                sd.append(d)
                send_len.append(max(total, 1))
                d, total = scattered(rng, [m[i][r] for i in range(n)])
                rd.append(d)
                recv_len.append(max(total, 1))
            sc = m
            rc = [[m[i][r] for i in range(n)] for r in range(n)]
        else:
            v = [T.alltoallvc_to_v(m, r) for r in range(n)]
            sc, sd, rc, rd = ([x[k] for x in v] for k in range(4))
            send_len = [max(sum(x), 1) for x in sc]
            recv_len = [max(sum(x), 1) for x in rc]
        xs = [rng.integers(0, top, size=send_len[r], dtype=npd, endpoint=True) for r in range(n)]
        before = [rng.integers(0, top, size=recv_len[r], dtype=npd, endpoint=True) for r in range(n)]
        send = [DevBuf(x, offset=int(rng.integers(4)) * esz) for x in xs]
        recv = [DevBuf(b, offset=int(rng.integers(4)) * esz) for b in before]
        torch.cuda.synchronize()
        for r in rng.permutation(n):
            r = int(r)
            sp = send[r].ptr if sum(sc[r]) else None
            rp = recv[r].ptr if sum(rc[r]) else None
            if kind == "v":
                assert w.all_to_all_v(r, sp, sc[r], sd[r], rp, rc[r], rd[r], dtype, s.cuda_stream) == 0
            elif kind == "vc":
                assert w.all_to_all_vc(r, sp, [x for row in m for x in row], rp, dtype, s.cuda_stream) == 0
            else:
                assert w.all_to_all(r, sp, m[0][0], rp, dtype, s.cuda_stream) == 0
        s.synchronize()
        what = f"seed {seed}: AlltoAll {kind} n={n} dtype={dtype} mode={mode}"
        want = T.run_alltoallv(xs, sc, sd, rc, rd, recv_len, before)
        for j in range(n):
            assert np.array_equal(recv[j].get(npd), want[j]), f"{what} rank {j}"
            assert recv[j].guard_intact() and send[j].guard_intact(), what
    finally:
        w.close()
