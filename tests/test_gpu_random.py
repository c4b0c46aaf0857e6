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
