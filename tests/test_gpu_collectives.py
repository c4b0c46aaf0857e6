"""GPU parity of the collectives through the HCCL entry points (HcclAllReduce ... HcclAlltoAllVC) for
virtual ranks, in both execution modes, against the CPU oracle's restatement of the same template."""
import threading

import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api

from gpu_util import DevBuf, assert_same_bits, payload

pytestmark = pytest.mark.gpu

SMALL_CCL = 1024 * 1024 + 64 * 1024
AR_ALGS = list(T.ALLREDUCE_TEMPLATES)
MODES = [api.EXEC_FUSED, api.EXEC_STEP]


@pytest.fixture(scope="module")
def stream():
    s = torch.cuda.Stream()
    yield s
    s.synchronize()


def wide_oracle_allreduce(xs, count, dtype, alg, ccl):
    """16-bit float SUM as a fused pass computes it: the template's order in fp32, one narrowing."""
    wide = [T.widen16(x, dtype) for x in xs]
    outs = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), wide, count, T.DTYPE_SIZE[dtype], alg, ccl_bytes=ccl)
    return [T.narrow16(o, dtype) for o in outs]


def run_allreduce(world, stream, xs, count, dtype, op, in_place=False):
    n = len(xs)
    send = [DevBuf(x) for x in xs]
    recv = send if in_place else [DevBuf(nbytes=xs[0].nbytes) for _ in range(n)]
    torch.cuda.synchronize()
    for r in range(n):
        assert world.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
    stream.synchronize()
    return [b.get(T.NP_STORAGE[dtype]) for b in recv], recv


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("dtype,op,n,count", [(T.FP32, T.SUM, 8, 131072 + 5), (T.FP32, T.PROD, 12, 40000),
                                             (T.INT32, T.MAX, 12, 70001), (T.BFP16, T.SUM, 8, 100003),
                                             (T.FP16, T.PROD, 5, 50001), (T.FP64, T.MIN, 3, 30000),
                                             (T.INT8, T.SUM, 16, 200001)])
def test_allreduce_every_template_both_modes(stream, mode, alg, dtype, op, n, count):
    rng = np.random.default_rng(n * 7 + count)
    kind = "prod" if op == T.PROD else "uniform" if dtype == T.FP32 else "normal"
    xs = [payload(rng, dtype, count, kind) for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        got, bufs = run_allreduce(w, stream, xs, count, dtype, op)
        info = w.last_info()
        if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
            want = wide_oracle_allreduce(xs, count, dtype, alg, SMALL_CCL)
        else:
            want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], alg, ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(got[r], want[r], dtype, f"{alg} rank {r} fused={info.fused}")
            assert bufs[r].guard_intact()
        if mode == api.EXEC_STEP:
            assert info.fused == 0 and info.launches >= info.levels
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_allreduce_in_place(stream, mode):
    rng = np.random.default_rng(3)
    n, count = 8, 65536 + 1
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n, ccl_bytes=4 << 20)
    try:
        w.set_mode(mode)
        got, _ = run_allreduce(w, stream, xs, count, T.FP32, T.SUM, in_place=True)
        alg = w.last_info().algName.decode()
        assert alg == "InsAllReduceMesh1DOneShot"
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, alg, ccl_bytes=4 << 20)
        for r in range(n):
            assert_same_bits(got[r], want[r], T.FP32, f"rank {r}")
    finally:
        w.close()


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("n,dtype,op,count", [(8, T.FP32, T.SUM, 70001), (20, T.FP32, T.MAX, 30011),
                                              (33, T.BFP16, T.SUM, 12345)])
def test_allreduce_in_place_every_template(stream, alg, n, dtype, op, count):
    """sendBuf == recvBuf on every rank, every template, planned from its closed form and fused into one pass (a
    destination is then exactly one source of its own fold) -- or, for the self-first orders among more than 16 ranks,
    staged."""
    rng = np.random.default_rng(n * 31 + count)
    xs = [payload(rng, dtype, count, "uniform" if dtype == T.FP32 else "normal") for _ in range(n)]
    ccl = SMALL_CCL if n <= 20 else T.CCL_BYTES_DEFAULT
    w = api.World(n, ccl_bytes=ccl)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        got, bufs = run_allreduce(w, stream, xs, count, dtype, op, in_place=True)
        info = w.last_info()
        assert info.fused == 1
        if dtype in (T.FP16, T.BFP16) and op == T.SUM:
            want = wide_oracle_allreduce(xs, count, dtype, alg, ccl)
        else:
            want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], alg, ccl_bytes=ccl)
        for r in range(n):
            assert_same_bits(got[r], want[r], dtype, f"{alg} n={n} rank {r}")
            assert bufs[r].guard_intact()
    finally:
        w.close()


def test_checked_world_verifies_then_launches(stream):
    """With the schedule check on, a collective is verified (no race, right semantics) and then runs as usual."""
    rng = np.random.default_rng(21)
    n, count = 8, 50001
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_check(True)
        for alg in ("InsAllReduceNHR", "InsAllReduceMesh1DTwoShotMeshChunk"):
            w.set_algorithm(api.CMD_ALLREDUCE, alg)
            got, _ = run_allreduce(w, stream, xs, count, T.FP32, T.SUM)
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0 and rep.steps > 0 and w.last_info().fused == 1
            want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, alg, ccl_bytes=SMALL_CCL)
            for r in range(n):
                assert_same_bits(got[r], want[r], T.FP32, f"{alg} rank {r}")
    finally:
        w.close()


@pytest.mark.parametrize("n,alg,dtype,op", [(24, "InsAllReduceMesh1DOneShot", T.FP32, T.SUM),
                                           (40, "InsAllReduceMesh1DOneShot", T.BFP16, T.SUM),
                                           (17, "InsAllReduceAicpuReduceNHR", T.FP64, T.PROD),
                                           (64, "InsAllReduceMesh1DOneShot", T.FP16, T.MAX)])
def test_one_shot_allreduce_in_place_among_many_ranks(stream, n, alg, dtype, op):
    """sendBuf == recvBuf with the per-rank orders of the one-shot template: among more than 16 ranks the outputs
    are computed sixteen at a time by different workgroups, so they go to a staging buffer and a second launch
    copies them over the inputs; repeated, on new data."""
    count = 30011
    rng = np.random.default_rng(n)
    esz = T.DTYPE_SIZE[dtype]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        for rep in range(2):
            kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
            xs = [payload(rng, dtype, count, kind) for _ in range(n)]
            got, bufs = run_allreduce(w, stream, xs, count, dtype, op, in_place=True)
            info = w.last_info()
            assert info.fused == 1 and info.launches == 2
            assert info.planCacheHit == 0   # new buffers: a plan with a staging buffer of its own is made for its addresses
            if dtype in (T.FP16, T.BFP16) and op == T.SUM:
                want = wide_oracle_allreduce(xs, count, dtype, alg, SMALL_CCL)
            else:
                want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=SMALL_CCL)
            for r in range(n):
                assert_same_bits(got[r], want[r], dtype, f"rep {rep} rank {r}")
                assert bufs[r].guard_intact()
    finally:
        w.close()


@pytest.mark.parametrize("n", [3, 9, 12, 20])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.MAX), (T.FP32, T.MIN), (T.BFP16, T.MIN), (T.FP64, T.MAX)])
def test_ring_max_min_keep_the_operand_order_in_one_pass(stream, n, dtype, op):
    """The ring hands the accumulated value on as the source operand (acc (+) x), and a floating-point MAX / MIN of
    signed zeros or NaNs depends on which operand comes first: the fused pass marks those steps and must give the
    bits of the step-by-step order, among any number of ranks."""
    rng = np.random.default_rng(n * 13 + dtype + op)
    count = 20011
    pool = np.array([0.0, -0.0, np.nan, 1.0, -1.0, np.inf, -np.inf, 0.5], dtype=np.float32)
    xs = []
    for _ in range(n):
        f = pool[rng.integers(0, pool.size, size=count)]
        xs.append(T.narrow16(f, dtype) if dtype == T.BFP16 else f.astype(T.NP_STORAGE[dtype]))
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceRing")
        got, bufs = run_allreduce(w, stream, xs, count, dtype, op)
        info = w.last_info()
        assert info.fused == 1 and info.launches == 1
        want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], "InsAllReduceRing",
                               ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(got[r], want[r], dtype, f"rank {r}")
            assert bufs[r].guard_intact()
    finally:
        w.close()


def test_step_by_step_plans_are_replayed_with_new_data(stream):
    """The step-by-step mode: the second identical call replays the per-level launches from the cache, on the data
    the buffers hold then."""
    n, count = 9, 40009
    for mode, alg, op in [(api.EXEC_STEP, "InsAllReduceRing", T.MAX), (api.EXEC_STEP, "InsAllReduceMesh1DTwoShot", T.SUM)]:
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            w.set_algorithm(api.CMD_ALLREDUCE, alg)
            rng = np.random.default_rng(3)
            send = [DevBuf(nbytes=count * 4) for _ in range(n)]
            recv = [DevBuf(nbytes=count * 4) for _ in range(n)]
            for rep in range(3):
                xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
                for r in range(n):
                    send[r].t[:count * 4] = torch.from_numpy(xs[r].view(np.uint8).copy()).to("cuda:0")
                torch.cuda.synchronize()
                for r in range(n):
                    assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, op, stream.cuda_stream) == 0
                stream.synchronize()
                info = w.last_info()
                assert info.fused == 0 and info.planCacheHit == (rep > 0) and info.launches >= info.levels > 1
                want = T.run_allreduce(T.NumericElems(T.FP32, op), xs, count, 4, alg, ccl_bytes=SMALL_CCL)
                for r in range(n):
                    assert_same_bits(recv[r].get(np.float32), want[r], T.FP32, f"{alg} rep {rep} rank {r}")
        finally:
            w.close()


def test_allreduce_default_selector_and_plan_cache(stream):
    """Config 1 of the baseline: AllReduce SUM fp32, 8 ranks x 1,048,576 elements, uniform[-1,1): the
    selector takes the one-shot mesh template at this size; the ring template is forced next."""
    rng = np.random.default_rng(11)
    n, count = 8, 1048576
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n)
    try:
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=count * 4) for _ in range(n)]
        torch.cuda.synchronize()
        for rep in range(2):
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            assert info.algName.decode() == "InsAllReduceMesh1DOneShot" and info.fused == 1
            assert info.planCacheHit == rep and info.launches == 1
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceMesh1DOneShot")
        for r in range(n):
            assert_same_bits(recv[r].get(np.float32), want[r], T.FP32, f"one-shot rank {r}")
        w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceRing")
        for r in range(n):
            assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().fused == 1 and w.last_info().planCacheHit == 0
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceRing")
        for r in range(n):
            assert_same_bits(recv[r].get(np.float32), want[r], T.FP32, f"ring rank {r}")
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg", list(T.REDUCE_SCATTER_TEMPLATES))
@pytest.mark.parametrize("dtype,op,n,rc", [(T.BFP16, T.SUM, 8, 65536 + 3), (T.FP32, T.SUM, 5, 30001),
                                          (T.INT64, T.MAX, 12, 10007), (T.FP16, T.SUM, 3, 50000)])
def test_reduce_scatter_both_templates_both_modes(stream, mode, alg, dtype, op, n, rc):
    rng = np.random.default_rng(rc)
    xs = [payload(rng, dtype, n * rc, "normal") for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=rc * T.DTYPE_SIZE[dtype]) for _ in range(n)]
        torch.cuda.synchronize()
        for r in range(n):
            assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, rc, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        esz = T.DTYPE_SIZE[dtype]
        if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), wide, rc, esz, alg, ccl_bytes=SMALL_CCL)]
        else:
            want = T.run_reduce_scatter(T.NumericElems(dtype, op), xs, rc, esz, alg, ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype, f"{alg} rank {r} fused={info.fused}")
            assert recv[r].guard_intact()
    finally:
        w.close()


@pytest.mark.parametrize("alg", ["InsAllReduceMesh1DTwoShot", "InsAllReduceMesh1DOneShot", "InsAllReduceRing",
                                 "InsAllReduceAicpuReduceNHR", "InsAllReduceNHR", "InsAllReduceRHD"])
@pytest.mark.parametrize("dtype,op,n,count", [(T.FP32, T.SUM, 24, 50021), (T.BFP16, T.SUM, 32, 70001),
                                             (T.INT32, T.MAX, 40, 30011), (T.FP64, T.PROD, 17, 20000),
                                             (T.FP16, T.SUM, 64, 66001)])
def test_allreduce_among_more_than_16_ranks(stream, alg, dtype, op, n, count):
    """Chains over more than 16 sources and the trees of the log-step templates (up to six levels) take the wide
    fold kernels and stay one pass."""
    rng = np.random.default_rng(n * 11 + count)
    kind = "prod" if op == T.PROD else "uniform" if dtype == T.FP32 else "normal"
    xs = [payload(rng, dtype, count, kind) for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        got, bufs = run_allreduce(w, stream, xs, count, dtype, op)
        info = w.last_info()
        assert info.fused == 1, alg
        if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
            want = wide_oracle_allreduce(xs, count, dtype, alg, SMALL_CCL)
        else:
            want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], alg, ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(got[r], want[r], dtype, f"{alg} rank {r} fused={info.fused}")
            assert bufs[r].guard_intact()
    finally:
        w.close()


@pytest.mark.parametrize("alg", ["InsReduceScatterMesh1D", "InsReduceScatterNHR", "InsReduceScatterAicpuReduceNHR"])
@pytest.mark.parametrize("dtype,op,n,rc", [(T.BFP16, T.SUM, 32, 9001), (T.FP32, T.SUM, 20, 12345), (T.INT8, T.MIN, 64, 5000)])
def test_reduce_scatter_among_more_than_16_ranks(stream, alg, dtype, op, n, rc):
    rng = np.random.default_rng(n + rc)
    xs = [payload(rng, dtype, n * rc, "normal") for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=rc * T.DTYPE_SIZE[dtype]) for _ in range(n)]
        torch.cuda.synchronize()
        for r in range(n):
            assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, rc, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        esz = T.DTYPE_SIZE[dtype]
        assert info.fused == 1, alg
        if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), wide, rc, esz, alg, ccl_bytes=SMALL_CCL)]
        else:
            want = T.run_reduce_scatter(T.NumericElems(dtype, op), xs, rc, esz, alg, ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype, f"{alg} rank {r} fused={info.fused}")
            assert recv[r].guard_intact()
    finally:
        w.close()


def test_reduce_scatter_order_preserved_at_40_ranks(stream):
    """The grouped variant for more than 32 ranks; its 40-leaf tree of six levels is one pass of the wide tree
    kernel."""
    n, rc, dtype = 40, 5003, T.FP32
    rng = np.random.default_rng(40)
    xs = [payload(rng, dtype, n * rc, "normal") for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_REDUCE_SCATTER, "ReduceScatterOrderPreservedGroup")
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=rc * 4) for _ in range(n)]
        torch.cuda.synchronize()
        for r in range(n):
            assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, rc, dtype, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().fused == 1
        want = T.run_reduce_scatter(T.NumericElems(dtype, T.SUM), xs, rc, 4, "ReduceScatterOrderPreservedGroup",
                                    ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(recv[r].get(np.float32), want[r], dtype, f"rank {r}")
            assert recv[r].guard_intact()
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype,op,counts", [
    (T.FP32, T.SUM, [100, 100, 100, 100, 100, 100, 100, 100, 500, 500]),       # reduce_scatter_v_testcase.cc:131-141
    (T.INT8, T.SUM, [700, 700, 600, 600, 500, 500, 400, 400, 300, 300, 200, 200, 100, 100]),   # :120-129
    (T.BFP16, T.SUM, [120001, 0, 7, 65536, 33333, 1, 250000, 4096]),
    (T.INT64, T.MIN, [30000, 5, 0, 70001]),
    (T.FP16, T.PROD, [50000, 20001, 3])])
def test_reduce_scatter_v_ragged(stream, mode, dtype, op, counts):
    """HcclReduceScatterV: ragged parts with gaps between them, zero-length parts, several executor loops."""
    n = len(counts)
    rng = np.random.default_rng(sum(counts))
    displs, off = [], 3
    for c in counts:
        displs.append(off)
        off += c + 5
    xs = [payload(rng, dtype, off, "prod" if op == T.PROD else "normal") for _ in range(n)]
    esz = T.DTYPE_SIZE[dtype]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=max(counts[r], 1) * esz) for r in range(n)]
        torch.cuda.synchronize()
        for r in range(n):
            assert w.reduce_scatter_v(r, send[r].ptr, counts, displs, recv[r].ptr, counts[r], dtype, op,
                                      stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        assert info.algName.decode() == "InsReduceScatterVMesh1D"
        assert info.fused == (1 if mode == api.EXEC_FUSED else 0)
        if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
            wide = [T.widen16(x, dtype) for x in xs]
            want = [T.narrow16(o, dtype) for o in
                    T.run_reduce_scatter_v(T.NumericElems(T.FP32, T.SUM), wide, counts, displs, esz, ccl_bytes=SMALL_CCL)]
        else:
            want = T.run_reduce_scatter_v(T.NumericElems(dtype, op), xs, counts, displs, esz, ccl_bytes=SMALL_CCL)
        for r in range(n):
            got = recv[r].get(T.NP_STORAGE[dtype])[:counts[r]]
            assert_same_bits(got, want[r], dtype, f"rank {r} fused={info.fused}")
            if counts[r]:
                assert recv[r].guard_intact()
            assert send[r].guard_intact()
    finally:
        w.close()


def test_reduce_scatter_bf16_within_one_ulp_of_fp32_accumulation(stream):
    """The tolerance the baseline states for 16-bit floats: every output within 1 bf16 ULP of the sum
    accumulated in fp32 (here: in float64, then compared on the bf16 grid)."""
    rng = np.random.default_rng(2)
    n, rc = 8, 1 << 16
    xs = [payload(rng, T.BFP16, n * rc, "normal") for _ in range(n)]
    w = api.World(n)
    try:
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=rc * 2) for _ in range(n)]
        torch.cuda.synchronize()
        for r in range(n):
            assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, rc, T.BFP16, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().algName.decode() == "InsReduceScatterMesh1D"
        exact = np.sum([T.widen16(x, T.BFP16).astype(np.float64) for x in xs], axis=0)
        for r in range(n):
            got = T.widen16(recv[r].get(np.uint16), T.BFP16).astype(np.float64)
            ref = exact[r * rc:(r + 1) * rc]
            ulp = np.maximum(np.abs(ref), 2.0 ** -126) * 2.0 ** -7      # spacing of bf16 at that magnitude
            assert np.all(np.abs(got - ref) <= ulp), f"rank {r}"         # tolerance: 1 bf16 ULP
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg", ["InsAllGatherMesh1D", "InsAllGatherNHR"])
def test_allgather(stream, mode, alg):
    rng = np.random.default_rng(4)
    for n, count in ((2, 5), (8, 70001), (12, 4097)):
        xs = [rng.integers(0, 65535, size=count, dtype=np.uint16) for _ in range(n)]
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            w.set_algorithm(api.CMD_ALLGATHER, alg)
            send = [DevBuf(x) for x in xs]
            recv = [DevBuf(nbytes=n * count * 2) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                assert w.all_gather(r, send[r].ptr, recv[r].ptr, count, T.FP16, stream.cuda_stream) == 0
            stream.synchronize()
            for r in range(n):
                assert np.array_equal(recv[r].get(np.uint16), np.concatenate(xs)) and recv[r].guard_intact()
        finally:
            w.close()


@pytest.mark.parametrize("mode", MODES)
def test_allgatherv_ragged(stream, mode):
    rng = np.random.default_rng(9)
    for counts in ([3, 0, 70001, 1, 4096, 0, 33, 12345], [0, 0, 9], list(rng.integers(0, 30000, 16))):
        counts = [int(c) for c in counts]
        n = len(counts)
        displs = [sum(counts[:i]) for i in range(n)]
        total = sum(counts)
        xs = [rng.integers(0, 65535, size=c, dtype=np.uint16) for c in counts]
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            send = [DevBuf(x) for x in xs]
            recv = [DevBuf(nbytes=total * 2) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                sp = send[r].ptr if counts[r] else None
                assert w.all_gather_v(r, sp, counts[r], recv[r].ptr, counts, displs, T.FP16, stream.cuda_stream) == 0
            stream.synchronize()
            for r in range(n):
                assert np.array_equal(recv[r].get(np.uint16), np.concatenate(xs)) and recv[r].guard_intact()
        finally:
            w.close()


def a2a_run(w, stream, m, dtype, npd, rng, kind="v"):
    n = len(m)
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    xs = [rng.integers(0, np.iinfo(npd).max, size=sum(m[i]), dtype=npd, endpoint=True) for i in range(n)]
    send = [DevBuf(x) for x in xs]
    recv = [DevBuf(nbytes=sum(x[2]) * np.dtype(npd).itemsize) for x in v]
    torch.cuda.synchronize()
    for r in range(n):
        sc, sd, rc, rd = v[r]
        sp = send[r].ptr if sum(sc) else None
        rp = recv[r].ptr if sum(rc) else None
        if kind == "v":
            assert w.all_to_all_v(r, sp, sc, sd, rp, rc, rd, dtype, stream.cuda_stream) == 0
        elif kind == "vc":
            assert w.all_to_all_vc(r, sp, [x for row in m for x in row], rp, dtype, stream.cuda_stream) == 0
        else:
            assert w.all_to_all(r, sp, m[0][0], rp, dtype, stream.cuda_stream) == 0
    stream.synchronize()
    want = T.run_alltoallv(xs, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                           [sum(x[2]) for x in v])
    for r in range(n):
        assert np.array_equal(recv[r].get(npd), want[r]), f"rank {r}"
        assert recv[r].guard_intact()


@pytest.mark.parametrize("mode", MODES)
def test_alltoall_family(stream, mode):
    rng = np.random.default_rng(21)
    for n in (2, 5, 8, 18):
        m = rng.integers(0, 3000, size=(n, n)).tolist()
        m[0][1] = 0
        if n == 8:
            m[2][6] = 120000          # larger than one scratch slot: the executor loops
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            a2a_run(w, stream, m, T.BFP16, np.uint16, rng, "v")
            a2a_run(w, stream, m, T.INT8, np.uint8, rng, "vc")
            a2a_run(w, stream, [[777] * n for _ in range(n)], T.FP32, np.uint32, rng, "uniform")
        finally:
            w.close()


def test_ranks_on_different_streams_and_threads():
    """One host thread and one stream per rank, blocking rendezvous: the reference's calling pattern."""
    n, count = 4, 50000
    rng = np.random.default_rng(8)
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n, ccl_bytes=4 << 20)
    try:
        w.set_blocking(True)
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=count * 4) for _ in range(n)]
        streams = [torch.cuda.Stream() for _ in range(n)]
        torch.cuda.synchronize()
        rcs = [None] * n

        def body(r):
            for _ in range(3):
                rcs[r] = w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, streams[r].cuda_stream)
            streams[r].synchronize()

        ts = [threading.Thread(target=body, args=(r,)) for r in range(n)]
        for t in ts:
            t.start()
        for t in ts:
            t.join(timeout=60)
        assert all(not t.is_alive() for t in ts) and rcs == [0] * n
        torch.cuda.synchronize()
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceMesh1DOneShot")
        for r in range(n):
            assert_same_bits(recv[r].get(np.float32), want[r], T.FP32, f"rank {r}")
    finally:
        w.close()


def test_plan_cache_keeps_a_thousand_shapes_and_retires_the_oldest(stream):
    """1100 different counts on one communicator (a training step has that many bucket sizes): the most recent
    1024 plans stay cached, older ones are retired without stalling the device, and a retired shape is simply
    planned again."""
    n = 2
    base = np.arange(1200, dtype=np.float32)
    xs = [base + 1, base * 2]
    w = api.World(n)
    try:
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=base.nbytes) for _ in range(n)]
        torch.cuda.synchronize()

        def run(count):
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
            return w.last_info().planCacheHit

        for count in range(1, 1101):
            assert run(count) == 0
        assert run(1100) == 1 and run(77) == 1          # the newest 1024 are counts 77 .. 1100
        assert run(76) == 0 and run(1) == 0             # retired; planned again
        assert run(500) == 1
        stream.synchronize()
        got = recv[0].get(np.float32)
        assert np.array_equal(got[:500], (xs[0] + xs[1])[:500])
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_a_communicator_of_one_rank(stream, mode):
    """Every collective among one rank is a copy of the input (or nothing, in place)."""
    count = 10007
    x = np.arange(count, dtype=np.float32) - 5000
    w = api.World(1, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        send = DevBuf(x)
        for call in ("all_reduce", "reduce_scatter", "all_gather", "all_to_all", "in_place"):
            recv = send if call == "in_place" else DevBuf(nbytes=x.nbytes)
            torch.cuda.synchronize()
            if call in ("all_reduce", "in_place"):
                rc = w.all_reduce(0, send.ptr, recv.ptr, count, T.FP32, T.SUM, stream.cuda_stream)
            elif call == "reduce_scatter":
                rc = w.reduce_scatter(0, send.ptr, recv.ptr, count, T.FP32, T.MAX, stream.cuda_stream)
            elif call == "all_gather":
                rc = w.all_gather(0, send.ptr, recv.ptr, count, T.FP32, stream.cuda_stream)
            else:
                rc = w.all_to_all(0, send.ptr, count, recv.ptr, T.FP32, stream.cuda_stream)
            assert rc == 0, call
            stream.synchronize()
            assert np.array_equal(recv.get(np.float32), x), call
            assert recv.guard_intact(), call
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
def test_alltoallv_same_buffers_new_tables_every_step(stream, mode):
    """An expert router changes the counts every step while the buffers stay where they are: the second call must
    move what ITS tables say (step plans are cached, and the tables are part of what they are cached under)."""
    n = 4
    rows = 3000
    rng = np.random.default_rng(33)
    xs = [rng.integers(0, 65535, size=rows, dtype=np.uint16) for _ in range(n)]
    send = [DevBuf(x) for x in xs]
    recv = [DevBuf(nbytes=2 * n * rows) for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        for step in range(3):
            # every rank sends all its rows each step, split differently: same extents, different blocks
            m = []
            for i in range(n):
                cut = np.sort(rng.integers(0, rows + 1, size=n - 1))
                m.append([int(c) for c in np.diff(np.concatenate([[0], cut, [rows]]))])
            v = [T.alltoallvc_to_v(m, r) for r in range(n)]
            for b in recv:
                b.t.fill_(0xA5)
            torch.cuda.synchronize()
            for r in range(n):
                sc, sd, rc, rd = v[r]
                assert w.all_to_all_v(r, send[r].ptr, sc, sd, recv[r].ptr, rc, rd, T.BFP16, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            assert bool(info.fused) == (mode == api.EXEC_FUSED)
            want = T.run_alltoallv(xs, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                                   [sum(x[2]) for x in v])
            for r in range(n):
                got = recv[r].get(np.uint16)[:len(want[r])]
                assert np.array_equal(got, want[r]), (mode, step, r)
    finally:
        w.close()


def test_ranks_on_different_streams_one_host_thread(stream):
    """One host thread issues every rank's call, each on that rank's own stream (the default, non-blocking
    rendezvous).  The collective enters every rank's stream when the LAST rank calls: what a stream holds before
    that moment (here: the kernels that produce the inputs) runs before it, what is enqueued afterwards (here: the
    consumers) runs after it."""
    n, count = 6, 200000
    w = api.World(n)
    try:
        streams = [torch.cuda.Stream() for _ in range(n)]
        base = [torch.arange(count, device="cuda:0", dtype=torch.float32) * (r + 1) for r in range(n)]
        send = [torch.zeros(count, device="cuda:0") for _ in range(n)]
        recv = [torch.zeros(count, device="cuda:0") for _ in range(n)]
        seen = [torch.zeros(count, device="cuda:0") for _ in range(n)]
        torch.cuda.synchronize()
        for it in range(1, 4):
            for r in range(n):
                with torch.cuda.stream(streams[r]):
                    for _ in range(20):                      # a producer that takes a while
                        send[r].copy_(base[r] * it)
                assert w.all_reduce(r, send[r].data_ptr(), recv[r].data_ptr(), count, T.FP32, T.SUM,
                                    streams[r].cuda_stream) == 0
            for r in range(n):                               # consumers, after every rank has called
                with torch.cuda.stream(streams[r]):
                    seen[r].copy_(recv[r])
            for s in streams:
                s.synchronize()
            want = torch.arange(count, device="cuda:0", dtype=torch.float32) * (it * n * (n + 1) // 2)
            for r in range(n):
                assert torch.equal(seen[r], want), (it, r)     # exact: small integers in fp32
    finally:
        w.close()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg,dtype,op,n,count", [("InsAllReduceMesh1DTwoShot", T.FP32, T.SUM, 8, 70003),
                                                  ("InsAllReduceRing", T.BFP16, T.SUM, 5, 40001),
                                                  ("InsAllReduceNHR", T.INT32, T.MAX, 12, 50021),
                                                  ("InsAllReduceAicpuReduceNHR", T.FP32, T.PROD, 12, 30011),
                                                  ("InsAllReduceMesh1DOneShot", T.FP16, T.SUM, 24, 9001),
                                                  ("InsAllReduceMesh1DTwoShotMeshChunk", T.FP32, T.SUM, 6, 60007)])
def test_a_plan_follows_its_collective_to_other_buffers(stream, mode, alg, dtype, op, n, count):
    """The same collective on buffers somewhere else (and differently aligned) is not planned again: the plan of the
    first call is moved there pointer by pointer, gets device tables of its own when the same buffers come a second
    time (large plans: at once), and is replayed from then on.  Every call's result is the oracle's.  Running in place is another shape."""
    rng = np.random.default_rng(count)
    esz = T.DTYPE_SIZE[dtype]
    kind = "prod" if op == T.PROD else "uniform" if dtype == T.FP32 else "normal"
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)

        def call(send, recv, xs):
            for r in range(n):
                send[r].t[send[r].offset:send[r].offset + send[r].nbytes] = torch.from_numpy(
                    xs[r].view(np.uint8).reshape(-1).copy()).to("cuda:0")
            torch.cuda.synchronize()
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            if info.fused and dtype in (T.FP16, T.BFP16) and op == T.SUM:
                want = wide_oracle_allreduce(xs, count, dtype, alg, SMALL_CCL)
            else:
                want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=SMALL_CCL)
            for r in range(n):
                assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want[r], dtype, f"{alg} rank {r}")
                assert recv[r].guard_intact()
            return info.planCacheHit, info.fused, info.launches

        def buffers(offsets):
            send = [DevBuf(nbytes=count * esz, offset=offsets[r % len(offsets)]) for r in range(n)]
            recv = [DevBuf(nbytes=count * esz, offset=offsets[(r + 1) % len(offsets)]) for r in range(n)]
            return send, recv

        first = buffers([0])
        second = buffers([esz, 0, 3 * esz, 128 + esz])   # other places, other alignments
        fresh = lambda: [payload(rng, dtype, count, kind) for _ in range(n)]
        hit0, fused0, launches0 = call(*first, fresh())
        assert hit0 == 0
        assert call(*second, fresh()) == (2, fused0, launches0)    # moved, launched from host tables
        again = call(*second, fresh())
        # moved once more, tables now in device memory -- or replayed already: a plan with more than 16 KiB of
        # segment lists gets its device tables the first time it is moved
        assert again in ((2, fused0, launches0), (1, fused0, launches0))
        assert call(*second, fresh()) == (1, fused0, launches0)    # replayed
        assert call(*first, fresh()) == (1, fused0, launches0)     # the first plan is still there
        hit, _, _ = call(first[0], first[0], fresh())              # in place: not the same collective
        assert hit == 0
        mixed = (first[0], second[1])                              # known buffers in a new combination
        assert call(*mixed, fresh())[0] == 2
    finally:
        w.close()


def test_overlapping_buffers_are_planned_for_their_addresses(stream):
    """When ranks' buffers overlap each other (here every rank receives into a slice of one allocation that is also a
    rank's input), what the plan may fuse depends on where they lie: such calls never borrow another call's plan."""
    n, count = 4, 4099
    rng = np.random.default_rng(5)
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=count * 4) for _ in range(n)]
        for r in range(n):
            assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().planCacheHit == 0
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, w.last_info().algName.decode(),
                               ccl_bytes=SMALL_CCL)
        # rank 1 now sends what rank 0 received: its input buffer is rank 0's old output, still apart from the rest
        xs2 = [xs[0], want[0], xs[2], xs[3]]
        send2 = [send[0], recv[0], send[2], send[3]]
        recv2 = [DevBuf(nbytes=count * 4) for _ in range(n)]
        for r in range(n):
            assert w.all_reduce(r, send2[r].ptr, recv2[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().planCacheHit == 2
        want2 = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs2, count, 4, w.last_info().algName.decode(),
                                ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(recv2[r].get(np.float32), want2[r], T.FP32, f"rank {r}")
        # two ranks share one input buffer: overlapping, so planned for these addresses
        send3 = [send[0], send[0], send[2], send[3]]
        xs3 = [xs[0], xs[0], xs[2], xs[3]]
        for r in range(n):
            assert w.all_reduce(r, send3[r].ptr, recv2[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        assert w.last_info().planCacheHit == 0
        want3 = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs3, count, 4, w.last_info().algName.decode(),
                                ccl_bytes=SMALL_CCL)
        for r in range(n):
            assert_same_bits(recv2[r].get(np.float32), want3[r], T.FP32, f"shared input, rank {r}")
    finally:
        w.close()


CLOSED_FORM_ALGS = {"all_reduce": "InsAllReduceMesh1DTwoShotMeshChunk", "reduce_scatter": "InsReduceScatterMesh1DMeshChunk",
                    "reduce_scatter_gather": "InsReduceScatterAicpuReduceNHR", "all_reduce_one_shot": "InsAllReduceMesh1DOneShot",
                    "all_reduce_two_shot": "InsAllReduceMesh1DTwoShot", "reduce_scatter_mesh": "InsReduceScatterMesh1D",
                    "all_reduce_gather": "InsAllReduceAicpuReduceNHR", "all_reduce_ring": "InsAllReduceRing",
                    "all_reduce_nhr": "InsAllReduceNHR", "reduce_scatter_nhr": "InsReduceScatterNHR",
                    "all_reduce_rhd": "InsAllReduceRHD", "reduce_scatter_ordered": "ReduceScatterOrderPreserved",
                    "reduce_scatter_ordered_group": "ReduceScatterOrderPreservedGroup"}


@pytest.mark.parametrize("kind,n,dtype,op,count", [("all_reduce", 64, T.FP32, T.SUM, 64 * 63 * 3 + 17),
                                                   ("all_reduce", 32, T.BFP16, T.SUM, 400003),
                                                   ("all_reduce", 12, T.INT32, T.MAX, 1 << 20),
                                                   ("reduce_scatter", 64, T.FP32, T.SUM, 5003),
                                                   ("reduce_scatter", 16, T.FP16, T.PROD, 70001),
                                                   ("reduce_scatter_gather", 12, T.FP64, T.PROD, 30011),
                                                   ("all_reduce_one_shot", 24, T.FP32, T.SUM, 100003),
                                                   ("all_reduce_one_shot", 8, T.FP16, T.MAX, 500001),
                                                   ("all_reduce_two_shot", 48, T.FP32, T.SUM, 300007),
                                                   ("all_reduce_two_shot", 8, T.BFP16, T.SUM, 1 << 21),
                                                   ("reduce_scatter_mesh", 32, T.FP32, T.SUM, 40009),
                                                   ("all_reduce_gather", 12, T.FP32, T.PROD, 200003),
                                                   ("all_reduce_gather", 40, T.INT64, T.SUM, 30011),
                                                   ("all_reduce_ring", 20, T.FP32, T.MAX, 150001),
                                                   ("all_reduce_ring", 8, T.BFP16, T.SUM, 1 << 20),
                                                   ("all_reduce_ring", 64, T.FP32, T.SUM, 37),
                                                   ("all_reduce_nhr", 24, T.FP32, T.SUM, 200003),
                                                   ("all_reduce_nhr", 33, T.BFP16, T.SUM, 70001),
                                                   ("all_reduce_nhr", 5, T.FP64, T.PROD, 1 << 18),
                                                   ("reduce_scatter_nhr", 12, T.FP32, T.MAX, 30011),
                                                   ("reduce_scatter_nhr", 64, T.FP16, T.MAX, 2003),
                                                   ("all_reduce_rhd", 12, T.FP32, T.SUM, 300007),
                                                   ("all_reduce_rhd", 48, T.BFP16, T.SUM, 90001),
                                                   ("all_reduce_rhd", 7, T.FP32, T.MIN, 1 << 19),
                                                   ("reduce_scatter_ordered", 12, T.FP32, T.SUM, 50021),
                                                   ("reduce_scatter_ordered_group", 40, T.FP32, T.SUM, 9001)])
def test_templates_planned_from_their_closed_form(stream, kind, n, dtype, op, count):
    """Templates that state their result in closed form are planned from it (nothing recorded) and run as one fused
    pass: the 64-rank mesh-chunk AllReduce too (4032 chains, eight launches of 512 segments).  The result is the oracle's replay of the template's
    steps, and the same collective with the closed form switched off (steps recorded and traced) gives the same bits."""
    alg = CLOSED_FORM_ALGS[kind]
    kind = "all_reduce" if kind.startswith("all_reduce") else "reduce_scatter"
    cmd = api.CMD_ALLREDUCE if kind == "all_reduce" else api.CMD_REDUCE_SCATTER
    rng = np.random.default_rng(n + count)
    esz = T.DTYPE_SIZE[dtype]
    ccl = 8 << 20
    kindof = "prod" if op == T.PROD else "uniform" if dtype == T.FP32 else "normal"
    send_count = count if kind == "all_reduce" else count * n
    xs = [payload(rng, dtype, send_count, kindof) for _ in range(n)]
    fused16 = dtype in (T.FP16, T.BFP16) and op == T.SUM
    if kind == "all_reduce":
        want = (wide_oracle_allreduce(xs, count, dtype, alg, ccl) if fused16 else
                T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=ccl))
    else:
        want = T.run_reduce_scatter(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=ccl)
    send = [DevBuf(x) for x in xs]
    results = []
    for closed_form in (1, 0):
        w = api.World(n, ccl_bytes=ccl)
        try:
            w.set_algorithm(cmd, alg)
            w.set_closed_form(closed_form)
            recv = [DevBuf(nbytes=count * esz) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                if kind == "all_reduce":
                    assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
                else:
                    assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            # kernels: a launch table holds 512 wide segments, so the 4032 chains of the 64-rank case take eight
            assert info.fused == 1 and info.launches <= 8, info.launches
            assert (info.levels == 0) == (closed_form == 1)
            got = [b.get(T.NP_STORAGE[dtype]) for b in recv]
            for r in range(n):
                assert_same_bits(got[r], want[r], dtype, f"{alg} rank {r} closed_form={closed_form}")
                assert recv[r].guard_intact()
            results.append(info.fusedSegments)
        finally:
            w.close()
    assert results[0] == results[1]


def test_a_schedule_that_cannot_be_fused_runs_its_steps(stream):
    """Rank 1 receives into the buffer rank 0 sends from, 64 bytes further on.  One pass over the inputs would overwrite
    what other workgroups still read, so the world falls back to the recorded steps (the two-shot template reads every
    input before it writes any output).  A world in FUSED mode has no scratch buffers until then: they are allocated
    now and the steps are recorded again against them.  (Exactly on top of rank 0's input it would still be one pass:
    every thread reads its elements before it writes them.)"""
    n, count, skew = 4, 50021, 64
    nbytes = count * 4
    rng = np.random.default_rng(77)
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    alg = "InsAllReduceMesh1DTwoShot"
    w = api.World(n, ccl_bytes=SMALL_CCL)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        send = [DevBuf(nbytes=nbytes + skew) for _ in range(n)]
        recv = [DevBuf(nbytes=nbytes) for _ in range(n)]

        def upload():
            for r in range(n):
                send[r].t[:nbytes] = torch.from_numpy(xs[r].view(np.uint8).copy()).to("cuda:0")
            torch.cuda.synchronize()

        def call(outs):
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, outs[r], count, T.FP32, T.SUM, stream.cuda_stream) == 0
            stream.synchronize()
            return w.last_info()

        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, alg, ccl_bytes=SMALL_CCL)
        upload()
        assert call([b.ptr for b in recv]).fused == 1      # the world has now run without scratch memory
        upload()
        info = call([recv[0].ptr, send[0].ptr, recv[2].ptr, recv[3].ptr])
        assert info.fused == 1 and info.launches == 1      # exactly on top: in place for that output
        assert_same_bits(send[0].get(np.uint8)[:nbytes].view(np.float32), want[1], T.FP32, "rank 1 on top of rank 0's input")
        for rep in range(2):
            upload()
            info = call([recv[0].ptr, send[0].ptr + skew, recv[2].ptr, recv[3].ptr])
            assert info.fused == 0 and info.launches >= info.levels > 1 and info.planCacheHit == rep
            got = [recv[0].get(np.float32), send[0].get(np.uint8)[skew:skew + nbytes].view(np.float32),
                   recv[2].get(np.float32), recv[3].get(np.float32)]
            for r in range(n):
                assert_same_bits(got[r], want[r], T.FP32, f"rank {r} rep {rep}")
            assert all(b.guard_intact() for b in recv + send)
    finally:
        w.close()
