"""The baseline's five configurations at their full sizes, through the HCCL entry points.

A dense CPU run of the oracle takes minutes at these sizes, so every case is checked two ways:
  * on the whole output against a plain torch computation that needs no knowledge of the schedule (a
    concatenation / permutation for the copies, an association-free max for integers, the rank-ordered fold
    in fp32 for the self-first templates);
  * bit for bit against the oracle's restatement of the template, followed on a sample of the element
    columns (oracle SampledElems: same executor chunks, slices and association order as the dense run).
"""
import numpy as np
import pytest
import torch

import bench
from oracle import templates as T
from hccl_amd import api, hcclx

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def stream():
    s = torch.cuda.Stream()
    yield s
    s.synchronize()


def sample_positions(rng, length, k, marks=()):
    """k random positions plus the first and last 70 and 8 either side of every mark (slice boundaries)."""
    parts = [rng.integers(0, length, k), np.arange(min(70, length)), np.arange(max(0, length - 70), length)]
    for m in marks:
        parts.append(np.arange(max(0, m - 8), min(length, m + 8)))
    return np.unique(np.concatenate(parts)).astype(np.int64)


def take(t, pos):
    return t[torch.from_numpy(pos).to(DEV)].cpu().numpy()


def uniform(n, seed, lo, hi):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return torch.rand(n, device=DEV, generator=g) * (hi - lo) + lo


# ---------------------------------------------------------------------------------------------------
# config 1: AllReduce SUM fp32, ring, 8 x 1,048,576 -- small enough for the dense oracle
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode", [api.EXEC_FUSED, api.EXEC_STEP])
def test_config1_allreduce_ring_fp32_8x1Mi(stream, mode):
    n, count = 8, 1048576
    xs = [uniform(count, 100 + k, -1.0, 1.0) for k in range(n)]
    outs = [torch.empty(count, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceRing")
        for r in range(n):
            assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        host = [x.cpu().numpy() for x in xs]
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), host, count, 4, "InsAllReduceRing")
        for r in range(n):
            assert np.array_equal(outs[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32)), r
    finally:
        w.close()


# ---------------------------------------------------------------------------------------------------
# config 2: ReduceScatter SUM bf16, mesh, 8 x 33,554,432 (64 MiB per rank)
# ---------------------------------------------------------------------------------------------------
def test_config2_reduce_scatter_bf16_8x64MiB(stream):
    n, rc = 8, 4 * 1024 * 1024
    g = torch.Generator(device=DEV)
    xs = []
    for k in range(n):
        g.manual_seed(200 + k)
        xs.append(torch.randn(n * rc, device=DEV, generator=g).to(torch.bfloat16))
    outs = [torch.zeros(rc, device=DEV, dtype=torch.bfloat16) for _ in range(n)]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        for r in range(n):
            assert w.reduce_scatter(r, xs[r].data_ptr(), outs[r].data_ptr(), rc, T.BFP16, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        assert info.algName.decode() == "InsReduceScatterMesh1D" and info.fused == 1 and info.launches == 1
        # whole output: own shard first, then ranks ascending, accumulated in fp32, one rounding to bf16
        for r in range(n):
            acc = xs[r][r * rc:(r + 1) * rc].float()
            for k in range(n):
                if k != r:
                    acc = xs[k][r * rc:(r + 1) * rc].float() + acc
            assert torch.equal(acc.to(torch.bfloat16).view(torch.int16), outs[r].view(torch.int16)), r
        # sampled columns against the oracle's template
        rng = np.random.default_rng(2)
        pos = sample_positions(rng, n * rc, 200000, marks=[k * rc for k in range(1, n)])
        e = T.SampledElems(T.FP32, T.SUM)
        ins = [e.sample(n * rc, pos, take(x, pos).astype(np.float32)) for x in [t.float() for t in xs]]
        want = T.run_reduce_scatter(e, ins, rc, 2, "InsReduceScatterMesh1D")
        for r in range(n):
            got = take(outs[r].view(torch.int16), want[r].pos).view(np.uint16)
            assert np.array_equal(got, T.narrow16(want[r].val, T.BFP16)), r
    finally:
        w.close()


# ---------------------------------------------------------------------------------------------------
# config 3: AllGatherV fp16, 16 ranks, counts uniform in [0, 8,388,608], arbitrary 16-bit patterns
# ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("tables", ["host", "device"])
def test_config3_allgatherv_fp16_16_ranks(stream, tables):
    n = 16
    rng = np.random.default_rng(3)
    counts = [int(c) for c in rng.integers(0, 8388608, size=n, endpoint=True)]
    counts[5] = 0                                   # a rank with nothing to send
    displs = [int(d) for d in np.concatenate([[0], np.cumsum(counts)[:-1]])]
    total = sum(counts)
    send = [torch.randint(-32768, 32767, (max(c, 1),), device=DEV, dtype=torch.int16) for c in counts]   # NaN/Inf patterns included
    recv = [torch.full((total + 16,), 0x5A5A, device=DEV, dtype=torch.int16) for _ in range(n)]
    torch.cuda.synchronize()
    if tables == "host":
        w = api.World(n)
        try:
            for r in range(n):
                assert w.all_gather_v(r, send[r].data_ptr(), counts[r], recv[r].data_ptr(), counts, displs, T.FP16,
                                      stream.cuda_stream) == 0
            stream.synchronize()
            assert w.last_info().algName.decode() == "InsAllGatherVMesh1D"
        finally:
            w.close()
    else:   # tables produced on the device: the kernel derives its tile map with a wavefront scan
        dc = torch.tensor(counts, dtype=torch.int64, device=DEV)
        dd = torch.tensor(displs, dtype=torch.int64, device=DEV)
        torch.cuda.synchronize()
        hcclx.allgatherv([t.data_ptr() for t in send], [t.data_ptr() for t in recv], dc.data_ptr(), dd.data_ptr(),
                         T.FP16, on_device=True, stream=stream.cuda_stream)
        stream.synchronize()
    whole = torch.cat([send[i][:counts[i]] for i in range(n)])
    for j in range(n):
        assert torch.equal(recv[j][:total], whole), j
        assert bool((recv[j][total:] == 0x5A5A).all()), j


# ---------------------------------------------------------------------------------------------------
# config 4: AlltoAllV bf16, MoE dispatch, 8 ranks x 4096 tokens x hidden 7168, Zipf(1.2) destinations
# ---------------------------------------------------------------------------------------------------
def test_config4_alltoallv_moe_dispatch():
    wl = bench.AllToAllV(torch, api, T)
    try:
        n = wl.n
        for t in wl.recv:
            t.fill_(0x1111)
        torch.cuda.synchronize()
        wl.step()
        wl.stream_obj.synchronize()
        assert sum(sum(wl.v[i][0]) for i in range(n)) == 8 * 4096 * 7168
        for i in range(n):
            sc, sd, _, _ = wl.v[i]
            for j in range(n):
                rd = wl.v[j][3][i]
                assert torch.equal(wl.recv[j][rd:rd + sc[j]], wl.send[i][sd[j]:sd[j] + sc[j]]), (i, j)
        assert wl.world.last_info().fused == 1
    finally:
        wl.world.close()


# ---------------------------------------------------------------------------------------------------
# config 5: AllReduce on 12 ranks, 4 KiB ... 1 GiB per rank in powers of 4
#   (i) int32 MAX through the NHR and RHD templates; (ii) fp32 PROD through the CPU-reduce NHR template
#   (per-rank order x_r, x_0, x_1, ...) and through RHD
# ---------------------------------------------------------------------------------------------------
SIZES = [4096 * 4 ** k for k in range(10)]          # bytes per rank


def run_ar12(stream, xs, outs, count, dtype, op, alg):
    n = len(xs)
    w = api.World(n)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        for r in range(n):
            assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        return w.last_info()
    finally:
        w.close()


def oracle_on_samples(xs, count, dtype, op, alg, rng, k):
    p2 = 8 if alg == "InsAllReduceRHD" else 12
    marks = [off for off, _ in T.split_data(min(count, 200 * 1024 * 1024 // 4), p2)][1:]
    pos = sample_positions(rng, count, k, marks=marks)
    e = T.SampledElems(dtype, op)
    ins = [e.sample(count, pos, take(x, pos)) for x in xs]
    return pos, T.run_allreduce(e, ins, count, 4, alg)


@pytest.mark.parametrize("nbytes", SIZES)
def test_config5_allreduce_12_ranks_int32_max(stream, nbytes):
    n, count = 12, nbytes // 4
    g = torch.Generator(device=DEV)
    xs = []
    for k in range(n):
        g.manual_seed(500 + k)
        xs.append(torch.randint(-2 ** 31, 2 ** 31 - 1, (count,), device=DEV, dtype=torch.int32, generator=g))
    best = xs[0]
    for k in range(1, n):
        best = torch.maximum(best, xs[k])          # integer max is association-free
    outs = [torch.empty(count, device=DEV, dtype=torch.int32) for _ in range(n)]
    for alg in ("InsAllReduceNHR", "InsAllReduceRHD"):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        info = run_ar12(stream, xs, outs, count, T.INT32, T.MAX, alg)
        assert info.fused == 1
        for r in range(n):
            assert torch.equal(outs[r], best), (alg, r)
    rng = np.random.default_rng(nbytes)
    pos, want = oracle_on_samples(xs, count, T.INT32, T.MAX, "InsAllReduceRHD", rng, 20000)
    for r in range(n):
        assert np.array_equal(take(outs[r], pos), want[r].val), r


@pytest.mark.parametrize("nbytes", SIZES)
def test_config5_allreduce_12_ranks_fp32_prod(stream, nbytes):
    n, count = 12, nbytes // 4
    xs = [uniform(count, 900 + k, 0.9, 1.1) for k in range(n)]
    outs = [torch.empty(count, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    # (a) the template the selector takes for PROD: gather by NHR, then fold x_r, x_0, x_1, ... on every rank
    info = run_ar12(stream, xs, outs, count, T.FP32, T.PROD, "InsAllReduceAicpuReduceNHR")
    assert info.fused == 1
    for r in range(n):
        acc = xs[r].clone()
        for k in range(n):
            if k != r:
                acc = xs[k] * acc
        assert torch.equal(acc.view(torch.int32), outs[r].view(torch.int32)), r
        del acc
    rng = np.random.default_rng(nbytes + 1)
    pos, want = oracle_on_samples(xs, count, T.FP32, T.PROD, "InsAllReduceAicpuReduceNHR", rng, 20000)
    for r in range(n):
        assert np.array_equal(take(outs[r], pos).view(np.uint32), want[r].val.view(np.uint32)), r
    # (b) halving-doubling: one tree per slice, the same bits on every rank
    info = run_ar12(stream, xs, outs, count, T.FP32, T.PROD, "InsAllReduceRHD")
    assert info.fused == 1
    for r in range(1, n):
        assert torch.equal(outs[r].view(torch.int32), outs[0].view(torch.int32)), r
    pos, want = oracle_on_samples(xs, count, T.FP32, T.PROD, "InsAllReduceRHD", rng, 20000)
    for r in range(n):
        assert np.array_equal(take(outs[r], pos).view(np.uint32), want[r].val.view(np.uint32)), r


# ---------------------------------------------------------------------------------------------------
# beyond the baseline's sizes: what the selector moves to for large messages (mesh-chunk templates)
# ---------------------------------------------------------------------------------------------------
def test_large_reduce_scatter_takes_the_chunked_mesh_template(stream):
    """bf16 shards of 32 MiB on 8 ranks (256 MiB per rank): above 16 MiB the selector picks the template that
    reduces in place chunk by chunk; every chunk of a shard has its own rotation of the ranks."""
    n, rc = 8, 16 * 1024 * 1024
    g = torch.Generator(device=DEV)
    xs = []
    for k in range(n):
        g.manual_seed(700 + k)
        xs.append(torch.randn(n * rc, device=DEV, generator=g).to(torch.bfloat16))
    outs = [torch.zeros(rc, device=DEV, dtype=torch.bfloat16) for _ in range(n)]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        for r in range(n):
            assert w.reduce_scatter(r, xs[r].data_ptr(), outs[r].data_ptr(), rc, T.BFP16, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        assert info.algName.decode() == "InsReduceScatterMesh1DMeshChunk" and info.fused == 1
        rng = np.random.default_rng(7)
        pos = sample_positions(rng, n * rc, 100000, marks=[k * rc for k in range(1, n)])
        e = T.SampledElems(T.FP32, T.SUM)
        ins = [e.sample(n * rc, pos, take(x.float(), pos)) for x in xs]
        want = T.run_reduce_scatter(e, ins, rc, 2, "InsReduceScatterMesh1DMeshChunk")
        for r in range(n):
            got = take(outs[r].view(torch.int16), want[r].pos).view(np.uint16)
            assert np.array_equal(got, T.narrow16(want[r].val, T.BFP16)), r
        # any order gives the same value up to rounding: within 1 bf16 ULP of the float64 sum on rank 0's shard
        exact = sum(x[:rc].double() for x in xs)
        err = (outs[0].double() - exact).abs()
        ulp = torch.clamp(exact.abs(), min=2.0 ** -126) * 2.0 ** -7
        assert bool((err <= ulp).all())
    finally:
        w.close()


def test_large_allreduce_takes_the_chunked_two_shot_template(stream):
    n, count = 8, 64 * 1024 * 1024 + 5            # 256 MiB + 20 bytes of fp32 per rank
    xs = [uniform(count, 800 + k, -1.0, 1.0) for k in range(n)]
    outs = [torch.empty(count, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        for r in range(n):
            assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        assert info.algName.decode() == "InsAllReduceMesh1DTwoShotMeshChunk" and info.fused == 1
        for r in range(1, n):
            assert torch.equal(outs[r].view(torch.int32), outs[0].view(torch.int32)), r
        rng = np.random.default_rng(8)
        pos = sample_positions(rng, count, 100000)
        e = T.SampledElems(T.FP32, T.SUM)
        want = T.run_allreduce(e, [e.sample(count, pos, take(x, pos)) for x in xs], count, 4,
                               "InsAllReduceMesh1DTwoShotMeshChunk")
        for r in range(n):
            assert np.array_equal(take(outs[r], pos).view(np.uint32), want[r].val.view(np.uint32)), r
    finally:
        w.close()


@pytest.mark.parametrize("n,alg,dtype,op", [(32, "InsAllReduceMesh1DTwoShot", T.FP32, T.SUM),     # wide chain kernel
                                           (32, "InsAllReduceNHR", T.FP32, T.SUM),              # wide tree kernel
                                           (64, "InsAllReduceRHD", T.FP32, T.PROD),
                                           (40, "InsAllReduceNHR", T.INT32, T.MAX)])
def test_allreduce_among_many_ranks_at_16MiB_per_rank(stream, n, alg, dtype, op):
    """Communicators of more than 16 ranks at a size where the kernels run in their full-tile paths: all ranks
    agree bit for bit, and 50,000 sampled columns equal the oracle's run of the same template."""
    count = 4 * 1024 * 1024 + 3
    if dtype == T.INT32:
        xs = [torch.randint(-2**31, 2**31 - 1, (count,), device=DEV, dtype=torch.int32) for _ in range(n)]
    elif op == T.PROD:
        xs = [uniform(count, 900 + k, 0.97, 1.03) for k in range(n)]
    else:
        xs = [uniform(count, 900 + k, -1.0, 1.0) for k in range(n)]
    outs = [torch.empty_like(x) for x in xs]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        for r in range(n):
            assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        assert info.fused == 1 and info.launches == 2, info.launches   # two kernels: the fold, then the fan-out copy
        for r in range(1, n):
            assert torch.equal(outs[r].view(torch.int32), outs[0].view(torch.int32)), r
        rng = np.random.default_rng(n)
        pos = sample_positions(rng, count, 50000, marks=[off for off, _ in T.split_data(count, n)][1:])
        e = T.SampledElems(dtype, op)
        want = T.run_allreduce(e, [e.sample(count, pos, take(x, pos)) for x in xs], count, 4, alg)
        for r in (0, n // 2, n - 1):
            assert np.array_equal(take(outs[r], pos).view(np.uint32), want[r].val.view(np.uint32)), r
    finally:
        w.close()
