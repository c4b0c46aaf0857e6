"""A warm collective is a handful of kernel launches with no allocation and no copy, so a caller can capture it
into a HIP graph: replays must give what the eager call gives, on the data the buffers hold at replay time."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api

from gpu_util import DevBuf, assert_same_bits, payload

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,count,dtype,op,alg,mode", [
    (8, 4099, T.FP32, T.SUM, "InsAllReduceMesh1DOneShot", api.EXEC_FUSED),
    (12, 70001, T.INT32, T.MAX, "InsAllReduceRHD", api.EXEC_FUSED),
    (32, 20001, T.FP32, T.SUM, "InsAllReduceNHR", api.EXEC_FUSED),          # the wide tree kernel
    (6, 30011, T.FP32, T.SUM, "InsAllReduceRing", api.EXEC_STEP)])          # per-level launches from cached plans
def test_warm_allreduce_captured_into_a_graph_and_replayed(n, count, dtype, op, alg, mode):
    rng = np.random.default_rng(n + count)
    npd = T.NP_STORAGE[dtype]
    nbytes = count * T.DTYPE_SIZE[dtype]
    w = api.World(n)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        send = [DevBuf(nbytes=nbytes) for _ in range(n)]
        recv = [DevBuf(nbytes=nbytes) for _ in range(n)]
        s = torch.cuda.Stream()

        def upload():
            xs = [payload(rng, dtype, count, "uniform" if dtype == T.FP32 else "normal") for _ in range(n)]
            for r in range(n):
                send[r].t[:nbytes] = torch.from_numpy(xs[r].view(np.uint8).copy()).to("cuda:0")
            torch.cuda.synchronize()
            return xs

        def issue():
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, s.cuda_stream) == 0

        upload()
        issue()                      # builds and caches the plan (allocates: not capturable)
        s.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            g.capture_begin()
            issue()
            g.capture_end()
        assert w.last_info().planCacheHit == 1
        for rep in range(3):
            xs = upload()            # eager work and a synchronisation between the replays
            for r in range(n):
                recv[r].t.fill_(0xA5)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], alg)
            for r in range(n):
                assert_same_bits(recv[r].get(npd), want[r], dtype, f"replay {rep} rank {r}")
                assert recv[r].guard_intact()
    finally:
        w.close()


def test_a_launch_that_uploads_its_tables_refuses_to_be_captured():
    """A one-shot launch copies its table through a ring of pinned slots that later calls reuse; captured, the copy
    would read a stale slot at every replay.  It must fail loudly instead, and leave the capture usable."""
    from hccl_amd import hcclx
    from hccl_amd._lib import HcclError
    x = np.arange(5000, dtype=np.float32)
    src, dst = DevBuf(x), DevBuf(nbytes=x.nbytes)
    s = torch.cuda.Stream()
    hcclx.fold([(x.size, [src.ptr], [dst.ptr])], T.FP32, stream=s.cuda_stream)    # eagerly: fine
    s.synchronize()
    assert np.array_equal(dst.get(np.float32), x)
    plan = hcclx.Plan([(x.size, [src.ptr], [dst.ptr])], T.FP32)
    dst.t[dst.offset:dst.offset + dst.nbytes] = 0
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        g.capture_begin()
        with pytest.raises(HcclError):
            hcclx.fold([(x.size, [src.ptr], [dst.ptr])], T.FP32, stream=s.cuda_stream)
        plan.launch(s.cuda_stream)                                                 # the capturable form
        g.capture_end()
    g.replay()
    torch.cuda.synchronize()
    assert np.array_equal(dst.get(np.float32), x) and dst.guard_intact()
    del g
    plan.close()


def test_data_movement_collectives_captured_from_their_first_call():
    """AllGatherV and AlltoAllV among 8 ranks carry their tables in the kernel arguments: they can be captured without
    a warm-up, and a replay moves what the buffers hold then."""
    n = 8
    rng = np.random.default_rng(5)
    counts = [int(c) for c in rng.integers(0, 3000, size=n)]
    displs = [int(d) for d in np.concatenate([[0], np.cumsum(counts)[:-1]])]
    total = sum(counts)
    m = rng.integers(0, 900, size=(n, n)).tolist()
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    ag_in = [DevBuf(nbytes=max(counts) * 2) for _ in range(n)]
    ag_out = [DevBuf(nbytes=total * 2) for _ in range(n)]
    aa_in = [DevBuf(nbytes=max(1, sum(m[i])) * 2) for i in range(n)]
    aa_out = [DevBuf(nbytes=max(1, sum(x[2])) * 2) for x in v]
    s = torch.cuda.Stream()
    w1, w2 = api.World(n), api.World(n)
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            g.capture_begin()
            for r in range(n):
                assert w1.all_gather_v(r, ag_in[r].ptr, counts[r], ag_out[r].ptr, counts, displs, T.FP16, s.cuda_stream) == 0
            for r in range(n):
                sc, sd, rc, rd = v[r]
                assert w2.all_to_all_v(r, aa_in[r].ptr, sc, sd, aa_out[r].ptr, rc, rd, T.BFP16, s.cuda_stream) == 0
            g.capture_end()
        for rep in range(2):
            xs = [rng.integers(0, 65536, size=max(counts), dtype=np.uint16) for _ in range(n)]
            ys = [rng.integers(0, 65536, size=max(1, sum(m[i])), dtype=np.uint16) for i in range(n)]
            for r in range(n):
                ag_in[r].t[ag_in[r].offset:ag_in[r].offset + xs[r].nbytes] = torch.from_numpy(xs[r].view(np.uint8).copy()).to("cuda:0")
                aa_in[r].t[aa_in[r].offset:aa_in[r].offset + ys[r].nbytes] = torch.from_numpy(ys[r].view(np.uint8).copy()).to("cuda:0")
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            want = T.run_allgatherv(xs, counts, displs, total, 0)
            for r in range(n):
                assert np.array_equal(ag_out[r].get(np.uint16)[:total], want[r]), f"AllGatherV replay {rep} rank {r}"
                assert ag_out[r].guard_intact()
            want = T.run_alltoallv([y[:sum(m[i])] for i, y in enumerate(ys)], [x[0] for x in v], [x[1] for x in v],
                                   [x[2] for x in v], [x[3] for x in v], [sum(x[2]) for x in v])
            for r in range(n):
                assert np.array_equal(aa_out[r].get(np.uint16)[:sum(v[r][2])], want[r]), f"AlltoAllV replay {rep} rank {r}"
                assert aa_out[r].guard_intact()
        del g
    finally:
        w1.close()
        w2.close()


def test_a_collective_without_a_plan_for_its_buffers_refuses_to_be_captured():
    """Planning a collective, or moving a known plan to other buffers, allocates tables or sends them through the
    pinned ring.  On a capturing stream such a call must say so (HCCL_E_NOT_SUPPORT) before it touches the GPU, and
    leave the capture usable for the collectives that are warm."""
    n, count = 8, 6007
    rng = np.random.default_rng(9)
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(n)]
    w = api.World(n)
    try:
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=count * 4) for _ in range(n)]
        other = [DevBuf(nbytes=count * 4) for _ in range(n)]
        s = torch.cuda.Stream()

        def issue(dst, cnt=count):
            return [w.all_reduce(r, send[r].ptr, dst[r].ptr, cnt, T.FP32, T.SUM, s.cuda_stream) for r in range(n)]

        assert issue(recv) == [0] * n            # warm for (send, recv)
        s.synchronize()
        alg = w.last_info().algName.decode()
        for r in range(n):
            recv[r].t.fill_(0xA5)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            g.capture_begin()
            assert issue(other) == [0] * (n - 1) + [5]          # known shape, other buffers: would use the ring
            assert issue(recv, count - 1) == [0] * (n - 1) + [5]   # unknown shape: would plan and allocate
            assert issue(recv) == [0] * n                       # warm: kernels only
            g.capture_end()
        assert w.last_info().planCacheHit == 1
        g.replay()
        torch.cuda.synchronize()
        want = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, alg)
        for r in range(n):
            assert_same_bits(recv[r].get(np.float32), want[r], T.FP32, f"rank {r}")
            assert recv[r].guard_intact() and other[r].guard_intact()
            assert (other[r].t == 0xA5).all()
        del g
    finally:
        w.close()
