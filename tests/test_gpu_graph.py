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
