"""GPU runs of what tests/test_host_verbs.py checks symbolically: the read mode of the NHR and AlltoAllV templates
(PCIe links: the receiver fetches) against the oracle and against write mode, in both execution modes, and the
plug-in templates that collect with the one-sided reduce verbs against a plain left fold."""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api, _lib

from gpu_util import DevBuf, assert_same_bits, payload

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SMALL_CCL = 1024 * 1024 + 64 * 1024
MODES = [api.EXEC_FUSED, api.EXEC_STEP]
LINKS = [api.LINK_HCCS, api.LINK_PCIE]
PLUGIN = os.path.join(ROOT, "hccl_amd", "lib", "libhccl_one_sided_templates.so")


@pytest.fixture(scope="module")
def stream():
    s = torch.cuda.Stream()
    yield s
    s.synchronize()


@pytest.fixture(scope="module")
def plugin():
    assert os.path.exists(PLUGIN), "build the library first (make -C hccl_amd/csrc): the plug-in example is part of it"
    _lib.load()
    return ctypes.CDLL(PLUGIN, mode=ctypes.RTLD_GLOBAL)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("n,dtype,op,count", [(5, T.FP32, T.SUM, 70001), (12, T.FP32, T.SUM, 100003),
                                              (12, T.INT32, T.MAX, 40009), (8, T.BFP16, T.SUM, 50001)])
def test_nhr_allreduce_read_mode_equals_write_mode_and_the_oracle(stream, mode, n, dtype, op, count):
    rng = np.random.default_rng(n + count)
    xs = [payload(rng, dtype, count, "uniform" if dtype == T.FP32 else "normal") for _ in range(n)]
    send = [DevBuf(x) for x in xs]
    results = []
    for link in LINKS:
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            w.set_link_protocol(link)
            w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceNHR")
            recv = [DevBuf(nbytes=xs[0].nbytes) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            assert info.fused == (1 if mode == api.EXEC_FUSED else 0)
            results.append([b.get(T.NP_STORAGE[dtype]) for b in recv])
            assert all(b.guard_intact() for b in recv)
        finally:
            w.close()
    if mode == api.EXEC_FUSED and dtype == T.BFP16:
        wide = [T.widen16(x, dtype) for x in xs]
        want = [T.narrow16(o, dtype) for o in T.run_allreduce(T.NumericElems(T.FP32, T.SUM), wide, count, 2,
                                                              "InsAllReduceNHR", ccl_bytes=SMALL_CCL)]
    else:
        want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], "InsAllReduceNHR",
                               ccl_bytes=SMALL_CCL)
    for r in range(n):
        assert_same_bits(results[0][r], want[r], dtype, f"write mode rank {r}")
        assert_same_bits(results[1][r], want[r], dtype, f"read mode rank {r}")


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg", ["InsReduceScatterNHR", "InsReduceScatterAicpuReduceNHR"])
def test_nhr_reduce_scatter_read_mode(stream, mode, alg):
    n, recv_count, dtype, op = 12, 20011, T.FP32, T.PROD
    rng = np.random.default_rng(recv_count)
    xs = [payload(rng, dtype, n * recv_count, "prod") for _ in range(n)]
    want = T.run_reduce_scatter(T.NumericElems(dtype, op), xs, recv_count, 4, alg, ccl_bytes=SMALL_CCL)
    send = [DevBuf(x) for x in xs]
    for link in LINKS:
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            w.set_link_protocol(link)
            w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
            recv = [DevBuf(nbytes=recv_count * 4) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                assert w.reduce_scatter(r, send[r].ptr, recv[r].ptr, recv_count, dtype, op, stream.cuda_stream) == 0
            stream.synchronize()
            for r in range(n):
                assert_same_bits(recv[r].get(np.float32), want[r], dtype, f"{alg} link {link} rank {r}")
                assert recv[r].guard_intact()
        finally:
            w.close()


def test_data_movement_templates_in_read_mode_step_by_step(stream):
    """AllGather NHR and AlltoAllV through their templates (STEP mode), PCIe links: the peers' scratch slots are
    fetched instead of written; 20 ranks take two rounds of AlltoAllV peers."""
    for n in (6, 20):
        rng = np.random.default_rng(n)
        count = 30011
        xs = [rng.integers(0, 65535, size=count, dtype=np.uint16) for _ in range(n)]
        m = rng.integers(0, 3000, size=(n, n))
        m[0, n - 1] = 0
        m[1, 0] = 0
        m[0, 1] = 0
        m = m.tolist()
        v = [T.alltoallvc_to_v(m, r) for r in range(n)]
        ys = [rng.integers(0, 65535, size=max(1, sum(m[i])), dtype=np.uint16) for i in range(n)]
        want = T.run_alltoallv(ys, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                               [max(1, sum(x[2])) for x in v], fill=0xA5A5)
        for link in LINKS:
            w = api.World(n, ccl_bytes=SMALL_CCL)
            try:
                w.set_mode(api.EXEC_STEP)
                w.set_link_protocol(link)
                w.set_algorithm(api.CMD_ALLGATHER, "InsAllGatherNHR")
                send = [DevBuf(x) for x in xs]
                recv = [DevBuf(nbytes=n * count * 2) for _ in range(n)]
                torch.cuda.synchronize()
                for r in range(n):
                    assert w.all_gather(r, send[r].ptr, recv[r].ptr, count, T.FP16, stream.cuda_stream) == 0
                stream.synchronize()
                assert w.last_info().fused == 0
                for r in range(n):
                    assert np.array_equal(recv[r].get(np.uint16), np.concatenate(xs)), (n, link, r)
                    assert recv[r].guard_intact()
                send = [DevBuf(y) for y in ys]
                recv = [DevBuf(np.full(max(1, sum(x[2])), 0xA5A5, dtype=np.uint16)) for x in v]
                torch.cuda.synchronize()
                for r in range(n):
                    sc, sd, rc, rd = v[r]
                    assert w.all_to_all_v(r, send[r].ptr, sc, sd, recv[r].ptr, rc, rd, T.BFP16, stream.cuda_stream) == 0
                stream.synchronize()
                assert w.last_info().fused == 0
                for r in range(n):
                    assert np.array_equal(recv[r].get(np.uint16), want[r]), (n, link, r)
                    assert recv[r].guard_intact()
            finally:
                w.close()


def left_fold(xs, dtype, op):
    """x_{n-1} (+) (... (x_1 (+) x_0)) with the oracle's pairwise element op."""
    acc = xs[0].copy()
    e = T.NumericElems(dtype, op)
    for x in xs[1:]:
        e.reduce(acc, 0, x, 0, acc.size)
    return acc


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("alg", ["ExampleAllReduceReadReduce", "ExampleAllReduceBatchReadReduce",
                                 "ExampleAllReduceWriteReduce", "ExampleAllReduceBatchWriteReduce",
                                 "ExampleAllReduceReadThenAicpuReduce"])
def test_plug_in_templates_on_the_one_sided_reduce_verbs(stream, plugin, mode, alg):
    for n, dtype, op, count in ((5, T.FP32, T.SUM, 60001), (3, T.FP32, T.PROD, 300007), (8, T.INT32, T.MAX, 9001)):
        rng = np.random.default_rng(n + count)
        kind = "prod" if op == T.PROD else "uniform"
        xs = [payload(rng, dtype, count, kind) for _ in range(n)]
        want = left_fold(xs, dtype, op)
        w = api.World(n, ccl_bytes=SMALL_CCL)
        try:
            w.set_mode(mode)
            w.set_algorithm(api.CMD_ALLREDUCE, alg)
            send = [DevBuf(x) for x in xs]
            recv = [DevBuf(nbytes=xs[0].nbytes) for _ in range(n)]
            torch.cuda.synchronize()
            for r in range(n):
                assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, dtype, op, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            assert info.algName.decode() == alg and info.fused == (1 if mode == api.EXEC_FUSED else 0)
            for r in range(n):
                assert_same_bits(recv[r].get(T.NP_STORAGE[dtype]), want, dtype, f"{alg} n={n} rank {r}")
                assert recv[r].guard_intact()
        finally:
            w.close()


@pytest.mark.parametrize("mode", MODES)
def test_plug_in_pair_template_on_the_two_sided_batch_read_reduce(stream, plugin, mode):
    rng = np.random.default_rng(2)
    count = 100003
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(2)]
    w = api.World(2, ccl_bytes=SMALL_CCL)
    try:
        w.set_mode(mode)
        w.set_algorithm(api.CMD_ALLREDUCE, "ExampleAllReducePairReadsEachOther")
        send = [DevBuf(x) for x in xs]
        recv = [DevBuf(nbytes=count * 4) for _ in range(2)]
        torch.cuda.synchronize()
        for r in range(2):
            assert w.all_reduce(r, send[r].ptr, recv[r].ptr, count, T.FP32, T.SUM, stream.cuda_stream) == 0
        stream.synchronize()
        for r in range(2):
            assert_same_bits(recv[r].get(np.float32), left_fold([xs[r], xs[1 - r]], T.FP32, T.SUM), T.FP32, f"rank {r}")
    finally:
        w.close()
