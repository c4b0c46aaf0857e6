"""The (topology, dtype, op, count) tuples of the reference's own AllReduce and ReduceScatter system tests
(test/st/algorithm/testcase/all_reduce_testcase.cc:119-301, reduce_scatter_aicpu_testcase.cc:117-387), at their
full sizes, through the HCCL entry points and the default selector.  The reference checks these cases
symbolically; here the payload is moved on the GPU and compared bit for bit with the oracle's restatement of
the template the selector picked, followed on a sample of the element columns (same executor chunks, slices and
association order as a dense run)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api
from gpu_util import device_payload, host_sample, sample_positions, fused_is_wide

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "st_cases.json")))
DT = {"int8": T.INT8, "int16": T.INT16, "int32": T.INT32, "fp16": T.FP16, "fp32": T.FP32, "bfp16": T.BFP16}
OP = {"sum": T.SUM, "max": T.MAX, "min": T.MIN}


@pytest.fixture(scope="module")
def stream():
    s = torch.cuda.Stream()
    yield s
    s.synchronize()


def oracle_inputs(xs, pos, dtype, op, length):
    """Sampled inputs for the oracle: 16-bit float SUM is accumulated in fp32 by a fused fold, everything else in
    its own type."""
    wide = fused_is_wide(dtype, op)
    e = T.SampledElems(T.FP32 if wide else dtype, op)
    ins = []
    for x in xs:
        v = host_sample(x, pos, dtype)
        ins.append(e.sample(length, pos, T.widen16(v, dtype) if wide else v))
    return e, ins, wide


def check(outs, want, dtype, wide, what):
    for r, o in enumerate(outs):
        got = host_sample(o, want[r].pos, dtype)
        exp = T.narrow16(want[r].val, dtype) if wide else want[r].val
        assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(exp).view(np.uint8)), (what, r)


@pytest.mark.parametrize("case", GOLD["allreduce_st"]["cases"], ids=lambda c: c["name"])
def test_allreduce_system_test_case(stream, case):
    n, count, dtype, op = case["ranks"], case["count"], DT[case["dtype"]], OP[case["op"]]
    esz = T.DTYPE_SIZE[dtype]
    xs = [device_payload(dtype, count, 7000 + 31 * k) for k in range(n)]
    outs = [torch.zeros_like(x) for x in xs]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        for r in range(n):
            assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        alg = info.algName.decode()
        nbytes = count * esz
        # the selector's thresholds (all_reduce_auto_selector.cc:483-489, ratio = 8 / N^2 for N ranks)
        if nbytes <= 8 * 1024 * 1024:
            assert alg == "InsAllReduceMesh1DOneShot"
        elif nbytes * (8.0 / n / n) > 32 * 1024 * 1024:
            assert alg == "InsAllReduceMesh1DTwoShotMeshChunk"
        else:
            assert alg == "InsAllReduceMesh1DTwoShot"
        assert info.fused == 1, alg
        rng = np.random.default_rng(count % 9973)
        per = -(-count // n)
        pos = sample_positions(rng, count, 40000, marks=[k * per for k in range(1, n) if k * per < count])
        e, ins, wide = oracle_inputs(xs, pos, dtype, op, count)
        want = T.run_allreduce(e, ins, count, esz, alg)
        check(outs, want, dtype, wide, case["name"])
    finally:
        w.close()


@pytest.mark.parametrize("case", GOLD["reducescatter_st"]["cases"], ids=lambda c: c["name"])
def test_reduce_scatter_system_test_case(stream, case):
    servers = case["servers"]
    n, rc, dtype, op = sum(servers), case["recv_count"], DT[case["dtype"]], OP[case["op"]]
    esz = T.DTYPE_SIZE[dtype]
    xs = [device_payload(dtype, n * rc, 9000 + 17 * k) for k in range(n)]
    outs = [torch.zeros(rc, device="cuda:0", dtype=x.dtype) for x in xs]
    torch.cuda.synchronize()
    w = api.World(n)
    try:
        if len(servers) > 1:
            w.set_topo(levels=2, shape=api.SHAPE_MESH_1D,
                       devices_per_server=servers[0] if len(set(servers)) == 1 else 0)
        for r in range(n):
            assert w.reduce_scatter(r, xs[r].data_ptr(), outs[r].data_ptr(), rc, dtype, op, stream.cuda_stream) == 0
        stream.synchronize()
        info = w.last_info()
        alg = info.algName.decode()
        if len(servers) > 1:
            assert alg == "InsReduceScatterNHR"
        elif rc * esz * (8.0 / n) ** 2 > 16 * 1024 * 1024:      # reduce_scatter_auto_selector.cc:383-408
            assert alg == "InsReduceScatterMesh1DMeshChunk"
        else:
            assert alg == "InsReduceScatterMesh1D"
        assert info.fused == 1, alg
        rng = np.random.default_rng(rc % 9973 + n)
        pos = sample_positions(rng, n * rc, 40000, marks=[k * rc for k in range(1, n)])
        e, ins, wide = oracle_inputs(xs, pos, dtype, op, n * rc)
        want = T.run_reduce_scatter(e, ins, rc, esz, alg)
        check(outs, want, dtype, wide, case["name"])
    finally:
        w.close()
        del xs, outs
        torch.cuda.empty_cache()
