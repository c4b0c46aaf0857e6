"""hcclx_fold_static, the entry point that allocates nothing, against hcclx_fold: same segments, same bits.  Two
calls in a row share the library's one fixed launch table; the second is smaller than the first."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import hcclx
from hccl_amd._lib import HcclError

from gpu_util import DevBuf, payload

pytestmark = pytest.mark.gpu


def run_both(cases, dtype, op, mode, stream):
    """cases: list of (count, sources as numpy arrays, number of destinations[, tree program]).  Returns the
    outputs of hcclx_fold and of hcclx_fold_static, per case and destination."""
    npd = T.NP_STORAGE[dtype]
    esz = T.DTYPE_SIZE[dtype]
    srcs = [[DevBuf(x, offset=(k % 2) * esz) for k, x in enumerate(c[1])] for c in cases]
    out = []
    for fn in (hcclx.fold, hcclx.fold_static):
        dsts = [[DevBuf(nbytes=c[0] * esz, offset=(1 + d) * esz) for d in range(c[2])] for c in cases]
        segs = []
        for c, ss, dd in zip(cases, srcs, dsts):
            seg = [c[0], [s.ptr for s in ss], [d.ptr for d in dd]]
            if len(c) > 3:
                seg.append(c[3])
            segs.append(tuple(seg))
        fn(segs, dtype, op, mode, stream=stream.cuda_stream)
        stream.synchronize()
        assert all(d.guard_intact() for dd in dsts for d in dd)
        out.append([[d.get(npd) for d in dd] for dd in dsts])
    return out


def same(a, b):
    for ca, cb in zip(a, b):
        for x, y in zip(ca, cb):
            assert np.array_equal(x.view(np.uint8), y.view(np.uint8))


def test_static_fold_matches_fold_on_two_calls_in_a_row():
    hcclx.init()
    stream = torch.cuda.Stream()
    rng = np.random.default_rng(77)
    # first call: 24 segments (the table spans several upload pieces), fp32 SUM chains of 8 sources, 2 destinations
    big = [(40000 + 17 * i, [payload(rng, T.FP32, 40000 + 17 * i, "uniform") for _ in range(8)], 2) for i in range(24)]
    ref, got = run_both(big, T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream)
    same(ref, got)
    # second call right after it, smaller: 3 segments of bf16 self-first folds among 4 ranks
    small = [(5001 + i, [payload(rng, T.BFP16, 5001 + i) for _ in range(4)], 4) for i in range(3)]
    ref, got = run_both(small, T.BFP16, T.SUM, hcclx.FOLD_SELF_FIRST, stream)
    same(ref, got)
    # third: one tiny tree over 5 sources (dst, src register pairs) and a pure copy to 3 places
    tree = [(777, [payload(rng, T.FP32, 777, "prod") for _ in range(5)], 1, [0, 1, 2, 3, 0, 2, 0, 4])]
    ref, got = run_both(tree, T.FP32, T.PROD, hcclx.FOLD_TREE, stream)
    same(ref, got)
    copy = [(100003, [payload(rng, T.INT8, 100003)], 3)]
    ref, got = run_both(copy, T.INT8, T.SUM, hcclx.FOLD_CHAIN, stream)
    same(ref, got)
    assert np.array_equal(got[0][0], copy[0][1][0])


def test_static_fold_rejects_more_segments_than_its_table_holds():
    hcclx.init()
    a = DevBuf(np.zeros(16, np.int32))
    b = DevBuf(nbytes=64)
    segs = [(16, [a.ptr], [b.ptr])] * (hcclx.STATIC_MAX_SEGS + 1)
    with pytest.raises(HcclError) as e:
        hcclx.fold_static(segs, T.INT32)
    assert "at most" in str(e.value)
    hcclx.fold_static(segs[:hcclx.STATIC_MAX_SEGS], T.INT32)     # the limit itself is accepted
    torch.cuda.synchronize()
    assert np.array_equal(b.get(np.int32), np.zeros(16, np.int32))
