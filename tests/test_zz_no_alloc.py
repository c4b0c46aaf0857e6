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


def _chain_case(rng, count, nsrc=8, ndst=2):
    xs = [payload(rng, T.FP32, count, "uniform") for _ in range(nsrc)]
    srcs = [DevBuf(x) for x in xs]
    return xs, srcs, ndst


def _reference(srcs, count, ndst, stream):
    """What hcclx_fold gives for the same chain."""
    dsts = [DevBuf(nbytes=count * 4) for _ in range(ndst)]
    hcclx.fold([(count, [s.ptr for s in srcs], [d.ptr for d in dsts])], T.FP32, T.SUM, hcclx.FOLD_CHAIN,
               stream=stream.cuda_stream)
    stream.synchronize()
    return dsts[0].get(np.uint32)


def test_static_fold_leaves_the_free_device_memory_as_it_was():
    """The property the entry point exists for: once the device is set up, calls allocate nothing.  hipMemGetInfo's
    free bytes are the same before and after calls of several sizes on two streams."""
    hcclx.init()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    rng = np.random.default_rng(5)
    count = 300007
    _, srcs, ndst = _chain_case(rng, count)
    dsts = [DevBuf(nbytes=count * 4) for _ in range(ndst)]

    def seg(total, parts=1):
        """`total` elements cut into `parts` segments."""
        cuts = [total * i // parts for i in range(parts + 1)]
        return [(b - a, [s.ptr + 4 * a for s in srcs], [d.ptr + 4 * a for d in dsts]) for a, b in zip(cuts, cuts[1:])]
    hcclx.fold_static(seg(count), T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream=s1.cuda_stream)   # the kernel's code is loaded now
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for k in range(6):
        st = s1 if k % 2 == 0 else s2
        hcclx.fold_static(seg(count - 1000 * k, 1 + 20 * (k % 3)), T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream=st.cuda_stream)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)


def test_static_fold_calls_on_two_streams_and_two_threads_take_turns_on_the_one_table():
    """Calls on different streams share the library's one launch table: each waits for the fold of the call before
    it, so none overwrites a table a running kernel still reads.  Alternating streams without any host
    synchronisation, then two host threads at once; every output equals hcclx_fold's."""
    import threading
    hcclx.init()
    rng = np.random.default_rng(9)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ref_stream = torch.cuda.Stream()
    # two different shapes, large enough that the fold of one call is still running when the next is issued
    shapes = [(1 << 21) + 11, (1 << 20) + 3]
    cases = []
    for k, count in enumerate(shapes):
        _, srcs, ndst = _chain_case(rng, count, nsrc=4 + 4 * k, ndst=1 + k)
        cases.append((count, srcs, ndst, _reference(srcs, count, ndst, ref_stream)))
    reps = 12
    outs = [[[DevBuf(nbytes=c[0] * 4) for _ in range(c[2])] for _ in range(reps)] for c in cases]
    torch.cuda.synchronize()
    for rep in range(reps):
        for k, (count, srcs, ndst, _) in enumerate(cases):
            # several segments per call, so that the table of one call differs from the other's in every entry
            cut = count // 3
            segs = [(cut, [s.ptr for s in srcs], [d.ptr for d in outs[k][rep]]),
                    (count - cut, [s.ptr + cut * 4 for s in srcs], [d.ptr + cut * 4 for d in outs[k][rep]])]
            hcclx.fold_static(segs, T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream=streams[k].cuda_stream)
    torch.cuda.synchronize()
    for k, (count, srcs, ndst, want) in enumerate(cases):
        for rep in range(reps):
            for d in outs[k][rep]:
                assert np.array_equal(d.get(np.uint32), want), (k, rep)
                assert d.guard_intact()

    # two host threads, one stream each
    outs2 = [[[DevBuf(nbytes=c[0] * 4) for _ in range(c[2])] for _ in range(reps)] for c in cases]
    torch.cuda.synchronize()
    errors = []

    def worker(k):
        try:
            count, srcs, ndst, _ = cases[k]
            for rep in range(reps):
                hcclx.fold_static([(count, [s.ptr for s in srcs], [d.ptr for d in outs2[k][rep]])], T.FP32, T.SUM,
                                  hcclx.FOLD_CHAIN, stream=streams[k].cuda_stream)
        except Exception as e:      # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)
    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for k, (count, srcs, ndst, want) in enumerate(cases):
        for rep in range(reps):
            for d in outs2[k][rep]:
                assert np.array_equal(d.get(np.uint32), want), (k, rep)


def test_static_fold_captured_into_a_graph_replays_after_other_calls_used_the_table():
    """The use include/hcclx.h names first: the call is captured into a HIP graph (no refusal: nothing is uploaded
    through a copy), and a replay re-sends its own table, so it still gives hcclx_fold's result after an eager call
    with other segments has overwritten the table in between."""
    hcclx.init()
    rng = np.random.default_rng(21)
    s = torch.cuda.Stream()
    count = 123457
    xs, srcs, ndst = _chain_case(rng, count, nsrc=5, ndst=3)
    dsts = [DevBuf(nbytes=count * 4) for _ in range(ndst)]
    segs = [(count, [b.ptr for b in srcs], [d.ptr for d in dsts])]
    other_x, other_src, _ = _chain_case(rng, 7001, nsrc=3, ndst=1)
    other_dst = DevBuf(nbytes=7001 * 4)
    hcclx.fold_static(segs, T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream=s.cuda_stream)     # warm: kernels loaded
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        g.capture_begin()
        hcclx.fold_static(segs, T.FP32, T.SUM, hcclx.FOLD_CHAIN, stream=s.cuda_stream)
        g.capture_end()
    for rep in range(3):
        # new data in the sources, outputs cleared, and an eager call that rewrites the table, all between replays
        for b in srcs:
            x = payload(rng, T.FP32, count, "uniform")
            b.t[b.offset:b.offset + b.nbytes] = torch.from_numpy(x.view(np.uint8).copy()).to("cuda:0")
        for d in dsts:
            d.t.fill_(0xA5)
        hcclx.fold_static([(7001, [b.ptr for b in other_src], [other_dst.ptr])], T.FP32, T.SUM, hcclx.FOLD_CHAIN,
                          stream=s.cuda_stream)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = _reference(srcs, count, ndst, s)
        for d in dsts:
            assert np.array_equal(d.get(np.uint32), want), rep
            assert d.guard_intact()
