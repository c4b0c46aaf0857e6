"""GPU parity of the fold kernels through the C ABI (hcclx_fold / hcclx_plan_*), against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import hcclx
from hccl_amd._lib import HcclError

from gpu_util import DevBuf, assert_same_bits, fold_oracle, fused_is_wide, payload

pytestmark = pytest.mark.gpu

REDUCE_DTYPES = [T.INT8, T.INT16, T.INT32, T.INT64, T.UINT64, T.FP16, T.FP32, T.FP64, T.BFP16]
OPS = [T.SUM, T.PROD, T.MAX, T.MIN]


def sync():
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", REDUCE_DTYPES)
@pytest.mark.parametrize("op", OPS)
def test_pairwise_step_in_place_matches_reference_loop(dtype, op):
    """dst = src (+) dst, the LocalReduce step, in place, with a ragged count and a misaligned source."""
    rng = np.random.default_rng(100 + dtype * 4 + op)
    n = 70001
    kind = "bits" if dtype in (T.FP16, T.BFP16) and op != T.PROD else ("prod" if op == T.PROD else "normal")
    a, b = payload(rng, dtype, n, kind), payload(rng, dtype, n, kind)
    esz = T.DTYPE_SIZE[dtype]
    src, dst = DevBuf(a, offset=esz), DevBuf(b, offset=256)
    hcclx.fold([(n, [dst.ptr, src.ptr], [dst.ptr])], dtype, op)
    sync()
    want = fold_oracle([b, a], dtype, op, [0, 1], wide=False)
    assert_same_bits(dst.get(T.NP_STORAGE[dtype]), want, dtype, f"dtype {dtype} op {op}")
    assert dst.guard_intact() and src.guard_intact()


@pytest.mark.parametrize("nsrc", [3, 4, 5, 8, 9, 12, 16])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.FP32, T.PROD), (T.BFP16, T.SUM), (T.FP16, T.SUM),
                                      (T.FP16, T.PROD), (T.FP64, T.SUM), (T.INT32, T.MAX), (T.FP32, T.MAX),
                                      (T.INT8, T.SUM), (T.INT8, T.PROD), (T.INT8, T.MAX), (T.INT8, T.MIN)])
def test_chain_fold_reproduces_the_fold_order(nsrc, dtype, op):
    rng = np.random.default_rng(nsrc * 100 + dtype)
    n = 2 * 4096 + 13
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    xs = [payload(rng, dtype, n, kind) for _ in range(nsrc)]
    order = list(rng.permutation(nsrc))
    esz = T.DTYPE_SIZE[dtype]
    bufs = [DevBuf(x, offset=(k % 3) * esz) for k, x in enumerate(xs)]       # element-aligned, not 16-byte aligned
    outs = [DevBuf(nbytes=xs[0].nbytes, offset=(1 + 2 * k) * esz) for k in range(3)]
    hcclx.fold([(n, [bufs[k].ptr for k in order], [o.ptr for o in outs])], dtype, op)
    sync()
    want = fold_oracle(xs, dtype, op, order, wide=fused_is_wide(dtype, op))
    for o in outs:
        assert_same_bits(o.get(T.NP_STORAGE[dtype]), want, dtype)
        assert o.guard_intact()


@pytest.mark.parametrize("nsrc", [2, 3, 8, 12, 16])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.FP32, T.PROD), (T.BFP16, T.SUM), (T.FP16, T.PROD),
                                      (T.INT32, T.SUM), (T.INT64, T.MIN), (T.FP64, T.PROD)])
def test_self_first_fold_gives_every_rank_its_own_order(nsrc, dtype, op):
    rng = np.random.default_rng(nsrc * 10 + dtype + op)
    n = 4096 + 3
    xs = [payload(rng, dtype, n, "prod" if op == T.PROD else "normal") for _ in range(nsrc)]
    bufs = [DevBuf(x) for x in xs]
    outs = [DevBuf(nbytes=xs[0].nbytes) for _ in range(nsrc)]
    hcclx.fold([(n, [b.ptr for b in bufs], [o.ptr for o in outs])], dtype, op, hcclx.FOLD_SELF_FIRST)
    sync()
    for r in range(nsrc):
        order = [r] + [k for k in range(nsrc) if k != r]
        want = fold_oracle(xs, dtype, op, order, wide=fused_is_wide(dtype, op))
        assert_same_bits(outs[r].get(T.NP_STORAGE[dtype]), want, dtype, f"rank {r}")


def test_self_first_in_place_allreduce():
    """sendBuf == recvBuf on every rank: each destination aliases one source."""
    rng = np.random.default_rng(5)
    n, nsrc = 10007, 8
    xs = [payload(rng, T.FP32, n, "uniform") for _ in range(nsrc)]
    bufs = [DevBuf(x) for x in xs]
    hcclx.fold([(n, [b.ptr for b in bufs], [b.ptr for b in bufs])], T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)
    sync()
    for r in range(nsrc):
        order = [r] + [k for k in range(nsrc) if k != r]
        assert_same_bits(bufs[r].get(np.float32), fold_oracle(xs, T.FP32, T.SUM, order, False), T.FP32)


@pytest.mark.parametrize("nsrc,ndst", [(1, 40), (2, 1), (17, 3), (24, 24), (33, 17), (40, 1), (64, 64)])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.BFP16, T.SUM), (T.FP16, T.PROD), (T.FP64, T.PROD),
                                      (T.INT8, T.MAX), (T.INT64, T.MIN), (T.INT16, T.SUM)])
def test_wide_chain_fold_up_to_64_sources_and_destinations(nsrc, ndst, dtype, op):
    """hcclx_fold_wide: the chain order over more sources than the register-resident kernel holds, operands at
    element alignment, a count that leaves a head and a tail, two segments in one launch."""
    rng = np.random.default_rng(nsrc * 1000 + ndst * 10 + dtype)
    esz = T.DTYPE_SIZE[dtype]
    counts = [3 * 4096 // esz + 13, 7]
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    segs, checks = [], []
    for si, n in enumerate(counts):
        xs = [payload(rng, dtype, n, kind) for _ in range(nsrc)]
        order = list(rng.permutation(nsrc))
        bufs = [DevBuf(x, offset=(k % 5) * esz) for k, x in enumerate(xs)]
        outs = [DevBuf(nbytes=xs[0].nbytes, offset=((si + k) % 7) * esz) for k in range(ndst)]
        segs.append((n, [bufs[k].ptr for k in order], [o.ptr for o in outs]))
        checks.append((xs, order, bufs, outs))
    hcclx.fold_wide(segs, dtype, op)
    sync()
    for xs, order, bufs, outs in checks:
        want = fold_oracle(xs, dtype, op, order, wide=fused_is_wide(dtype, op))
        for o in outs:
            assert_same_bits(o.get(T.NP_STORAGE[dtype]), want, dtype)
            assert o.guard_intact()
        assert all(b.guard_intact() for b in bufs)


def test_wide_fold_in_place_copy_of_any_type_plan_and_errors():
    rng = np.random.default_rng(77)
    n, nsrc = 50001, 20
    xs = [payload(rng, T.FP32, n, "uniform") for _ in range(nsrc)]
    bufs = [DevBuf(x) for x in xs]
    segs = [(n, [b.ptr for b in bufs], [bufs[0].ptr, bufs[7].ptr])]     # two destinations alias sources
    plan = hcclx.Plan(segs, T.FP32, T.SUM, wide=True)
    assert plan.bytes == (nsrc + 2) * n * 4
    plan.launch()
    sync()
    want = fold_oracle(xs, T.FP32, T.SUM, list(range(nsrc)), False)
    assert_same_bits(bufs[0].get(np.float32), want, T.FP32)
    assert_same_bits(bufs[7].get(np.float32), want, T.FP32)
    plan.close()
    raw = rng.integers(0, 255, size=30011, dtype=np.uint8)              # a copy moves any type as bytes
    src = DevBuf(raw, offset=3)
    outs = [DevBuf(nbytes=raw.nbytes, offset=k % 16) for k in range(33)]
    hcclx.fold_wide([(raw.size, [src.ptr], [o.ptr for o in outs])], T.UINT8)
    sync()
    for o in outs:
        assert np.array_equal(o.get(np.uint8), raw) and o.guard_intact()
    b = DevBuf(nbytes=64)
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(4, [b.ptr] * 65, [b.ptr])], T.FP32, T.SUM)
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(4, [b.ptr] * 20, [b.ptr] * 19 + [0])], T.FP32, T.SUM)
    assert e.value.code == 2
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(4, [b.ptr] * 20, [b.ptr])], T.UINT8, T.SUM)
    assert e.value.code == 5
    hcclx.fold_wide([], T.FP32, T.SUM)
    hcclx.fold_wide([(0, [0] * 20, [0])], T.FP32)
    sync()


def random_tree(rng, nsrc, max_levels=4):
    """A random (dst register, src register) program over nsrc registers whose tree has at most
    max_levels levels, register 0 holding the root."""
    while True:
        depth = {k: 0 for k in range(nsrc)}
        prog = []
        for _ in range(nsrc - 1):
            live = list(depth)
            pairs = [(d, s) for d in live for s in live
                     if d != s and s != 0 and max(depth[d], depth[s]) + 1 <= max_levels]
            if not pairs:
                break
            d, s = pairs[rng.integers(len(pairs))]
            depth[d] = max(depth[d], depth[s]) + 1
            del depth[s]
            prog += [d, s]
        if len(prog) == 2 * (nsrc - 1):
            return prog


def tree_oracle(xs, dtype, op, prog, wide):
    if wide:
        regs = [T.widen16(x, dtype) for x in xs]
        e = T.NumericElems(T.FP32, op)
    else:
        regs = [np.ascontiguousarray(x).copy() for x in xs]
        e = T.NumericElems(dtype, op)
    for t in range(len(prog) // 2):
        d, s = prog[2 * t], prog[2 * t + 1]
        e.reduce(regs[d], 0, regs[s], 0, regs[d].size)
    return T.narrow16(regs[0], dtype) if wide else regs[0]


@pytest.mark.parametrize("nsrc", [2, 3, 4, 5, 7, 8, 11, 12, 16])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.FP32, T.MAX), (T.BFP16, T.SUM), (T.FP16, T.PROD),
                                      (T.FP64, T.SUM), (T.INT32, T.SUM), (T.FP16, T.MIN)])
def test_tree_fold_keeps_the_association_of_the_program(nsrc, dtype, op):
    """Log-step schedules (NHR, halving-doubling) pair partial results with partial results; the tree
    mode evaluates exactly that pairing, operand order included."""
    rng = np.random.default_rng(nsrc * 31 + dtype * 5 + op)
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    segs, cases = [], []
    for count in (4096 * 3 + 7, 1, 1000):
        xs = [payload(rng, dtype, count, kind) for _ in range(nsrc)]
        prog = random_tree(rng, nsrc)
        bufs = [DevBuf(x) for x in xs]
        outs = [DevBuf(nbytes=xs[0].nbytes) for _ in range(2)]
        segs.append((count, [b.ptr for b in bufs], [o.ptr for o in outs], prog))
        cases.append((xs, prog, bufs, outs))
    hcclx.fold(segs, dtype, op, hcclx.FOLD_TREE)
    sync()
    for xs, prog, bufs, outs in cases:
        want = tree_oracle(xs, dtype, op, prog, fused_is_wide(dtype, op))
        for o in outs:
            assert_same_bits(o.get(T.NP_STORAGE[dtype]), want, dtype, f"program {prog}")
            assert o.guard_intact()


def split_tree(rng, nsrc, max_levels):
    """A random program over nsrc registers whose tree has at most max_levels levels: the registers (0 first)
    are split recursively into a dst side and a src side that both still fit."""
    regs = [0] + [int(r) + 1 for r in rng.permutation(nsrc - 1)]
    prog = []

    def node(lst, levels):
        if len(lst) == 1:
            return lst[0]
        half = 1 << (levels - 1)
        lo, hi = max(1, len(lst) - half), min(half, len(lst) - 1)
        k = int(rng.integers(lo, hi + 1))
        d = node(lst[:k], levels - 1)
        s_ = node(lst[k:], levels - 1)
        prog.extend([d, s_])
        return d

    node(regs, max_levels)
    return prog


@pytest.mark.parametrize("nsrc,levels", [(6, 5), (7, 6), (17, 5), (20, 6), (33, 6), (40, 6), (64, 6)])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.BFP16, T.SUM), (T.FP16, T.PROD), (T.FP64, T.MAX),
                                      (T.INT32, T.SUM)])
def test_wide_tree_fold_up_to_six_levels(nsrc, levels, dtype, op):
    """hcclx_fold_wide in tree mode: trees with more leaves or levels than the 16-slot kernel holds (the NHR and
    halving-doubling schedules among 17 .. 64 ranks)."""
    rng = np.random.default_rng(nsrc * 77 + dtype * 3 + op)
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    esz = T.DTYPE_SIZE[dtype]
    segs, cases = [], []
    for si, count in enumerate((2 * 4096 // esz + 5, 3)):
        xs = [payload(rng, dtype, count, kind) for _ in range(nsrc)]
        prog = split_tree(rng, nsrc, levels)
        bufs = [DevBuf(x, offset=(k % 4) * esz) for k, x in enumerate(xs)]
        outs = [DevBuf(nbytes=xs[0].nbytes, offset=(si + 3 * k) % 5 * esz) for k in range(18)]
        segs.append((count, [b.ptr for b in bufs], [o.ptr for o in outs], prog))
        cases.append((xs, prog, outs, bufs))     # the sources must stay allocated until the launch has run
    hcclx.fold_wide(segs, dtype, op, hcclx.FOLD_TREE)
    sync()
    for xs, prog, outs, _ in cases:
        want = tree_oracle(xs, dtype, op, prog, fused_is_wide(dtype, op))
        for o in outs:
            assert_same_bits(o.get(T.NP_STORAGE[dtype]), want, dtype, f"program {prog}")
            assert o.guard_intact()


@pytest.mark.parametrize("nsrc", [17, 24, 32, 33, 48, 64])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.BFP16, T.SUM), (T.FP16, T.PROD), (T.FP64, T.MAX), (T.INT32, T.SUM)])
def test_wide_self_first_fold_gives_every_rank_its_own_order(nsrc, dtype, op):
    """The per-rank orders of the one-shot templates among 17 .. 64 ranks: output j starts from source j and takes
    the others ascending; outputs are computed sixteen at a time."""
    rng = np.random.default_rng(nsrc * 13 + dtype + op)
    esz = T.DTYPE_SIZE[dtype]
    n = 2 * 4096 // esz + 11
    kind = "prod" if op == T.PROD else "uniform" if dtype in (T.FP32, T.FP64) else "normal"
    xs = [payload(rng, dtype, n, kind) for _ in range(nsrc)]
    bufs = [DevBuf(x, offset=(k % 3) * esz) for k, x in enumerate(xs)]
    outs = [DevBuf(nbytes=xs[0].nbytes, offset=(k % 5) * esz) for k in range(nsrc)]
    hcclx.fold_wide([(n, [b.ptr for b in bufs], [o.ptr for o in outs])], dtype, op, hcclx.FOLD_SELF_FIRST)
    sync()
    for r in range(nsrc):
        order = [r] + [k for k in range(nsrc) if k != r]
        want = fold_oracle(xs, dtype, op, order, wide=fused_is_wide(dtype, op))
        assert_same_bits(outs[r].get(T.NP_STORAGE[dtype]), want, dtype, f"rank {r}")
        assert outs[r].guard_intact()


def test_wide_self_first_fold_rejects_in_place():
    x = np.arange(1024, dtype=np.float32)
    bufs = [DevBuf(x + k) for k in range(20)]
    outs = [DevBuf(nbytes=x.nbytes) for _ in range(20)]
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(1024, [b.ptr for b in bufs], [b.ptr for b in bufs])], T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(1024, [b.ptr for b in bufs], [o.ptr for o in outs[:19]])], T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)
    assert e.value.code == 1
    # integers have one value whatever the order, so in place is taken (one chain, twenty destinations)
    xi = [np.arange(1024, dtype=np.int32) * (k + 1) for k in range(20)]
    ib = [DevBuf(v) for v in xi]
    hcclx.fold_wide([(1024, [b.ptr for b in ib], [b.ptr for b in ib])], T.INT32, T.SUM, hcclx.FOLD_SELF_FIRST)
    sync()
    for b in ib:
        assert np.array_equal(b.get(np.int32), np.arange(1024, dtype=np.int32) * 210)


def test_wide_tree_fold_rejects_seven_levels_and_malformed_programs():
    b = DevBuf(nbytes=64)
    deep = [x for k in range(1, 8) for x in (0, k)]     # a spine of seven levels
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(4, [b.ptr] * 8, [b.ptr], deep)], T.FP32, T.SUM, hcclx.FOLD_TREE)
    assert e.value.code == 5
    with pytest.raises(HcclError) as e:
        hcclx.fold_wide([(4, [b.ptr] * 3, [b.ptr], [0, 1, 0, 1])], T.FP32, T.SUM, hcclx.FOLD_TREE)
    assert e.value.code == 1


def test_tree_fold_in_place_and_chain_shaped_program():
    """The result may overwrite register 0's source; a left-deep program of up to four steps equals the
    chain fold of the same order."""
    rng = np.random.default_rng(77)
    n = 30011
    xs = [payload(rng, T.FP32, n, "uniform") for _ in range(5)]
    bufs = [DevBuf(x) for x in xs]
    prog = [0, 1, 0, 2, 0, 3, 0, 4]
    hcclx.fold([(n, [b.ptr for b in bufs], [bufs[0].ptr], prog)], T.FP32, T.SUM, hcclx.FOLD_TREE)
    sync()
    assert_same_bits(bufs[0].get(np.float32), fold_oracle(xs, T.FP32, T.SUM, [0, 1, 2, 3, 4], False), T.FP32)


def test_tree_fold_rejects_what_the_kernel_cannot_hold():
    b = DevBuf(nbytes=64)
    deep = [0, 1, 0, 2, 0, 3, 0, 4, 0, 5]     # five levels
    with pytest.raises(HcclError) as e:
        hcclx.fold([(4, [b.ptr] * 6, [b.ptr], deep)], T.FP32, T.SUM, hcclx.FOLD_TREE)
    assert e.value.code == 5
    for bad in ([1, 0, 1, 2], [0, 1, 0, 1], [0, 3, 0, 1], [0, 1, 1, 2]):   # consumes 0 / twice / out of range / dead dst
        with pytest.raises(HcclError) as e:
            hcclx.fold([(4, [b.ptr] * 3, [b.ptr], bad)], T.FP32, T.SUM, hcclx.FOLD_TREE)
        assert e.value.code == 1, bad
    # integers are association-free: any well-formed program is taken, however deep
    x = np.arange(16, dtype=np.int32)
    bufs = [DevBuf(x + k) for k in range(6)]
    out = DevBuf(nbytes=64)
    hcclx.fold([(16, [q.ptr for q in bufs], [out.ptr], deep)], T.INT32, T.SUM, hcclx.FOLD_TREE)
    sync()
    assert np.array_equal(out.get(np.int32), 6 * x + 15)


def test_fp32_subnormals_and_signed_zeros_survive():
    a = np.array([1e-45, -1e-45, 1e-39, 0.0, -0.0, 3e-39, 1.17549435e-38] * 37, dtype=np.float32)
    b = np.array([1e-45, 1e-45, -2e-39, -0.0, -0.0, 3e-39, -1e-45] * 37, dtype=np.float32)
    for op in OPS:
        da, db = DevBuf(a), DevBuf(b)
        hcclx.fold([(a.size, [db.ptr, da.ptr], [db.ptr])], T.FP32, op)
        sync()
        assert_same_bits(db.get(np.float32), fold_oracle([b, a], T.FP32, op, [0, 1], False), T.FP32, f"op {op}")


def test_float_max_min_nan_and_zero_operand_order():
    src = np.array([np.nan, 1.0, 0.0, -0.0, np.inf, -np.inf] * 11, dtype=np.float32)
    dst = np.array([1.0, np.nan, -0.0, 0.0, np.nan, 2.0] * 11, dtype=np.float32)
    for op in (T.MAX, T.MIN):
        ds, dd = DevBuf(src), DevBuf(dst)
        hcclx.fold([(src.size, [dd.ptr, ds.ptr], [dd.ptr])], T.FP32, op)
        sync()
        assert_same_bits(dd.get(np.float32), fold_oracle([dst, src], T.FP32, op, [0, 1], False), T.FP32)


def special_floats(rng, dtype, n):
    """Values whose max / min depends on which operand comes first: signed zeros, NaNs, repeated values."""
    pool = np.array([0.0, -0.0, np.nan, 1.0, -1.0, np.inf, -np.inf, 0.5], dtype=np.float32)
    f = pool[rng.integers(0, pool.size, size=n)]
    if dtype in (T.FP16, T.BFP16):
        return T.narrow16(f, dtype)
    return f.astype(T.NP_STORAGE[dtype])


@pytest.mark.parametrize("nsrc", [2, 3, 8, 9, 16, 23, 64])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.MAX), (T.FP32, T.MIN), (T.BFP16, T.MAX), (T.FP16, T.MIN),
                                      (T.FP64, T.MAX), (T.FP32, T.SUM), (T.INT32, T.MAX)])
def test_chain_steps_with_swapped_operands(nsrc, dtype, op):
    """A chain step marked in prog[] computes acc (+) src[k] instead of src[k] (+) acc: what a ring does when it
    hands the accumulated value on.  Floating-point max and min tell the two apart for signed zeros and NaNs."""
    rng = np.random.default_rng(nsrc * 31 + dtype * 7 + op)
    n = 4096 + 13
    is_float = dtype in (T.FP16, T.BFP16, T.FP32, T.FP64)
    if is_float and op != T.SUM:
        xs = [special_floats(rng, dtype, n) for _ in range(nsrc)]
    else:
        xs = [payload(rng, dtype, n, "uniform" if is_float else "normal") for _ in range(nsrc)]
    swaps = [0] + [int(b) for b in rng.integers(0, 2, size=nsrc - 1)]
    swaps[-1] = 1
    e = T.NumericElems(dtype, op)
    acc = xs[0].copy()
    for k in range(1, nsrc):
        if swaps[k]:                       # acc is the source operand: the value lands where src[k] was
            nxt = xs[k].copy()
            e.reduce(nxt, 0, acc, 0, n)
            acc = nxt
        else:
            e.reduce(acc, 0, xs[k], 0, n)
    bufs = [DevBuf(x) for x in xs]
    outs = [DevBuf(nbytes=xs[0].nbytes) for _ in range(2)]
    seg = (n, [b.ptr for b in bufs], [o.ptr for o in outs], swaps)
    if nsrc <= 16:
        hcclx.fold([seg], dtype, op)
    else:
        hcclx.fold_wide([seg], dtype, op)
    sync()
    for o in outs:
        assert_same_bits(o.get(T.NP_STORAGE[dtype]), acc, dtype)
        assert o.guard_intact()


def test_many_ragged_segments_and_empty_ones():
    rng = np.random.default_rng(8)
    counts = [0, 1, 3, 4, 5, 255, 256, 257, 1023, 1024, 4099, 0, 8191, 65537] + list(rng.integers(0, 3000, 2200))
    segs, checks = [], []
    big_a = payload(rng, T.INT32, int(sum(counts)) + 8)
    big_b = payload(rng, T.INT32, int(sum(counts)) + 8)
    da, db = DevBuf(big_a), DevBuf(big_b)
    out = DevBuf(nbytes=big_a.nbytes)
    off = 0
    for c in counts:
        c = int(c)
        segs.append((c, [da.ptr + off * 4, db.ptr + off * 4], [out.ptr + off * 4]))
        off += c
    hcclx.fold(segs, T.INT32, T.SUM)      # more segments than one launch holds: the launcher splits
    sync()
    want = fold_oracle([big_a, big_b], T.INT32, T.SUM, [0, 1], False)
    assert np.array_equal(out.get(np.int32)[:off], want[:off])
    assert (out.get(np.uint8)[off * 4:] == 0xA5).all()


@pytest.mark.parametrize("soff,doff", [(0, 0), (1, 0), (0, 3), (5, 9), (16, 2), (7, 7)])
def test_copy_any_alignment_to_several_destinations(soff, doff):
    rng = np.random.default_rng(soff * 16 + doff)
    n = 300003
    x = rng.integers(0, 256, size=n, dtype=np.uint8)
    src = DevBuf(x, offset=soff)
    dsts = [DevBuf(nbytes=n, offset=doff) for _ in range(3)]
    hcclx.fold([(n, [src.ptr], [d.ptr for d in dsts])], T.UINT8)
    sync()
    for d in dsts:
        assert np.array_equal(d.get(np.uint8), x) and d.guard_intact()


def test_plan_relaunch_and_algorithmic_bytes():
    rng = np.random.default_rng(1)
    n = 50000
    xs = [payload(rng, T.FP32, n, "uniform") for _ in range(4)]
    bufs = [DevBuf(x) for x in xs]
    out = DevBuf(nbytes=n * 4)
    plan = hcclx.Plan([(n, [b.ptr for b in bufs], [out.ptr])], T.FP32, T.SUM)
    assert plan.bytes == 5 * n * 4
    for _ in range(3):
        out.t.zero_()
        plan.launch()
        sync()
        assert_same_bits(out.get(np.float32), fold_oracle(xs, T.FP32, T.SUM, [0, 1, 2, 3], False), T.FP32)
    plan.close()


def test_errors_are_reported_not_launched():
    b = DevBuf(nbytes=64)
    with pytest.raises(HcclError) as e:
        hcclx.fold([(4, [b.ptr] * 17, [b.ptr])], T.FP32, T.SUM)
    assert e.value.code == 1      # HCCL_E_PARA
    with pytest.raises(HcclError) as e:
        hcclx.fold([(4, [b.ptr, 0], [b.ptr])], T.FP32, T.SUM)
    assert e.value.code == 2      # HCCL_E_PTR
    with pytest.raises(HcclError) as e:
        hcclx.fold([(4, [b.ptr, b.ptr], [b.ptr])], T.UINT8, T.SUM)
    assert e.value.code == 5      # HCCL_E_NOT_SUPPORT: uint8 is not a reduce type
    with pytest.raises(HcclError) as e:
        hcclx.fold([(4, [b.ptr, b.ptr], [b.ptr, b.ptr, b.ptr])], T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)
    assert e.value.code == 1
    hcclx.fold([], T.FP32, T.SUM)           # nothing to do is fine
    hcclx.fold([(0, [0, 0], [0])], T.FP32)  # zero-size slices are skipped (LocalCopy/LocalReduce do the same)
    sync()
