"""The fold kernel with one wavefront per source / destination (every wavefront issues a single store per piece)
against the oracle and against the register kernel: same bits.  The kernel is a launch policy, not a mode, so the
tests switch it on for every eligible launch through hcclx_tune and switch the defaults back afterwards."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import api, hcclx
from hccl_amd._lib import HcclError

from gpu_util import DevBuf, assert_same_bits, fold_oracle, fused_is_wide, payload

pytestmark = pytest.mark.gpu

DEFAULTS = {"waves_from": 1, "waves_max_fan": 16, "waves_chains": 0, "waves_pieces": 0}


@pytest.fixture()
def waves_everywhere():
    hcclx.init()
    hcclx.tune("waves_from", 1)
    hcclx.tune("waves_max_fan", 16)
    hcclx.tune("waves_chains", 1)
    yield
    for name, value in DEFAULTS.items():
        hcclx.tune(name, value)


def chain_oracle(xs, dtype, op, swaps):
    """acc = xs[0]; step k: acc = xs[k] (+) acc, or acc (+) xs[k] where swaps[k]; 16-bit SUM accumulates in fp32."""
    if fused_is_wide(dtype, op):
        return fold_oracle(xs, dtype, op, list(range(len(xs))), wide=True)
    e = T.NumericElems(dtype, op)
    acc = xs[0].copy()
    for k in range(1, len(xs)):
        if swaps[k]:
            nxt = xs[k].copy()
            e.reduce(nxt, 0, acc, 0, acc.size)
            acc = nxt
        else:
            e.reduce(acc, 0, xs[k], 0, acc.size)
    return acc


def fold_both(segs, dtype, op, mode, dsts):
    """Runs the launch with the wavefront kernel (the fixture has switched it on) and with the register kernels;
    returns the destinations' contents of both runs."""
    out = []
    for waves in (True, False):
        hcclx.tune("waves_from", 1 if waves else 0)
        for d in dsts:
            d.t.fill_(0xA5)
        hcclx.fold(segs, dtype, op, mode)
        torch.cuda.synchronize()
        out.append([d.get(T.NP_STORAGE[dtype]) for d in dsts])
        assert all(d.guard_intact() for d in dsts)
    hcclx.tune("waves_from", 1)
    return out


SELF_FIRST_CASES = [(pieces, nsrc, dtype, op)
                    for pieces in (0, 8) for nsrc in (2, 3, 4, 5, 8, 11, 12, 16)
                    for dtype, op in ((T.FP32, T.PROD), (T.FP32, T.SUM), (T.BFP16, T.SUM), (T.FP16, T.PROD), (T.FP64, T.MAX))]
SELF_FIRST_CASES += [(pieces, nsrc, T.FP32, op) for pieces in (1, 3) for nsrc in (3, 12) for op in (T.PROD, T.SUM)]


@pytest.mark.parametrize("pieces,nsrc,dtype,op", SELF_FIRST_CASES)
def test_self_first_orders_on_the_wavefront_kernel(waves_everywhere, pieces, nsrc, dtype, op):
    """Every rank's own order, for source counts with and without a straight-line fold path, several pieces per
    workgroup, counts that leave a head, a tail and a partly filled last tile, sources at element alignment."""
    hcclx.tune("waves_pieces", pieces)
    rng = np.random.default_rng(nsrc * 10 + dtype + op + pieces)
    esz = T.DTYPE_SIZE[dtype]
    for n in (5, 3 * 4096 // esz + 13, 70001):
        xs = [payload(rng, dtype, n, "prod" if op == T.PROD else "normal") for _ in range(nsrc)]
        bufs = [DevBuf(x, offset=(k % 3) * esz) for k, x in enumerate(xs)]
        outs = [DevBuf(nbytes=xs[0].nbytes, offset=(1 + k % 5) * esz) for k in range(nsrc)]
        before = hcclx.kernels_launched()
        got, ref = fold_both([(n, [b.ptr for b in bufs], [o.ptr for o in outs])], dtype, op, hcclx.FOLD_SELF_FIRST, outs)
        assert hcclx.kernels_launched() - before == 2
        for r in range(nsrc):
            order = [r] + [k for k in range(nsrc) if k != r]
            want = fold_oracle(xs, dtype, op, order, wide=fused_is_wide(dtype, op))
            assert_same_bits(got[r], want, dtype, f"n={n} rank {r}")
            assert np.array_equal(got[r].view(np.uint8), ref[r].view(np.uint8)), f"n={n} rank {r}: differs from the register kernel"


@pytest.mark.parametrize("nsrc,ndst", [(2, 2), (3, 7), (8, 8), (6, 16), (12, 12), (16, 2)])
@pytest.mark.parametrize("dtype,op", [(T.FP32, T.SUM), (T.FP32, T.MAX), (T.BFP16, T.SUM), (T.INT8, T.SUM), (T.INT32, T.MAX),
                                      (T.INT64, T.PROD)])
def test_chains_to_several_places_on_the_wavefront_kernel(waves_everywhere, nsrc, ndst, dtype, op):
    """A chain whose value goes to ndst places, in a fold order that is a permutation, with the operand order of some
    steps swapped (floating-point max tells), three segments of different length in one launch."""
    rng = np.random.default_rng(nsrc * 100 + ndst + dtype + op)
    esz = T.DTYPE_SIZE[dtype]
    segs, checks, all_outs, alive = [], [], [], []
    for si, n in enumerate((4099, 9, 50021)):
        kind = "prod" if op == T.PROD else "uniform" if dtype == T.FP32 else "normal"
        xs = [payload(rng, dtype, n, kind) for _ in range(nsrc)]
        if dtype == T.FP32 and op == T.MAX:
            xs[0][::7] = -0.0
            xs[1][::7] = 0.0
        order = list(rng.permutation(nsrc))
        prog = [0] + [int(rng.integers(2)) for _ in range(nsrc - 1)]
        bufs = [DevBuf(x, offset=(k % 4) * esz) for k, x in enumerate(xs)]
        outs = [DevBuf(nbytes=xs[0].nbytes, offset=((si + k) % 6) * esz) for k in range(ndst)]
        segs.append((n, [bufs[k].ptr for k in order], [o.ptr for o in outs], prog))
        checks.append(([xs[k] for k in order], prog, outs))
        alive.append(bufs)
        all_outs += outs
    got, ref = fold_both(segs, dtype, op, hcclx.FOLD_CHAIN, all_outs)
    at = 0
    for si, (xs, prog, outs) in enumerate(checks):
        want = chain_oracle(xs, dtype, op, prog)
        for k in range(len(outs)):
            assert_same_bits(ref[at + k], want, dtype, f"register kernel, segment {si} place {k}")
            assert_same_bits(got[at + k], want, dtype, f"segment {si} place {k}")
        at += len(outs)


def test_in_place_self_first_and_the_default_policy(waves_everywhere):
    """sendBuf == recvBuf on every rank (each destination is one of the sources); the knobs refuse values out of range."""
    rng = np.random.default_rng(5)
    n, nsrc = 100003, 8
    xs = [payload(rng, T.FP32, n, "uniform") for _ in range(nsrc)]
    bufs = [DevBuf(x) for x in xs]
    hcclx.fold([(n, [b.ptr for b in bufs], [b.ptr for b in bufs])], T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)
    torch.cuda.synchronize()
    for r in range(nsrc):
        order = [r] + [k for k in range(nsrc) if k != r]
        assert_same_bits(bufs[r].get(np.float32), fold_oracle(xs, T.FP32, T.SUM, order, False), T.FP32)
        assert bufs[r].guard_intact()
    with pytest.raises(HcclError):
        hcclx.tune("waves_max_fan", 17)
    with pytest.raises(HcclError):
        hcclx.tune("no_such_knob", 1)


def test_self_first_segments_of_different_widths_in_one_launch(waves_everywhere):
    """Segments of 3, 8 and 5 ranks in one launch: the kernel instance that reads the rank count per segment."""
    rng = np.random.default_rng(21)
    segs, checks, outs_all, alive = [], [], [], []
    for nsrc, n in ((3, 4099), (8, 70001), (5, 13)):
        xs = [payload(rng, T.FP32, n, "prod") for _ in range(nsrc)]
        bufs = [DevBuf(x, offset=(k % 2) * 4) for k, x in enumerate(xs)]
        outs = [DevBuf(nbytes=xs[0].nbytes, offset=(k % 3) * 4) for k in range(nsrc)]
        segs.append((n, [b.ptr for b in bufs], [o.ptr for o in outs]))
        checks.append((xs, outs))
        outs_all += outs
        alive.append(bufs)
    got, ref = fold_both(segs, T.FP32, T.PROD, hcclx.FOLD_SELF_FIRST, outs_all)
    at = 0
    for xs, outs in checks:
        for r in range(len(xs)):
            order = [r] + [k for k in range(len(xs)) if k != r]
            want = fold_oracle(xs, T.FP32, T.PROD, order, wide=False)
            assert_same_bits(got[at + r], want, T.FP32, f"{len(xs)} ranks, rank {r}")
            assert_same_bits(ref[at + r], want, T.FP32, f"register kernel, {len(xs)} ranks, rank {r}")
        at += len(xs)


@pytest.mark.parametrize("ragged", [True, False])
def test_many_segments_in_one_launch(waves_everywhere, ragged):
    """150 segments of four ranks cut from four inputs: ragged lengths (more than 64 segments: the tile prefix is staged
    in LDS and searched there) and equal lengths (a tile's segment follows from a division)."""
    rng = np.random.default_rng(31 + ragged)
    nsrc = 4
    counts = [int(c) for c in (rng.integers(1, 3000, 150) if ragged else [1536] * 150)]
    total = sum(counts)
    xs = [payload(rng, T.FP32, total, "prod") for _ in range(nsrc)]
    bufs = [DevBuf(x) for x in xs]
    outs = [DevBuf(nbytes=xs[0].nbytes) for _ in range(nsrc)]
    segs, off = [], 0
    for c in counts:
        segs.append((c, [b.ptr + off * 4 for b in bufs], [o.ptr + off * 4 for o in outs]))
        off += c
    hcclx.tune("waves_pieces", 2)
    before = hcclx.kernels_launched()
    got, ref = fold_both(segs, T.FP32, T.PROD, hcclx.FOLD_SELF_FIRST, outs)
    assert hcclx.kernels_launched() - before == 2
    for r in range(nsrc):
        order = [r] + [k for k in range(nsrc) if k != r]
        want = fold_oracle(xs, T.FP32, T.PROD, order, wide=False)
        assert_same_bits(got[r], want, T.FP32, f"rank {r}")
        assert_same_bits(ref[r], want, T.FP32, f"register kernel, rank {r}")


def test_prod_allreduce_of_four_ranks_takes_the_wavefront_kernel_by_default():
    """HcclAllReduce fp32 PROD among four ranks at 32 MiB per rank (the CPU-reduce NHR template: four outputs in four
    orders, 128 MiB written) with the shipped policy, sampled against the oracle; the same collective with the kernel
    switched off gives the same bits."""
    hcclx.init()
    for name, value in DEFAULTS.items():
        hcclx.tune(name, value)
    n, count = 4, 8 * 1024 * 1024 + 3
    g = torch.Generator(device="cuda:0")
    g.manual_seed(11)
    xs = [torch.rand(count, device="cuda:0", generator=g) * 0.2 + 0.9 for _ in range(n)]
    stream = torch.cuda.Stream()
    results = []
    for waves_from in (DEFAULTS["waves_from"], 0):
        hcclx.tune("waves_from", waves_from)
        outs = [torch.empty_like(x) for x in xs]
        torch.cuda.synchronize()
        w = api.World(n)
        try:
            w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceAicpuReduceNHR")
            for r in range(n):
                assert w.all_reduce(r, xs[r].data_ptr(), outs[r].data_ptr(), count, T.FP32, T.PROD, stream.cuda_stream) == 0
            stream.synchronize()
            info = w.last_info()
            assert info.algName.decode() == "InsAllReduceAicpuReduceNHR" and info.fused == 1 and info.launches == 1
        finally:
            w.close()
        results.append(outs)
    hcclx.tune("waves_from", DEFAULTS["waves_from"])
    rng = np.random.default_rng(3)
    cols = np.unique(np.concatenate([rng.integers(0, count, size=20000), np.arange(64), np.arange(count - 64, count)]))
    idx = torch.from_numpy(cols).to("cuda:0")
    sample = [x[idx].cpu().numpy() for x in xs]
    want = T.run_allreduce(T.NumericElems(T.FP32, T.PROD), sample, cols.size, 4, "InsAllReduceAicpuReduceNHR")
    for r in range(n):
        assert torch.equal(results[0][r].view(torch.int32), results[1][r].view(torch.int32)), r
        assert_same_bits(results[0][r][idx].cpu().numpy(), want[r], T.FP32, f"rank {r}")
