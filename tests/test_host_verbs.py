"""The middle and bottom boundary beyond what the built-in templates in write mode use: the one-sided reduce verbs
of the wrapper (through the plug-in of example templates, hccl_amd/examples/one_sided_templates.cc), the waits with
the process-wide time-out, and the read mode that the NHR and AlltoAllV templates take over PCIe links.  All in dry
worlds: the schedules are recorded, checked (deadlock, race, semantics) and traced without a GPU."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from oracle import templates as T
from hccl_amd import api, _lib

from host_util import FAKE_STREAM, fake_ptrs, parse_expr, parse_trace

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SMALL_CCL = 1024 * 1024 + 64 * 1024
PLUGIN = os.path.join(ROOT, "hccl_amd", "lib", "libhccl_one_sided_templates.so")
ROOT_COLLECTS = ["ExampleAllReduceReadReduce", "ExampleAllReduceBatchReadReduce", "ExampleAllReduceWriteReduce",
                 "ExampleAllReduceBatchWriteReduce", "ExampleAllReduceReadThenAicpuReduce"]


@pytest.fixture(scope="module")
def plugin():
    if not os.path.exists(PLUGIN):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "hccl_amd", "csrc"), PLUGIN])
    _lib.load()
    return ctypes.CDLL(PLUGIN, mode=ctypes.RTLD_GLOBAL)


def chain(n, off=0):
    """x_{n-1} (+) (... (x_1 (+) x_0)) in the trace's notation: "(a+b)" means dst = b, src = a."""
    s = f"x0@{off}"
    for k in range(1, n):
        s = f"(x{k}@{off}+{s})"
    return s


@pytest.mark.parametrize("alg", ROOT_COLLECTS)
@pytest.mark.parametrize("n", [2, 3, 5, 8])
def test_templates_on_the_one_sided_reduce_verbs_pass_the_check_and_fold_in_rank_order(plugin, alg, n):
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_check(True)
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        ins, outs = fake_ptrs(n)
        count = 1000
        for dtype, op in ((T.FP32, T.SUM), (T.FP32, T.PROD), (T.INT32, T.MAX)):
            for r in range(n):
                assert w.all_reduce(r, ins[r], outs[r], count, dtype, op, FAKE_STREAM) == 0, (alg, dtype, op)
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0, rep.firstProblem
            assert rep.reduces == n - 1                      # the root's fold, one step per peer
            rows = parse_trace(w.last_trace())
            assert sorted(r[0] for r in rows) == list(range(n))
            for rank, off, nbytes, expr in rows:
                assert (off, nbytes) == (0, 4 * count)
                if dtype == T.FP32:                          # integer folds are traced as the chain of their leaves
                    assert expr == chain(n), (rank, expr)
    finally:
        w.close()


def test_the_one_sided_templates_run_through_the_executor_chunk_loop(plugin):
    """A count beyond one scratch slot: the executor cuts it into loops and every piece is the same chain."""
    n, count = 3, 200000          # (n + 2) slots of the 1 MiB + 64 KiB buffer: 222822 bytes per loop
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_check(True)
        w.set_algorithm(api.CMD_ALLREDUCE, "ExampleAllReduceWriteReduce")
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_reduce(r, ins[r], outs[r], count, T.FP32, T.SUM, FAKE_STREAM) == 0
        assert w.last_check().semanticErrors == 0, w.last_check().firstProblem
        rows = parse_trace(w.last_trace())
        for rank in range(n):
            mine = sorted((off, nbytes, expr) for r, off, nbytes, expr in rows if r == rank)
            assert len(mine) > 1 and sum(b for _, b, _ in mine) == 4 * count
            at = 0
            for off, nbytes, expr in mine:
                assert off == at and expr == chain(n, off)
                at += nbytes
    finally:
        w.close()


def test_the_two_sided_batch_read_reduce_between_two_ranks(plugin):
    w = api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_check(True)
        w.set_algorithm(api.CMD_ALLREDUCE, "ExampleAllReducePairReadsEachOther")
        ins, outs = fake_ptrs(2)
        for r in range(2):
            assert w.all_reduce(r, ins[r], outs[r], 777, T.FP32, T.SUM, FAKE_STREAM) == 0
        rep = w.last_check()
        assert rep.races == 0 and rep.semanticErrors == 0 and rep.reduces == 2, rep.firstProblem
        rows = {r[0]: r[3] for r in parse_trace(w.last_trace())}
        assert rows == {0: "(x1@0+x0@0)", 1: "(x0@0+x1@0)"}
    finally:
        w.close()
    w = api.World(3, ccl_bytes=SMALL_CCL, dry=True)      # the template says it needs two ranks
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "ExampleAllReducePairReadsEachOther")
        ins, outs = fake_ptrs(3)
        assert [w.all_reduce(r, ins[r], outs[r], 10, T.FP32, T.SUM, FAKE_STREAM) for r in range(3)][-1] != 0
    finally:
        w.close()


def test_aicpu_reduce_rejects_the_types_the_reference_rejects(plugin):
    """AicpuReduce handles int8, int32, fp16, fp32, int64, uint64, fp64; anything else is HCCL_E_INTERNAL
    (alg_data_trans_wrapper.cc:1176-1207).  The entry point accepts int16 and bf16 SUM, so the error comes from the
    verb inside the template."""
    w = api.World(3, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "ExampleAllReduceReadThenAicpuReduce")
        ins, outs = fake_ptrs(3)
        for dtype in (T.INT16, T.BFP16):
            rcs = [w.all_reduce(r, ins[r], outs[r], 100, dtype, T.SUM, FAKE_STREAM) for r in range(3)]
            assert rcs[-1] == 4, (dtype, rcs)
        for dtype in (T.INT8, T.FP16, T.INT64, T.UINT64, T.FP64):
            rcs = [w.all_reduce(r, ins[r], outs[r], 100, dtype, T.SUM, FAKE_STREAM) for r in range(3)]
            assert rcs[-1] == 0, (dtype, rcs)
    finally:
        w.close()


# ---- read mode ----------------------------------------------------------------------------------------------------

def traced_world(n, link):
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    w.set_check(True)
    w.set_link_protocol(link)
    return w


def both_modes(n, call):
    """call(world) issues a collective on every rank; returns (trace, check report) per link protocol."""
    out = []
    for link in (api.LINK_HCCS, api.LINK_PCIE):
        w = traced_world(n, link)
        try:
            call(w)
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0, (link, rep.firstProblem)
            out.append((w.last_trace(), rep.steps, rep.copies, rep.reduces))
        finally:
            w.close()
    return out


@pytest.mark.parametrize("n", [2, 3, 5, 8, 12, 16])
def test_nhr_allreduce_in_read_mode_gives_the_same_expressions(n):
    ins, outs = fake_ptrs(n)

    def call(w):
        w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceNHR")
        for r in range(n):
            assert w.all_reduce(r, ins[r], outs[r], n * 1000 + 7, T.FP32, T.SUM, FAKE_STREAM) == 0
    (wt, ws, wc, wr), (rt, rs, rc, rr) = both_modes(n, call)
    assert rt == wt and (rs, rc, rr) == (ws, wc, wr)        # same steps, the other side issues them


@pytest.mark.parametrize("alg", ["InsReduceScatterNHR", "InsReduceScatterAicpuReduceNHR"])
@pytest.mark.parametrize("n", [2, 3, 5, 8, 12])
def test_nhr_reduce_scatter_in_read_mode_gives_the_same_expressions(alg, n):
    ins, outs = fake_ptrs(n)

    def call(w):
        w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
        for r in range(n):
            assert w.reduce_scatter(r, ins[r], outs[r], 1001, T.FP32, T.PROD, FAKE_STREAM) == 0    # one executor loop
    (wt, ws, wc, wr), (rt, rs, rc, rr) = both_modes(n, call)
    assert rt == wt and rr == wr
    if alg == "InsReduceScatterNHR" and n > 1:
        # write mode sends the shards of step 0 straight from the input; read mode has to stage them first
        sent_in_step0 = (n - 1 + 1) // 2
        assert rc == wc + n * sent_in_step0
    else:
        assert rc == wc


@pytest.mark.parametrize("n", [2, 3, 8, 13])
def test_nhr_allgather_in_read_mode_delivers_the_same(n):
    ins, outs = fake_ptrs(n)

    def call(w):
        w.set_algorithm(api.CMD_ALLGATHER, "InsAllGatherNHR")
        for r in range(n):
            assert w.all_gather(r, ins[r], outs[r], 4099, T.FP16, FAKE_STREAM) == 0
    (wt, ws, wc, _), (rt, rs, rc, _) = both_modes(n, call)
    assert rt == wt and (rs, rc) == (ws, wc)
    rows = parse_trace(rt)
    assert sorted({r[0] for r in rows}) == list(range(n))


@pytest.mark.parametrize("n", [2, 3, 5, 8, 17, 20])
def test_alltoallv_in_read_mode_permutes_as_the_contract_says(n):
    """Read mode packs every block into a slot of the SENDER's scratch buffer and the receiver fetches it straight
    into its output: one copy fewer per block than write mode does, the same bytes in the same places.  Among more
    than 17 ranks the peers take two rounds, the second of which packs per peer."""
    rng = np.random.default_rng(n)
    m = rng.integers(0, 40, size=(n, n)).tolist()
    m[0][n - 1] = 0                   # a pair that only moves data one way
    m[1 % n][0] = 0
    m[0][1 % n] = 0                   # and one that moves nothing
    if n == 8:
        m[3][5] = 90000               # one block larger than a scratch slot: several executor loops
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    ins, outs = fake_ptrs(n)

    def call(w):
        for r in range(n):
            sc, sd, rc, rd = v[r]
            assert w.all_to_all_v(r, ins[r], sc, sd, outs[r], rc, rd, T.FP32, FAKE_STREAM) == 0
    (wt, _, wc, _), (rt, _, rc, _) = both_modes(n, call)
    xs = [rng.integers(0, 2**32 - 1, size=max(1, sum(m[i])), dtype=np.uint32) for i in range(n)]
    want = T.run_alltoallv(xs, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                           [max(1, sum(x[2])) for x in v], fill=0xA5A5)
    for text in (wt, rt):
        got = [np.full(max(1, sum(x[2])), 0xA5A5, dtype=np.uint32) for x in v]
        for rank, off, nbytes, expr in parse_trace(text):
            tree = parse_expr(expr)
            assert tree[0] == "x"
            got[rank][off // 4:(off + nbytes) // 4] = xs[tree[1]][tree[2] // 4:(tree[2] + nbytes) // 4]
        for r in range(n):
            assert np.array_equal(got[r], want[r]), r
    assert rc == wc                    # pack + fetch against write + unpack: the same number of copy steps


def test_link_protocol_argument_is_checked():
    w = api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    try:
        with pytest.raises(_lib.HcclError) as e:
            w.set_link_protocol(7)
        assert e.value.code == 1
        w.set_link_protocol(api.LINK_ROCE)     # not PCIe: write mode
    finally:
        w.close()


def test_waits_take_the_explicit_timeout_when_the_default_form_is_switched_off():
    """The wrapper's waits use the *WithDefaultTimeout primitives and fall back to the explicit form
    (alg_data_trans_wrapper.cc:22-31); HCCL_VRANK_NO_DEFAULT_TIMEOUT=1 takes the fallback.  Both record the same
    schedule.  The switch is read once per process, so the fallback runs in a child process."""
    code = r'''
import sys
sys.path.insert(0, %r)
sys.path.insert(0, %r)
from hccl_amd import api
from host_util import FAKE_STREAM, fake_ptrs
w = api.World(5, ccl_bytes=%d, dry=True)
w.set_check(True)
w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceNHR")
ins, outs = fake_ptrs(5)
for r in range(5):
    assert w.all_reduce(r, ins[r], outs[r], 5007, 4, 0, FAKE_STREAM) == 0
rep = w.last_check()
assert rep.races == 0 and rep.semanticErrors == 0
sys.stdout.write(w.last_trace())
''' % (ROOT, os.path.join(ROOT, "tests"), SMALL_CCL)
    import sys
    texts = []
    for flag in ("0", "1"):
        env = dict(os.environ, HCCL_VRANK_NO_DEFAULT_TIMEOUT=flag)
        out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env)
        assert out.returncode == 0, out.stderr
        texts.append(out.stdout)
    assert texts[0] == texts[1] and texts[0].count("\n") >= 5
