"""Pins oracle/templates.py: the schedules must satisfy what the reference's semantics checkers demand
(every output element reduced from each rank exactly once, at the right offset), agree with plain numpy
folds wherever the operator is associative, reduce to a single pairwise op for two ranks, and show the
association orders the step formulas imply."""
import json
import math
import os

import re

import numpy as np
import pytest

from oracle import templates as T

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "st_cases.json")))
AR_ALGS = list(T.ALLREDUCE_TEMPLATES)
RS_ALGS = list(T.REDUCE_SCATTER_TEMPLATES)


def sym_inputs(n, count, tag_index=False):
    out = []
    for r in range(n):
        a = np.empty(count, dtype=object)
        a[:] = [f"x{r}[{i}]" if tag_index else f"x{r}" for i in range(count)]
        out.append(a)
    return out


def leaves(expr):
    return sorted(expr.replace("(", "").replace(")", "").split("+"))


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("n", [2, 3, 4, 5, 7, 8, 12, 13, 16])
def test_allreduce_every_element_reduces_every_rank_once_at_its_own_offset(alg, n):
    for count in (1, n - 1, n, 3 * n + 2):
        outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, count, True), count, 4, alg)
        for r in range(n):
            for i in range(count):
                assert leaves(outs[r][i]) == sorted(f"x{k}[{i}]" for k in range(n)), (alg, n, count, r, i)


@pytest.mark.parametrize("alg", RS_ALGS)
@pytest.mark.parametrize("n", [2, 3, 5, 8, 12])
def test_reduce_scatter_shard_offsets(alg, n):
    rc = 5
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc, True), rc, 2, alg)
    for r in range(n):
        for i in range(rc):
            assert leaves(outs[r][i]) == sorted(f"x{k}[{r * rc + i}]" for k in range(n))


@pytest.mark.parametrize("alg", AR_ALGS + RS_ALGS)
def test_two_ranks_is_one_pairwise_op(alg):
    if alg in T.ALLREDUCE_TEMPLATES:
        outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(2, 2), 2, 4, alg)
    else:
        outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(2, 2), 1, 4, alg)
    for o in outs:
        assert o[0] in ("(x0+x1)", "(x1+x0)")


def test_nhr_association_order_matches_hand_worked_shapes():
    for n_str, want in GOLD["nhr"]["slice0"].items():
        n = int(n_str)
        outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, n), n, 4, "InsAllReduceNHR")
        assert all(o[0] == want for o in outs)
        # other slices rotate the rank indices by the slice number
        for k in range(1, n):
            rot = want
            for r in reversed(range(n)):
                rot = rot.replace(f"x{r}+", f"y{(r + k) % n}+").replace(f"x{r})", f"y{(r + k) % n})")
            assert outs[0][k] == rot.replace("y", "x")
        rs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n), 1, 4, "InsReduceScatterNHR")
        assert rs[0][0] == want


def test_nhr_step_table_rank0_of_12():
    steps = T.nhr_rs_steps(12, 0)
    assert [{"to": s[0], "tx": s[2]} for s in steps] == GOLD["nhr"]["rank0_of_12_steps"]


@pytest.mark.parametrize("n", range(2, 65))
def test_nhr_closed_forms(n):
    ns = T.nhr_step_num(n)
    assert ns == math.ceil(math.log2(n))
    total = 0
    for s in range(ns):
        for r in range(n):
            to, frm, tx, rx = T.nhr_rs_steps(n, r)[s]
            assert to == (r - (1 << s)) % n and frm == (r + (1 << s)) % n
            assert not set(tx) & set(rx)                      # a step never sends what it receives
            assert T.nhr_rs_steps(n, to)[s][3] == tx          # the peer expects exactly these slices
            for k in tx:                                       # sender rule on d = (rank - slice) mod n
                d = (r - k) % n
                assert d % (1 << (s + 1)) == (1 << s)
            if r == 0:
                total += len(tx)
    assert total == n - 1
    have = {r: {r} for r in range(n)}                        # all-gather completeness
    for s in range(ns):
        new = {r: set(have[r]) for r in range(n)}
        for r in range(n):
            to, _, tx, _ = T.nhr_ag_steps(n, r)[s]
            assert set(tx) <= have[r]
            new[to] |= set(tx)
        have = new
    assert all(have[r] == set(range(n)) for r in range(n))


def test_self_first_orders():
    n = 5
    for alg in ("InsAllReduceMesh1DOneShot", "InsAllReduceAicpuReduceNHR"):
        outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, 1), 1, 4, alg)
        for r in range(n):
            want = f"x{r}"
            for k in range(n):
                if k != r:
                    want = f"(x{k}+{want})"
            assert outs[r][0] == want
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n), 1, 4, "InsReduceScatterMesh1D")
    assert outs[2][0] == "(x4+(x3+(x1+(x0+x2))))"
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, 1), 1, 4, "InsAllReduceMesh1DTwoShot")
    assert all(o[0] == "(x4+(x3+(x2+(x1+x0))))" for o in outs)


@pytest.mark.parametrize("count,n", [(0, 4), (1, 4), (3, 4), (4, 4), (5, 4), (17, 8), (1048576, 8), (100, 12)])
def test_split_data_tiles_the_range(count, n):
    sl = T.split_data(count, n)
    assert len(sl) == n
    off = 0
    short_seen = False
    full = -(-count // n)
    for o, c in sl:
        assert o == off
        off += c
        if short_seen:
            assert c == 0
        elif c < full:
            short_seen = True
    assert off == count


def test_chunk_sizes_of_the_default_scratch_buffer():
    ccl = T.CCL_BYTES_DEFAULT
    ch = T.chunk_counts(1 << 40, ccl - (1 << 20), 8, 1, ccl - (1 << 20))
    assert ch[0][1] == GOLD["chunks"]["reduce_scatter_mesh_n8"]
    ch = T.chunk_counts(1 << 30, ccl, 12, 1, ccl)
    assert ch[0][1] == GOLD["chunks"]["allreduce_aicpu_nhr_n12"] and len(ch) == 62
    assert len(T.chunk_counts(1 << 30, ccl, 1, 1, ccl)) == 6
    assert T.chunk_counts(1, ccl, 7, 1, ccl) == [(0, 1)]
    assert ccl // 7 // 128 * 128 == GOLD["chunks"]["alltoallv_mult7"]


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("dtype,op", [(T.INT32, T.SUM), (T.INT32, T.MAX), (T.INT64, T.MIN), (T.INT8, T.PROD),
                                      (T.UINT64, T.SUM), (T.INT16, T.SUM)])
def test_allreduce_integers_equal_numpy_fold_with_chunking(alg, dtype, op):
    rng = np.random.default_rng(1)
    npd = T.NP_STORAGE[dtype]
    ii = np.iinfo(npd)
    for n, count in ((3, 1000), (8, 777), (12, 4099)):
        xs = [rng.integers(ii.min, ii.max, size=count, dtype=npd, endpoint=True) for _ in range(n)]
        # a 4 KiB scratch buffer forces many executor chunks
        outs = T.run_allreduce(T.NumericElems(dtype, op), xs, count, T.DTYPE_SIZE[dtype], alg, ccl_bytes=4096)
        stack = np.stack(xs)
        with np.errstate(over="ignore"):
            want = {T.SUM: lambda: np.add.reduce(stack, 0, dtype=npd), T.PROD: lambda: np.multiply.reduce(stack, 0, dtype=npd),
                    T.MAX: lambda: stack.max(0), T.MIN: lambda: stack.min(0)}[op]()
        for o in outs:
            assert np.array_equal(o, want)


@pytest.mark.parametrize("alg", RS_ALGS)
def test_reduce_scatter_integers_equal_numpy_fold_with_chunking(alg):
    rng = np.random.default_rng(2)
    n, rc = 6, 1111
    xs = [rng.integers(-2**31, 2**31 - 1, size=n * rc, dtype=np.int32) for _ in range(n)]
    outs = T.run_reduce_scatter(T.NumericElems(T.INT32, T.SUM), xs, rc, 4, alg, ccl_bytes=(1 << 20) + 6 * 512)
    want = np.add.reduce(np.stack(xs), 0, dtype=np.int32)
    for r in range(n):
        assert np.array_equal(outs[r], want[r * rc:(r + 1) * rc])


def test_fp32_orders_differ_between_templates_and_between_ranks():
    rng = np.random.default_rng(3)
    n, count = 8, 4096
    xs = [(rng.random(count, dtype=np.float32) * 2 - 1) for _ in range(n)]
    one = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceMesh1DOneShot")
    two = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceMesh1DTwoShot")
    assert not np.array_equal(one[2].view(np.uint32), one[5].view(np.uint32))      # rank-dependent order
    assert all(np.array_equal(two[0].view(np.uint32), t.view(np.uint32)) for t in two)
    acc = xs[3].copy()                                                               # one-shot, rank 3, by hand
    for k in range(n):
        if k != 3:
            acc = xs[k] + acc
    assert np.array_equal(acc.view(np.uint32), one[3].view(np.uint32))


def scaled(matrix, div):
    return [[-(-c // div) for c in row] for row in matrix]


@pytest.mark.parametrize("case", GOLD["alltoallv"], ids=lambda c: c["name"])
def test_alltoallv_contract_on_reference_matrices(case):
    n = case["ranks"]
    m = scaled(case["matrix"], 1 << 19)      # counts divided by 2^19, rounded up: zeros stay zero
    rng = np.random.default_rng(n)
    ins = [rng.integers(0, 65535, size=sum(m[i]), dtype=np.uint16) for i in range(n)]
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    outs = T.run_alltoallv(ins, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                           [sum(x[2]) for x in v])
    for j in range(n):                          # element by element, straight from the API text
        pos = 0
        for i in range(n):
            start = sum(m[i][:j])
            for e in range(m[i][j]):
                assert outs[j][pos] == ins[i][start + e]
                pos += 1
        assert pos == len(outs[j])


@pytest.mark.parametrize("case", GOLD["allgatherv"], ids=lambda c: c["name"])
def test_allgatherv_contract_on_reference_lists(case):
    div = 1 << 12 if max(case["counts"]) > 100000 else 1
    counts = [-(-c // div) for c in case["counts"]]
    displs = [sum(counts[:i]) for i in range(len(counts))] if div > 1 else case["displs"]
    rng = np.random.default_rng(len(counts))
    ins = [rng.integers(0, 65535, size=c, dtype=np.uint16) for c in counts]
    outs = T.run_allgatherv(ins, counts, displs, displs[-1] + counts[-1], 0)
    for o in outs:
        assert np.array_equal(o, np.concatenate(ins))


DT_BY_NAME = {"int8": T.INT8, "int16": T.INT16, "int32": T.INT32, "fp16": T.FP16, "fp32": T.FP32}


def symbolic_inputs(n, length):
    out = []
    for r in range(n):
        a = np.empty(length, dtype=object)
        a[:] = [f"x{r}[{i}]" for i in range(length)]
        out.append(a)
    return out


@pytest.mark.parametrize("case", GOLD["reducescatterv"], ids=lambda c: c["name"])
@pytest.mark.parametrize("ccl", [T.CCL_BYTES_DEFAULT, 16 * 1024])
def test_reduce_scatter_v_on_reference_lists_satisfies_the_checker(case, ccl):
    """The predicates of reduce_scatter_v_semantics_checker.cc:17-95 on the symbolic run: output r is
    gap-free, every element reduces all N ranks exactly once, each taken at displs[r] + position; and the
    order is own rank first, then ranks ascending."""
    counts, displs = case["counts"], case["displs"]
    n = len(counts)
    esz = T.DTYPE_SIZE[DT_BY_NAME[case["dtype"]]]
    total = max(d + c for d, c in zip(displs, counts))
    outs = T.run_reduce_scatter_v(T.SymbolicElems(), symbolic_inputs(n, total), counts, displs, esz, ccl_bytes=ccl)
    for r in range(n):
        assert len(outs[r]) == counts[r]
        for t in (0, counts[r] // 2, counts[r] - 1):
            leaves = re.findall(r"x(\d+)\[(\d+)\]", outs[r][t])
            assert sorted(int(k) for k, _ in leaves) == list(range(n))
            assert all(int(i) == displs[r] + t for _, i in leaves)
            order = [r] + [k for k in range(n) if k != r]
            want = f"x{order[0]}[{displs[r] + t}]"
            for k in order[1:]:
                want = f"(x{k}[{displs[r] + t}]+{want})"
            assert outs[r][t] == want


def test_reduce_scatter_v_integers_equal_numpy_fold_with_ragged_chunks():
    rng = np.random.default_rng(17)
    counts = [5000, 0, 1, 4097, 333, 2048]
    displs, off = [], 3
    for c in counts:
        displs.append(off)
        off += c + 2
    n = len(counts)
    xs = [rng.integers(-2**31, 2**31 - 1, size=off, dtype=np.int32) for _ in range(n)]
    ccl = 6 * 4 * 1024                  # 1024 int32 per slot: the longest part takes 5 loops
    for op, fold in ((T.SUM, lambda a: a.sum(axis=0, dtype=np.int64).astype(np.int32)),
                     (T.MAX, lambda a: a.max(axis=0)), (T.MIN, lambda a: a.min(axis=0))):
        outs = T.run_reduce_scatter_v(T.NumericElems(T.INT32, op), xs, counts, displs, 4, ccl_bytes=ccl)
        for r in range(n):
            part = np.stack([x[displs[r]:displs[r] + counts[r]] for x in xs])
            assert np.array_equal(outs[r], fold(part)), (op, r)


def test_reduce_scatter_v_with_equal_counts_is_reduce_scatter():
    rng = np.random.default_rng(4)
    n, rc = 5, 777
    xs = [(rng.random(n * rc) * 2 - 1).astype(np.float32) for _ in range(n)]
    a = T.run_reduce_scatter_v(T.NumericElems(T.FP32, T.SUM), xs, [rc] * n, [r * rc for r in range(n)], 4)
    b = T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), xs, rc, 4, "InsReduceScatterMesh1D")
    for r in range(n):
        assert np.array_equal(a[r].view(np.uint32), b[r].view(np.uint32))


@pytest.mark.parametrize("alg", AR_ALGS)
def test_sampled_run_equals_dense_run_allreduce(alg):
    """SampledElems follows a template on a subset of the columns: it must give the dense run's values there,
    with executor chunks and ragged slices in play."""
    rng = np.random.default_rng(31)
    n, count, ccl = 12, 50021, 64 * 1024
    xs = [(0.9 + 0.2 * rng.random(count)).astype(np.float32) for _ in range(n)]
    dense = T.run_allreduce(T.NumericElems(T.FP32, T.PROD), xs, count, 4, alg, ccl_bytes=ccl)
    pos = np.unique(np.concatenate([rng.integers(0, count, 3000), np.arange(40), np.arange(count - 40, count)]))
    e = T.SampledElems(T.FP32, T.PROD)
    outs = T.run_allreduce(e, [e.sample(count, pos, x[pos]) for x in xs], count, 4, alg, ccl_bytes=ccl)
    for r in range(n):
        assert np.array_equal(outs[r].pos, pos)
        assert np.array_equal(outs[r].val.view(np.uint32), dense[r][pos].view(np.uint32)), (alg, r)


@pytest.mark.parametrize("alg", RS_ALGS)
def test_sampled_run_equals_dense_run_reduce_scatter(alg):
    rng = np.random.default_rng(32)
    n, rc, ccl = 5, 30011, 1024 * 1024 + 40 * 1024
    xs = [rng.standard_normal(n * rc).astype(np.float32) for _ in range(n)]
    dense = T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), xs, rc, 4, alg, ccl_bytes=ccl)
    pos = np.unique(rng.integers(0, n * rc, 5000))
    e = T.SampledElems(T.FP32, T.SUM)
    outs = T.run_reduce_scatter(e, [e.sample(n * rc, pos, x[pos]) for x in xs], rc, 4, alg, ccl_bytes=ccl)
    for r in range(n):
        mine = pos[(pos >= r * rc) & (pos < (r + 1) * rc)] - r * rc
        assert np.array_equal(outs[r].pos, mine)
        assert np.array_equal(outs[r].val.view(np.uint32), dense[r][mine].view(np.uint32)), (alg, r)


def test_moe_route_is_a_stable_grouping_brute_force():
    """Row of entry e = number of kept entries with a smaller destination + number of earlier kept entries with
    the same destination; tables follow from the counts (checked with plain loops on small inputs)."""
    rng = np.random.default_rng(41)
    for n, entries in ((1, 7), (3, 50), (8, 301), (5, 1)):
        dests = [rng.integers(-1, n + 1, size=entries) for _ in range(n)]       # -1 and n are dropped
        sc, sd, rc, rd, perms = T.moe_route(dests, n, 6)
        for i in range(n):
            d = dests[i]
            for e in range(entries):
                if d[e] < 0 or d[e] >= n:
                    assert perms[i][e] == T.MOE_DROPPED
                    continue
                smaller = sum(1 for x in d if 0 <= x < d[e])
                earlier = sum(1 for x in d[:e] if x == d[e])
                assert perms[i][e] == smaller + earlier
            for j in range(n):
                assert sc[i][j] == 6 * sum(1 for x in d if x == j)
                assert sd[i][j] == sum(sc[i][:j])
                assert rc[j][i] == sc[i][j]
                assert rd[j][i] == sum(sc[k][j] for k in range(i))


def test_moe_dispatch_alltoallv_and_back_is_the_identity():
    """pack -> AlltoAllV -> AlltoAllV with the tables of the way back -> combine(topk = 1) returns the tokens
    (dropped ones come back as zeros): ties the routing tables to run_alltoallv."""
    rng = np.random.default_rng(42)
    n, tokens, width = 4, 37, 8
    dests = [rng.integers(0, n + 1, size=tokens) for _ in range(n)]               # n = dropped
    toks = [rng.integers(0, 60000, size=(tokens, width)).astype(np.uint16) for _ in range(n)]
    sc, sd, rc, rd, perms = T.moe_route(dests, n, width)
    packed = [T.moe_pack(toks[i], perms[i], 1, max(1, sum(sc[i]) // width)).reshape(-1) for i in range(n)]
    recv = T.run_alltoallv(packed, sc, sd, rc, rd, [sum(rc[j]) for j in range(n)])
    back = T.run_alltoallv(recv, rc, rd, sc, sd, [sum(sc[i]) for i in range(n)])
    for i in range(n):
        rows = back[i].reshape(-1, width) if back[i].size else np.zeros((0, width), np.uint16)
        pad = np.zeros((max(1, rows.shape[0]), width), np.uint16)
        pad[:rows.shape[0]] = rows
        out = T.moe_combine(pad, perms[i], 1, T.BFP16)
        want = toks[i].copy()
        want[(dests[i] < 0) | (dests[i] >= n)] = 0
        assert np.array_equal(out, want)
    # what rank j receives from rank i are i's tokens for j, in token order
    for j in range(n):
        pos = 0
        for i in range(n):
            mine = toks[i][dests[i] == j].reshape(-1)
            assert np.array_equal(recv[j][pos:pos + mine.size], mine)
            pos += mine.size


def test_order_preserved_tree_is_the_same_on_every_rank():
    """Strict determinism: the association over the ranks' blocks does not depend on the rank that owns the
    shard.  Hand-worked from the fold rule (upper blocks onto block v % m): 8 ranks and 12 ranks."""
    want = {
        3: "(x1+(x2+x0))",
        8: "(((x7+x3)+(x5+x1))+((x6+x2)+(x4+x0)))",
    }
    for n in (3, 8):
        outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * 2), 2, 4, "ReduceScatterOrderPreserved")
        for r in range(n):
            assert outs[r][0] == want[n], (n, r, outs[r][0])
    # 12 ranks: blocks 8..11 fold onto 0..3 first, then 4..7 onto 0..3, then 2,3 onto 0,1, then 1 onto 0
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(12, 12), 1, 4, "ReduceScatterOrderPreserved")
    b = [f"x{k}" for k in range(12)]
    for v in range(8, 12):
        b[v - 8] = f"({b[v]}+{b[v - 8]})"
    for v in range(4, 8):
        b[v - 4] = f"({b[v]}+{b[v - 4]})"
    for v in range(2, 4):
        b[v - 2] = f"({b[v]}+{b[v - 2]})"
    b[0] = f"({b[1]}+{b[0]})"
    for r in range(12):
        assert outs[r][0] == b[0]


# ------------------------------------------------------------------------------------------------
# Association orders worked by hand from the sources named in tests/golden/st_cases.json
# ------------------------------------------------------------------------------------------------

def run_lengths(seq):
    out = []
    for x in seq:
        if out and out[-1][0] == x:
            out[-1][1] += 1
        else:
            out.append([x, 1])
    return [(a, b) for a, b in out]


@pytest.mark.parametrize("n", [3, 5, 8])
def test_ring_association_order_matches_the_hand_worked_chains(n):
    want = GOLD["ring"]["slices"][str(n)]
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, n), n, 4, "InsAllReduceRing")   # one element per slice
    for r in range(n):
        assert list(outs[r]) == want, (n, r)
    # ragged slices keep the order: 2n + 3 elements, slices of ceil(count / n)
    count = 2 * n + 3
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, count), count, 4, "InsAllReduceRing")
    per = -(-count // n)
    for r in range(n):
        for i in range(count):
            assert outs[r][i] == want[i // per], (n, r, i)


@pytest.mark.parametrize("n", [3, 5, 8])
def test_ring_fp32_equals_the_plain_chain_along_the_ring(n):
    """The closed form stated without the oracle's machinery: slice c = ((x_c + x_{c+1}) + x_{c+2}) + ... in fp32."""
    rng = np.random.default_rng(50 + n)
    count = 16 * n
    xs = [(rng.random(count, dtype=np.float32) * 2 - 1) for _ in range(n)]
    outs = T.run_allreduce(T.NumericElems(T.FP32, T.SUM), xs, count, 4, "InsAllReduceRing")
    for c in range(n):
        lo, hi = c * 16, (c + 1) * 16
        acc = xs[c][lo:hi].copy()
        for k in range(1, n):
            acc = acc + xs[(c + k) % n][lo:hi]
        for r in range(n):
            assert np.array_equal(outs[r][lo:hi].view(np.uint32), acc.view(np.uint32)), (n, c, r)


@pytest.mark.parametrize("n", [5, 12])
def test_rhd_association_order_matches_the_hand_worked_trees(n):
    want = GOLD["rhd"]["slices"][str(n)]
    extra, block = T.rhd_block(n)
    assert block == GOLD["rhd"]["block"][str(n)] and extra == n - len(block)
    p2 = len(want)
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, p2), p2, 4, "InsAllReduceRHD")  # one element per slice
    for r in range(n):
        assert list(outs[r]) == want, (n, r)


def test_rhd_fp32_of_five_ranks_equals_the_tree_written_out():
    rng = np.random.default_rng(55)
    xs = [(0.9 + 0.2 * rng.random(4)).astype(np.float32) for _ in range(5)]
    outs = T.run_allreduce(T.NumericElems(T.FP32, T.PROD), xs, 4, 4, "InsAllReduceRHD")
    a = xs[1] * xs[0]                 # rank 1 folded into rank 0
    want = [(xs[4] * xs[3]) * (xs[2] * a), (xs[2] * a) * (xs[4] * xs[3]), (xs[3] * xs[4]) * (a * xs[2]),
            (a * xs[2]) * (xs[3] * xs[4])]
    for r in range(5):
        for k in range(4):
            assert outs[r][k].view(np.uint32) == want[k][k].view(np.uint32), (r, k)


@pytest.mark.parametrize("n", [3, 4])
def test_mesh_chunk_rotation_matches_the_hand_worked_orders(n):
    want = GOLD["mesh_chunk"]["by_owner_chunk"][str(n)]
    parts = n - 1
    # ReduceScatter: one element per chunk of every shard
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * parts), parts, 4, "InsReduceScatterMesh1DMeshChunk")
    for f in range(n):
        assert list(outs[f]) == want[f], (n, f)
    # AllReduce: slice f = elements [f * parts, (f + 1) * parts), the same on every rank
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, n * parts), n * parts, 4, "InsAllReduceMesh1DTwoShotMeshChunk")
    flat = [s for f in range(n) for s in want[f]]
    for r in range(n):
        assert list(outs[r]) == flat, (n, r)


@pytest.mark.parametrize("case", GOLD["mesh_chunk"]["reduce_scatter_split"]["cases"],
                         ids=lambda c: "%dx%d" % (c["ranks"], c["recv_count"]))
def test_mesh_chunk_reduce_scatter_cuts_shards_at_4_kib(case):
    n, rc, esz = case["ranks"], case["recv_count"], case["esz"]
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc), rc, esz, "InsReduceScatterMesh1DMeshChunk")
    for f in range(n):
        assert [b for _, b in run_lengths(outs[f])] == case["chunk_elems"], (f, run_lengths(outs[f])[:4])
    assert sum(case["chunk_elems"]) == rc


@pytest.mark.parametrize("case", GOLD["mesh_chunk"]["all_reduce_split"]["cases"],
                         ids=lambda c: "%dx%d" % (c["ranks"], c["count"]))
def test_mesh_chunk_allreduce_cuts_slices_by_elements(case):
    n, count = case["ranks"], case["count"]
    assert [c for _, c in T.split_data(count, n)] == case["slice_elems"]
    outs = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, count), count, 4, "InsAllReduceMesh1DTwoShotMeshChunk")
    want = [c for row in case["chunk_elems"] for c in row if c]
    for r in range(n):
        assert [b for _, b in run_lengths(outs[r])] == want, r


@pytest.mark.parametrize("n", [3, 5])
def test_reduce_scatter_cpu_reduce_nhr_starts_from_the_own_shard(n):
    want = GOLD["reduce_scatter_aicpu_reduce_nhr"]["by_rank"][str(n)]
    outs = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * 2), 2, 8, "InsReduceScatterAicpuReduceNHR")
    for r in range(n):
        assert list(outs[r]) == [want[r]] * 2, (n, r)


def test_reference_system_test_tuples_are_well_formed():
    names = {"int8", "int16", "int32", "fp16", "fp32", "bfp16"}
    ar = GOLD["allreduce_st"]["cases"]
    assert len(ar) == 18 and all(c["dtype"] in names and c["op"] in ("sum", "max", "min") for c in ar)
    assert [c["count"] for c in ar if c["name"] == "2shot_upper_boundary_data"] == [32 * 1024 * 1024 - 1]
    rs = GOLD["reducescatter_st"]["cases"]
    assert len(rs) == 27 and all(c["dtype"] in names for c in rs)
    assert sum(next(c for c in rs if c["name"].startswith("nhr_asymmetric"))["servers"]) == 17
