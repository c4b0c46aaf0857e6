"""The host runtime without a GPU: op entry -> selector -> executor -> template -> recorded steps ->
dependency order -> symbolic trace.  The trace of every output is evaluated with the oracle's element
arithmetic and compared, bit for bit, with the oracle's own restatement of the same template."""
import json
import os

import numpy as np
import pytest

from oracle import templates as T
from hccl_amd import api

from host_util import (FAKE_STREAM, eval_expr, eval_trace, expr_to_oracle_string, fake_ptrs, parse_expr, parse_trace)

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "st_cases.json")))

SMALL_CCL = 1024 * 1024 + 64 * 1024     # forces several executor chunks at a few thousand elements
AR_ALGS = list(T.ALLREDUCE_TEMPLATES)
RS_ALGS = list(T.REDUCE_SCATTER_TEMPLATES)


def sym_inputs(n, count):
    out = []
    for r in range(n):
        a = np.empty(count, dtype=object)
        a[:] = [f"x{r}[{i}]" for i in range(count)]
        out.append(a)
    return out


def dry_allreduce(n, count, dtype, op, alg, ccl=SMALL_CCL):
    w = api.World(n, ccl_bytes=ccl, dry=True)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_reduce(r, ins[r], outs[r], count, dtype, op, FAKE_STREAM) == 0
        return w.last_trace(), w.last_info()
    finally:
        w.close()


def dry_reduce_scatter(n, recv_count, dtype, op, alg, ccl=SMALL_CCL):
    w = api.World(n, ccl_bytes=ccl, dry=True)
    try:
        w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.reduce_scatter(r, ins[r], outs[r], recv_count, dtype, op, FAKE_STREAM) == 0
        return w.last_trace(), w.last_info()
    finally:
        w.close()


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("n", [2, 3, 4, 5, 8, 12, 13])
def test_allreduce_association_order_equals_oracle(alg, n):
    for count in (1, n - 1, n, 2 * n + 3):
        text, _ = dry_allreduce(n, count, T.FP32, T.SUM, alg)
        want = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, count), count, 4, alg)
        seen = [set() for _ in range(n)]
        for rank, off, nbytes, expr in parse_trace(text):
            tree = parse_expr(expr)
            for e in range(nbytes // 4):
                idx = off // 4 + e
                assert expr_to_oracle_string(tree, e, 4, off) == want[rank][idx], (alg, n, count, rank, idx)
                seen[rank].add(idx)
        assert all(s == set(range(count)) for s in seen)      # every output element is produced


@pytest.mark.parametrize("alg", RS_ALGS)
@pytest.mark.parametrize("n", [2, 3, 5, 8, 12])
def test_reduce_scatter_association_order_equals_oracle(alg, n):
    rc = 7
    text, _ = dry_reduce_scatter(n, rc, T.BFP16, T.SUM, alg)
    want = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc), rc, 2, alg)
    seen = [set() for _ in range(n)]
    for rank, off, nbytes, expr in parse_trace(text):
        tree = parse_expr(expr)
        for e in range(nbytes // 2):
            assert expr_to_oracle_string(tree, e, 2, off) == want[rank][off // 2 + e]
            seen[rank].add(off // 2 + e)
    assert all(s == set(range(rc)) for s in seen)


def test_grouped_order_preserved_reduce_scatter_at_40_ranks():
    """More than 32 ranks: the all-to-all runs on 32 threads, shards leave by growing distance
    (ins_temp_reduce_scatter_order_preserved_group.cc:236-262); the tree is the one of the 32-rank template."""
    n, rc = 40, 3
    text, info = dry_reduce_scatter(n, rc, T.FP32, T.SUM, "ReduceScatterOrderPreservedGroup")
    want = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc), rc, 4, "ReduceScatterOrderPreservedGroup")
    plain = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc), rc, 4, "ReduceScatterOrderPreserved")
    seen = [set() for _ in range(n)]
    for rank, off, nbytes, expr in parse_trace(text):
        tree = parse_expr(expr)
        for e in range(nbytes // 4):
            assert expr_to_oracle_string(tree, e, 4, off) == want[rank][off // 4 + e] == plain[rank][off // 4 + e]
            seen[rank].add(off // 4 + e)
    assert all(s == set(range(rc)) for s in seen)


@pytest.mark.parametrize("alg", AR_ALGS)
@pytest.mark.parametrize("dtype,op,n,count", [(T.FP32, T.SUM, 8, 70001), (T.FP32, T.PROD, 12, 30011),
                                             (T.FP64, T.SUM, 5, 40000), (T.INT32, T.MAX, 12, 50000),
                                             (T.FP16, T.PROD, 3, 190001)])
def test_allreduce_values_with_executor_chunks(alg, dtype, op, n, count):
    """Several chunks of the small scratch buffer: slice boundaries move with the chunk, and so does the
    association tree an element sees."""
    rng = np.random.default_rng(n * 1000 + count)
    npd = T.NP_STORAGE[dtype]
    if dtype == T.INT32:
        xs = [rng.integers(-2**31, 2**31 - 1, size=count, dtype=np.int32) for _ in range(n)]
    elif dtype == T.FP16:
        xs = [T.narrow16((0.9 + 0.2 * rng.random(count)).astype(np.float32), T.FP16) for _ in range(n)]
    else:
        lo, hi = (0.9, 1.1) if op == T.PROD else (-1.0, 1.0)
        xs = [(lo + (hi - lo) * rng.random(count)).astype(npd) for _ in range(n)]
    esz = T.DTYPE_SIZE[dtype]
    text, _ = dry_allreduce(n, count, dtype, op, alg)
    got = eval_trace(text, xs, count, dtype, op, 0)
    want = T.run_allreduce(T.NumericElems(dtype, op), xs, count, esz, alg, ccl_bytes=SMALL_CCL)
    mult = T.ALLREDUCE_TEMPLATES[alg][1](n)
    if mult >= n:      # the slot-per-rank templates run several chunks at these sizes
        assert len(T.chunk_counts(count, SMALL_CCL, mult, esz, SMALL_CCL)) >= 2
    for r in range(n):
        assert np.array_equal(got[r].view(np.uint8), want[r].view(np.uint8)), (alg, r)


@pytest.mark.parametrize("alg", RS_ALGS)
def test_reduce_scatter_values_with_executor_chunks(alg):
    rng = np.random.default_rng(5)
    n, rc = 8, 9000          # (64 KiB usable scratch) / 8 slots = 8 KiB = 2048 fp32 per chunk
    xs = [(rng.random(n * rc) * 2 - 1).astype(np.float32) for _ in range(n)]
    text, _ = dry_reduce_scatter(n, rc, T.FP32, T.SUM, alg)
    got = eval_trace(text, xs, rc, T.FP32, T.SUM, 0)
    want = T.run_reduce_scatter(T.NumericElems(T.FP32, T.SUM), xs, rc, 4, alg, ccl_bytes=SMALL_CCL)
    assert len(T.chunk_counts(rc, SMALL_CCL - (1 << 20), n, 4, SMALL_CCL - (1 << 20))) == 5
    for r in range(n):
        assert np.array_equal(got[r].view(np.uint32), want[r].view(np.uint32))


def test_random_worlds_trace_equals_oracle():
    """Seeded random (ranks, count, element size, template) draws up to 48 ranks, odd counts included: what the
    recorded schedule computes for every output element is the oracle's expression, for AllReduce and
    ReduceScatter alike."""
    rng = np.random.default_rng(2024)
    for _ in range(60):
        n = int(rng.integers(1, 49))
        dtype = [T.FP32, T.BFP16, T.FP64][int(rng.integers(3))]
        esz = T.DTYPE_SIZE[dtype]
        if rng.integers(2):
            alg = AR_ALGS[int(rng.integers(len(AR_ALGS)))]
            count = int(rng.integers(1, 4 * n + 40))
            text, _ = dry_allreduce(n, count, dtype, T.SUM, alg)
            want = T.run_allreduce(T.SymbolicElems(), sym_inputs(n, count), count, esz, alg, ccl_bytes=SMALL_CCL)
            out_count = count
        else:
            alg = RS_ALGS[int(rng.integers(len(RS_ALGS)))]
            rc = int(rng.integers(1, 60))
            text, _ = dry_reduce_scatter(n, rc, dtype, T.SUM, alg)
            want = T.run_reduce_scatter(T.SymbolicElems(), sym_inputs(n, n * rc), rc, esz, alg, ccl_bytes=SMALL_CCL)
            out_count = rc
        seen = [set() for _ in range(n)]
        for rank, off, nbytes, expr in parse_trace(text):
            tree = parse_expr(expr)
            for e in range(nbytes // esz):
                idx = off // esz + e
                assert expr_to_oracle_string(tree, e, esz, off) == want[rank][idx], (alg, n, dtype, rank, idx)
                seen[rank].add(idx)
        if n > 1:
            assert all(s_ == set(range(out_count)) for s_ in seen), (alg, n, out_count)


def dry_reduce_scatter_v(counts, displs, dtype, op, ccl=SMALL_CCL):
    n = len(counts)
    w = api.World(n, ccl_bytes=ccl, dry=True)
    try:
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.reduce_scatter_v(r, ins[r], counts, displs, outs[r], counts[r], dtype, op, FAKE_STREAM) == 0
        return w.last_trace(), w.last_info()
    finally:
        w.close()


@pytest.mark.parametrize("case", GOLD["reducescatterv"], ids=lambda c: c["name"])
def test_reduce_scatter_v_reference_lists_trace_equals_oracle(case):
    """The reference's own ReduceScatterV shapes (reduce_scatter_v_testcase.cc:64-141): the traced
    expression of every output element is the oracle's, own rank first then ranks ascending."""
    counts, displs = case["counts"], case["displs"]
    dtype = {"int8": T.INT8, "int16": T.INT16, "int32": T.INT32, "fp16": T.FP16, "fp32": T.FP32}[case["dtype"]]
    esz = T.DTYPE_SIZE[dtype]
    n = len(counts)
    text, info = dry_reduce_scatter_v(counts, displs, dtype, T.SUM)
    assert info.algName.decode() == "InsReduceScatterVMesh1D" and info.fused == 1
    total = max(d + c for d, c in zip(displs, counts))
    want = T.run_reduce_scatter_v(T.SymbolicElems(), sym_inputs(n, total), counts, displs, esz, ccl_bytes=SMALL_CCL)
    seen = [0] * n
    for rank, off, nbytes, expr in parse_trace(text):
        tree = parse_expr(expr)
        for elem in (0, nbytes // esz - 1):
            assert expr_to_oracle_string(tree, elem, esz, off) == want[rank][off // esz + elem]
        seen[rank] += nbytes
    assert seen == [c * esz for c in counts]


def test_reduce_scatter_v_values_with_ragged_chunks_and_checks():
    rng = np.random.default_rng(23)
    counts = [120000, 0, 1, 60001, 333]       # scratch / 5 slots = 55,705 fp32 per loop: 3 loops
    displs, off = [], 1
    for c in counts:
        displs.append(off)
        off += c + 3
    n = len(counts)
    xs = [(rng.random(off) * 2 - 1).astype(np.float32) for _ in range(n)]
    text, _ = dry_reduce_scatter_v(counts, displs, T.FP32, T.SUM, ccl=SMALL_CCL)
    want = T.run_reduce_scatter_v(T.NumericElems(T.FP32, T.SUM), xs, counts, displs, 4, ccl_bytes=SMALL_CCL)
    got = [np.zeros(c, dtype=np.float32) for c in counts]
    for rank, o, nbytes, expr in parse_trace(text):
        got[rank][o // 4:(o + nbytes) // 4] = eval_expr(parse_expr(expr), xs, nbytes, T.FP32, T.SUM)
    for r in range(n):
        assert np.array_equal(got[r].view(np.uint32), want[r].view(np.uint32)), r
    # parameter checks (reduce_scatter_v_op.cc:142-167 and :49-66)
    w = api.World(3, ccl_bytes=SMALL_CCL, dry=True)
    try:
        ins, outs = fake_ptrs(3)
        c, d = [4, 4, 4], [0, 4, 8]
        assert w.reduce_scatter_v(0, ins[0], c, d, outs[0], 4, T.FP32, T.SUM, 0) == 2             # null stream
        assert w.reduce_scatter_v(0, ins[0], c, d, 0, 4, T.FP32, T.SUM, FAKE_STREAM) == 2         # null recvBuf
        assert w.reduce_scatter_v(0, ins[0], [0, 0, 0], d, 0, 0, T.FP32, T.SUM, FAKE_STREAM) == 0  # nothing to do
        assert w.reduce_scatter_v(0, ins[0], c, d, outs[0], 4, T.UINT8, T.SUM, FAKE_STREAM) == 5   # not a reduce type
        assert w.reduce_scatter_v(0, ins[0], c, d, outs[0], 4, T.BFP16, T.PROD, FAKE_STREAM) == 5  # PROD on bf16
        assert w.reduce_scatter_v(0, ins[0], c, d, outs[0], 5, T.FP32, T.SUM, FAKE_STREAM) == 1    # recvCount != counts[rank]
        # uint64 / fp64 have no algorithm in the AICPU branch: the selector finds no match
        for r in range(3):
            rc = w.reduce_scatter_v(r, ins[r], c, d, outs[r], 4, T.FP64, T.SUM, FAKE_STREAM)
        assert rc == 5
    finally:
        w.close()


def test_mesh_chunk_rotation_and_4k_chunks():
    """Chunk i of rank f's shard takes f's own data, then the ranks f+i+1, f+i+2, ... (wrapping, skipping f);
    with a shard of 20,000 bytes on 4 ranks the chunks are 4096, 4096 and 11,808 bytes."""
    n, rc = 4, 5000
    text, info = dry_reduce_scatter(n, rc, T.FP32, T.SUM, "InsReduceScatterMesh1DMeshChunk")
    assert info.fused == 1
    pieces = {}
    for rank, off, nbytes, expr in parse_trace(text):
        pieces.setdefault(rank, []).append((off, nbytes, expr))
    for f in range(n):
        got = sorted(pieces[f])
        assert [(o, b) for o, b, _ in got] == [(0, 4096), (4096, 4096), (8192, 11808)]
        for i, (off, _, expr) in enumerate(got):
            order = [f] + [(f + i + 1 + s + (1 if i + 1 + s >= n else 0)) % n for s in range(n - 1)]
            want = f"x{order[0]}@{f * rc * 4 + off}"
            for k in order[1:]:
                want = f"(x{k}@{f * rc * 4 + off}+{want})"
            assert expr == want
    # AllReduce: first level ceil(count / N), second level N-1 even chunks, same rotation
    text, info = dry_allreduce(5, 1003, T.FP32, T.SUM, "InsAllReduceMesh1DTwoShotMeshChunk")
    assert info.fused == 1
    want = T.run_allreduce(T.SymbolicElems(), sym_inputs(5, 1003), 1003, 4, "InsAllReduceMesh1DTwoShotMeshChunk",
                           ccl_bytes=SMALL_CCL)
    for rank, off, nbytes, expr in parse_trace(text):
        tree = parse_expr(expr)
        for elem in (0, nbytes // 4 - 1):
            assert expr_to_oracle_string(tree, elem, 4, off) == want[rank][off // 4 + elem]


def test_which_templates_fuse():
    """Chains, every integer schedule and floating-point trees of up to four levels become fused passes."""
    for alg, dtype, fused in [("InsAllReduceMesh1DOneShot", T.FP32, 1), ("InsAllReduceMesh1DTwoShot", T.FP32, 1),
                              ("InsAllReduceAicpuReduceNHR", T.FP32, 1), ("InsAllReduceRing", T.FP32, 1),
                              ("InsAllReduceNHR", T.FP32, 1), ("InsAllReduceRHD", T.FP32, 1),
                              ("InsAllReduceNHR", T.INT32, 1), ("InsAllReduceRHD", T.INT32, 1)]:
        _, info = dry_allreduce(12, 1200, dtype, T.SUM, alg)
        assert info.fused == fused, alg
        assert info.algName.decode() == alg
    # the one-shot order of all 12 ranks is one segment: 12 sources read once, 12 outputs
    _, info = dry_allreduce(12, 1200, T.FP32, T.SUM, "InsAllReduceMesh1DOneShot")
    assert info.fusedSegments == 1
    # float max keeps operand order: the ring's "acc (+) leaf" steps stay a chain whose marked steps swap their
    # operands, among any number of ranks
    _, info = dry_allreduce(4, 64, T.FP32, T.MAX, "InsAllReduceRing")
    assert info.fused == 1
    _, info = dry_allreduce(12, 1200, T.FP32, T.MAX, "InsAllReduceRing")
    assert info.fused == 1
    _, info = dry_allreduce(40, 4000, T.FP32, T.MIN, "InsAllReduceRing")
    assert info.fused == 1


def test_selector_choices_follow_the_reference_thresholds():
    def pick(n, count, dtype, op, topo=None, cmd="ar"):
        # the default 200 MiB scratch for large counts: a small one would mean thousands of executor loops
        w = api.World(n, ccl_bytes=SMALL_CCL if count < (1 << 22) else 0, dry=True)
        try:
            if topo:
                w.set_topo(*topo)
            ins, outs = fake_ptrs(n)
            for r in range(n):
                if cmd == "ar":
                    assert w.all_reduce(r, ins[r], outs[r], count, dtype, op, FAKE_STREAM) == 0
                elif cmd == "rs":
                    assert w.reduce_scatter(r, ins[r], outs[r], count, dtype, op, FAKE_STREAM) == 0
                elif cmd == "a2a":
                    assert w.all_to_all(r, ins[r], count, outs[r], dtype, FAKE_STREAM) == 0
                else:
                    assert w.all_gather(r, ins[r], outs[r], count, dtype, FAKE_STREAM) == 0
            return w.last_info().algName.decode()
        finally:
            w.close()

    mib = 1 << 20
    assert pick(8, 8 * mib // 4, T.FP32, T.SUM) == "InsAllReduceMesh1DOneShot"          # <= 8 MiB
    # size * 8 / N^2 > 32 MiB: the chunked two-shot (all_reduce_auto_selector.cc:485-487)
    assert pick(8, 256 * mib // 4, T.FP32, T.SUM) == "InsAllReduceMesh1DTwoShot"
    assert pick(8, 256 * mib // 4 + 1, T.FP32, T.SUM) == "InsAllReduceMesh1DTwoShotMeshChunk"
    assert pick(4, 64 * mib // 4 + 1, T.FP32, T.SUM) == "InsAllReduceMesh1DTwoShotMeshChunk"
    assert pick(8, 512 * mib // 8, T.FP64, T.SUM) == "InsAllReduceMesh1DTwoShot"        # 64-bit types never
    # shard * (8/N)^2 > 16 MiB: the chunked mesh ReduceScatter (reduce_scatter_auto_selector.cc:383-408)
    assert pick(8, 16 * mib // 2, T.BFP16, T.SUM, cmd="rs") == "InsReduceScatterMesh1D"
    assert pick(8, 16 * mib // 2 + 1, T.BFP16, T.SUM, cmd="rs") == "InsReduceScatterMesh1DMeshChunk"
    assert pick(16, 16 * mib // 2 + 1, T.BFP16, T.SUM, cmd="rs") == "InsReduceScatterMesh1D"
    assert pick(8, 64 * mib // 4, T.FP32, T.PROD, cmd="rs") == "InsReduceScatterMesh1D"
    assert pick(8, 8 * mib // 4 + 1, T.FP32, T.SUM) == "InsAllReduceMesh1DTwoShot"
    assert pick(8, 1024, T.FP32, T.PROD) == "InsAllReduceMesh1DOneShot"
    assert pick(8, 8 * mib // 8 + 1, T.FP64, T.SUM) == "InsAllReduceMesh1DTwoShot"
    # 12 single-device servers: the log-step family; PROD / 64-bit types reduce after an NHR gather
    assert pick(12, 4096, T.INT32, T.MAX, topo=(2, api.SHAPE_MESH_1D, 1)) == "InsAllReduceNHR"
    assert pick(12, 4096, T.FP32, T.PROD, topo=(2, api.SHAPE_MESH_1D, 1)) == "InsAllReduceAicpuReduceNHR"
    assert pick(12, 4096, T.FP32, T.SUM, topo=(1, api.SHAPE_CLOS, 0)) == "InsAllReduceNHR"
    assert pick(8, 4096, T.BFP16, T.SUM, cmd="rs") == "InsReduceScatterMesh1D"
    assert pick(8, 4096, T.BFP16, T.SUM, topo=(2, api.SHAPE_MESH_1D, 1), cmd="rs") == "InsReduceScatterNHR"
    # reduce_scatter_auto_selector.cc:350-352, :429-431
    assert pick(8, 4096, T.FP32, T.PROD, topo=(2, api.SHAPE_MESH_1D, 1), cmd="rs") == "InsReduceScatterAicpuReduceNHR"
    assert pick(6, 4096, T.INT64, T.SUM, topo=(1, api.SHAPE_CLOS, 0), cmd="rs") == "InsReduceScatterAicpuReduceNHR"
    assert pick(8, 4096, T.FP16, None, cmd="ag") == "InsAllGatherMesh1D"
    # one link per pair up to 150 MiB per rank (alltoall_auto_selector.cc:127-135)
    assert pick(8, 150 * mib // 8 // 2, T.FP16, None, cmd="a2a") == "InsAlltoAllMesh1DSingleChannel"
    assert pick(8, 150 * mib // 8 // 2 + 1, T.FP16, None, cmd="a2a") == "InsAlltoAllMesh1D"
    assert pick(8, 4096, T.FP16, None, topo=(1, api.SHAPE_CLOS, 0), cmd="ag") == "InsAllGatherNHR"


def test_parameter_checks_and_early_returns():
    w = api.World(4, ccl_bytes=SMALL_CCL, dry=True)
    ins, outs = fake_ptrs(4)
    try:
        assert w.all_reduce(0, ins[0], outs[0], 0, T.FP32, T.SUM, FAKE_STREAM) == 0          # count 0: success, nothing queued
        assert w.all_reduce(0, ins[0], outs[0], 8, T.FP32, T.SUM, None) == 2                 # null stream: HCCL_E_PTR
        assert w.all_reduce(0, None, outs[0], 8, T.FP32, T.SUM, FAKE_STREAM) == 2
        assert w.all_reduce(0, ins[0], outs[0], 0x800000000, T.FP32, T.SUM, FAKE_STREAM) == 1   # > SYS_MAX_COUNT
        assert w.all_reduce(0, ins[0], outs[0], 8, T.UINT8, T.SUM, FAKE_STREAM) == 5         # not a reduce type
        assert w.all_reduce(0, ins[0], outs[0], 8, T.BFP16, T.PROD, FAKE_STREAM) == 5        # PROD excludes bf16
        assert w.all_reduce(0, ins[0], outs[0], 8, T.INT16, T.PROD, FAKE_STREAM) == 5
        assert w.reduce_scatter(0, ins[0], outs[0], 8, T.UINT32, T.SUM, FAKE_STREAM) == 5
        assert w.all_gather(0, ins[0], outs[0], 8, 12, FAKE_STREAM) == 5                     # int128
        assert w.all_to_all_v(0, ins[0], [1] * 4, [0] * 4, ins[0], [1] * 4, [0] * 4, T.INT8, FAKE_STREAM) == 1  # in place
        assert w.all_to_all_v(0, None, [1] * 4, [0] * 4, outs[0], [1] * 4, [0] * 4, T.INT8, FAKE_STREAM) == 2
        assert w.all_gather_v(0, ins[0], 3, outs[0], [0] * 4, [0] * 4, T.FP16, FAKE_STREAM) == 0   # all counts 0
        assert w.all_gather_v(0, ins[0], 3, None, [3, 1, 1, 1], [0, 3, 4, 5], T.FP16, FAKE_STREAM) == 2
    finally:
        w.close()


def test_ranks_that_disagree_are_rejected():
    w = api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    ins, outs = fake_ptrs(2)
    try:
        assert w.all_reduce(0, ins[0], outs[0], 8, T.FP32, T.SUM, FAKE_STREAM) == 0
        assert w.all_reduce(1, ins[1], outs[1], 9, T.FP32, T.SUM, FAKE_STREAM) == 1   # HCCL_E_PARA
    finally:
        w.close()


def test_single_rank_world_is_a_local_copy():
    w = api.World(1, ccl_bytes=SMALL_CCL, dry=True)
    ins, outs = fake_ptrs(1)
    try:
        assert w.all_reduce(0, ins[0], outs[0], 8, T.FP32, T.SUM, FAKE_STREAM) == 0
        assert w.all_reduce(0, ins[0], ins[0], 8, T.FP32, T.SUM, FAKE_STREAM) == 0    # in place: nothing to do
    finally:
        w.close()


def test_calls_queue_per_rank_and_pair_up_in_order():
    """Rank 0 may run ahead: its second call waits in its queue until rank 1 has made both calls."""
    w = api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    ins, outs = fake_ptrs(2)
    try:
        assert w.all_reduce(0, ins[0], outs[0], 8, T.FP32, T.SUM, FAKE_STREAM) == 0
        assert w.all_reduce(0, ins[0], outs[0], 16, T.INT32, T.MAX, FAKE_STREAM) == 0
        assert w.all_reduce(1, ins[1], outs[1], 8, T.FP32, T.SUM, FAKE_STREAM) == 0
        assert "out[0,32)" in w.last_trace()
        assert w.all_reduce(1, ins[1], outs[1], 16, T.INT32, T.MAX, FAKE_STREAM) == 0
        assert "out[0,64)" in w.last_trace()
    finally:
        w.close()


# ---- data movement: the traced schedule must be the API contract ---------------------------------

def copy_trace_outputs(text, inputs, out_lens, esz):
    fill = 0xA5A5 & int(np.iinfo(inputs[0].dtype).max)
    outs = [np.full(l, fill, dtype=inputs[0].dtype) for l in out_lens]
    for rank, off, nbytes, expr in parse_trace(text):
        tree = parse_expr(expr)
        assert tree[0] == "x", "a data-movement collective must not reduce"
        _, k, b = tree
        outs[rank][off // esz:(off + nbytes) // esz] = inputs[k][b // esz:(b + nbytes) // esz]
    return outs


@pytest.mark.parametrize("alg", ["InsAllGatherMesh1D", "InsAllGatherNHR"])
@pytest.mark.parametrize("n,count", [(2, 5), (3, 1000), (8, 33), (12, 70000), (16, 9)])
def test_allgather_templates_deliver_the_concatenation(alg, n, count):
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_algorithm(api.CMD_ALLGATHER, alg)
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_gather(r, ins[r], outs[r], count, T.FP16, FAKE_STREAM) == 0
        rng = np.random.default_rng(n)
        xs = [rng.integers(0, 65535, size=count, dtype=np.uint16) for _ in range(n)]
        got = copy_trace_outputs(w.last_trace(), xs, [n * count] * n, 2)
        for r in range(n):
            assert np.array_equal(got[r], np.concatenate(xs))
    finally:
        w.close()


@pytest.mark.parametrize("counts", [[3, 0, 7, 1], [100, 100, 100, 100], [0, 0, 5], [70000, 1, 0, 33000, 12, 9, 400, 8],
                                    [700, 700, 600, 600, 500, 500, 400, 400, 300, 300, 200, 200, 100, 100]])
def test_allgatherv_template_with_ragged_counts_and_chunks(counts):
    n = len(counts)
    displs, off = [], 2
    for c in counts:
        displs.append(off)
        off += c + 1                      # one element of slack between blocks: it must stay untouched
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_gather_v(r, ins[r], counts[r], outs[r], counts, displs, T.FP16, FAKE_STREAM) == 0
        assert w.last_info().algName.decode() == "InsAllGatherVMesh1D"
        rng = np.random.default_rng(n)
        xs = [rng.integers(0, 65535, size=max(c, 1), dtype=np.uint16) for c in counts]
        got = copy_trace_outputs(w.last_trace(), xs, [off] * n, 2)
        want = T.run_allgatherv(xs, counts, displs, off, 0xA5A5)
        for r in range(n):
            assert np.array_equal(got[r], want[r]), r
    finally:
        w.close()


def a2a_tables(m):
    n = len(m)
    return [T.alltoallvc_to_v(m, r) for r in range(n)]


@pytest.mark.parametrize("n", [2, 3, 5, 8, 17, 20])
def test_alltoallv_template_permutes_as_the_contract_says(n):
    rng = np.random.default_rng(n)
    m = rng.integers(0, 40, size=(n, n)).tolist()
    m[0][n - 1] = 0
    m[n - 1][0] = 0
    if n == 8:
        m[3][5] = 90000                   # one block larger than a scratch slot: several executor loops
    v = a2a_tables(m)
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        ins, outs = fake_ptrs(n)
        for r in range(n):
            sc, sd, rc, rd = v[r]
            assert w.all_to_all_v(r, ins[r], sc, sd, outs[r], rc, rd, T.FP32, FAKE_STREAM) == 0
        xs = [rng.integers(0, 2**32 - 1, size=max(1, sum(m[i])), dtype=np.uint32) for i in range(n)]
        got = copy_trace_outputs(w.last_trace(), xs, [max(1, sum(x[2])) for x in v], 4)
        want = T.run_alltoallv(xs, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                               [max(1, sum(x[2])) for x in v], fill=0xA5A5)
        for r in range(n):
            assert np.array_equal(got[r][:sum(v[r][2])], want[r][:sum(v[r][2])]), r
    finally:
        w.close()


def test_alltoall_and_alltoallvc_reduce_to_alltoallv():
    n, c = 4, 6
    rng = np.random.default_rng(1)
    xs = [rng.integers(0, 255, size=n * c, dtype=np.uint8) for _ in range(n)]
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_to_all(r, ins[r], c, outs[r], T.UINT8, FAKE_STREAM) == 0
        assert w.last_info().algName.decode() == "InsAlltoAllMesh1DSingleChannel"   # <= 150 MiB per rank
        got = copy_trace_outputs(w.last_trace(), xs, [n * c] * n, 1)
        for j in range(n):
            assert np.array_equal(got[j], np.concatenate([xs[i][j * c:(j + 1) * c] for i in range(n)]))
        m = [[1, 2, 0, 3], [4, 0, 1, 1], [2, 2, 2, 0], [0, 5, 1, 1]]
        flat = [x for row in m for x in row]
        for r in range(n):
            assert w.all_to_all_vc(r, ins[r], flat, outs[r], T.UINT8, FAKE_STREAM) == 0
        assert w.last_info().algName.decode() == "InsAlltoAllVCMesh1D"
        v = a2a_tables(m)
        got = copy_trace_outputs(w.last_trace(), xs, [sum(x[2]) for x in v], 1)
        want = T.run_alltoallv(xs, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                               [sum(x[2]) for x in v])
        for r in range(n):
            assert np.array_equal(got[r], want[r])
    finally:
        w.close()


def test_alltoallv_count_mismatch_between_ranks_is_rejected():
    w = api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    ins, outs = fake_ptrs(2)
    try:
        assert w.all_to_all_v(0, ins[0], [1, 2], [0, 1], outs[0], [1, 3], [0, 1], T.INT8, FAKE_STREAM) == 0
        # rank 1 expects 4 elements from rank 0, which sends 2
        assert w.all_to_all_v(1, ins[1], [3, 1], [0, 3], outs[1], [4, 1], [0, 4], T.INT8, FAKE_STREAM) == 1
    finally:
        w.close()


def test_one_host_thread_per_rank_meets_at_every_collective():
    """The reference's test style (one host thread per rank, all_reduce_testcase.cc:73-107) on a world without a
    device: in blocking mode a call returns when the last rank has arrived, whatever the order of arrival, and a
    thread that runs ahead queues its next collective behind the one in flight."""
    import threading
    n, rounds = 8, 40
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_blocking(True)
        ins, outs = fake_ptrs(n)
        rcs = [[] for _ in range(n)]

        def body(r):
            for k in range(rounds):
                if k % 2 == 0:
                    rcs[r].append(w.all_reduce(r, ins[r], outs[r], 100 + k, T.FP32, T.SUM, FAKE_STREAM))
                else:
                    rcs[r].append(w.reduce_scatter(r, ins[r], outs[r], 10 + k, T.INT32, T.MAX, FAKE_STREAM))

        ts = [threading.Thread(target=body, args=(r,)) for r in range(n)]
        for t in ts:
            t.start()
        for t in ts:
            t.join(timeout=60)
        assert all(not t.is_alive() for t in ts)
        assert rcs == [[0] * rounds for _ in range(n)]
        assert w.last_info().algName.decode().startswith("InsReduceScatter")
    finally:
        w.close()


def traced(n, call, closed_form):
    """Trace text and op info of one dry collective; `call(world, rank, in, out)` issues a rank's call."""
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_closed_form(closed_form)
        return call(w), w.last_info()
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 3, 4, 5, 7, 8, 12, 16, 17, 31, 32])
@pytest.mark.parametrize("kind", ["all_reduce", "reduce_scatter", "reduce_scatter_gather", "all_reduce_one_shot",
                                  "all_reduce_two_shot", "reduce_scatter_mesh", "all_reduce_gather", "all_reduce_ring",
                                  "all_reduce_nhr", "reduce_scatter_nhr", "all_reduce_rhd", "reduce_scatter_ordered",
                                  "reduce_scatter_ordered_group"])
def test_closed_form_of_a_template_equals_its_recorded_steps(kind, n):
    """The mesh-chunk templates and the gather-then-fold ReduceScatter state their result directly (N (N-1) chains,
    N chains) so that a world need not record, order and trace their N^3 steps; the one-shot, two-shot and mesh
    ReduceScatter templates (N^2 steps, N chains) do the same.  The statement must be exactly what the steps amount to: line for line the same
    trace -- same pieces, same association order -- for short, ragged, 4 KiB-aligned and multi-chunk operands, every
    element size, and in place."""
    alg = {"all_reduce": "InsAllReduceMesh1DTwoShotMeshChunk", "reduce_scatter": "InsReduceScatterMesh1DMeshChunk",
           "reduce_scatter_gather": "InsReduceScatterAicpuReduceNHR", "all_reduce_one_shot": "InsAllReduceMesh1DOneShot",
           "all_reduce_two_shot": "InsAllReduceMesh1DTwoShot", "reduce_scatter_mesh": "InsReduceScatterMesh1D",
           "all_reduce_gather": "InsAllReduceAicpuReduceNHR", "all_reduce_ring": "InsAllReduceRing",
           "all_reduce_nhr": "InsAllReduceNHR", "reduce_scatter_nhr": "InsReduceScatterNHR",
           "all_reduce_rhd": "InsAllReduceRHD", "reduce_scatter_ordered": "ReduceScatterOrderPreserved",
           "reduce_scatter_ordered_group": "ReduceScatterOrderPreservedGroup"}[kind]
    reduces_all = kind.startswith("all_reduce")
    cmd = api.CMD_ALLREDUCE if reduces_all else api.CMD_REDUCE_SCATTER
    ins, outs = fake_ptrs(n)
    # per-rank received count for ReduceScatter; several executor chunks at the last sizes
    # (the ReduceScatter template takes N-1 scratch slots per chunk, so its chunks are short among many ranks)
    counts = [1, max(1, n - 1), n, n * (n - 1) + 1, 4099] + ([70001] if n <= 12 or reduces_all else [])
    counts += [300001] if n <= 8 else []
    for count in counts:
        for dtype in (T.INT8, T.FP32, T.FP64):
            for in_place in (False, True):
                if not reduces_all and in_place:
                    continue   # a ReduceScatter's output is a part of its input: not apart, never in closed form
                if (dtype != T.FP32 or in_place) and count not in (n, 4099, counts[-1]):
                    continue

                def call(w):
                    w.set_algorithm(cmd, alg)
                    for r in range(n):
                        dst = ins[r] if in_place else outs[r]
                        if reduces_all:
                            assert w.all_reduce(r, ins[r], dst, count, dtype, T.SUM, FAKE_STREAM) == 0
                        else:
                            assert w.reduce_scatter(r, ins[r], dst, count, dtype, T.SUM, FAKE_STREAM) == 0
                    return w.last_trace()

                recorded, info_r = traced(n, call, 0)
                closed, info_c = traced(n, call, 2)
                assert info_r.levels > 0 and info_c.levels == 0, "the closed form was not used"
                assert closed == recorded, f"{alg} n={n} count={count} dtype={dtype} in_place={in_place}"
                assert info_c.fused == info_r.fused == 1 and info_c.fusedSegments == info_r.fusedSegments


@pytest.mark.parametrize("n", [2, 3, 5, 8, 12, 17, 32, 64])
def test_closed_form_of_reduce_scatter_v_equals_its_recorded_steps(n):
    """The ragged mesh ReduceScatter states its result too: per executor loop, every rank whose part has not run out
    gets its part of its own input with the other ranks' reduced onto it, ranks ascending.  Ragged parts with zeros,
    parts at scattered places of the input, one and several executor loops, three element sizes."""
    rng = np.random.default_rng(n)
    ins, outs = fake_ptrs(n)
    for top in (7, 3000, 40000 if n <= 17 else 9000):
        counts = [int(c) for c in rng.integers(0, top, size=n)]
        counts[int(rng.integers(n))] = 0
        counts[int(rng.integers(n))] = top              # at least one part, and the longest takes several loops
        displs, at = [0] * n, 3
        for i in rng.permutation(n):
            displs[i] = at
            at += counts[i] + int(rng.integers(5))
        for dtype in (T.INT8, T.FP32, T.INT64):
            if dtype != T.FP32 and top != 3000:
                continue

            def call(w):
                for r in range(n):
                    assert w.reduce_scatter_v(r, ins[r], counts, displs, outs[r], counts[r], dtype, T.SUM, FAKE_STREAM) == 0
                return w.last_trace()

            recorded, info_r = traced(n, call, 0)
            closed, info_c = traced(n, call, 2)
            assert info_r.levels > 0 and info_c.levels == 0, "the closed form was not used"
            assert closed == recorded, f"n={n} counts={counts} displs={displs} dtype={dtype}"
            assert info_c.fused == info_r.fused == 1 and info_c.fusedSegments == info_r.fusedSegments


def test_closed_form_among_64_ranks_and_when_it_is_not_used():
    alg = "InsAllReduceMesh1DTwoShotMeshChunk"
    n, count = 64, 64 * 63 * 2 + 5
    ins, outs = fake_ptrs(n)

    def call(w, alg=alg, srcs=ins):
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        for r in range(n):
            assert w.all_reduce(r, srcs[r], outs[r], count, T.FP32, T.SUM, FAKE_STREAM) == 0
        return w.last_trace()

    recorded, info_r = traced(n, call, 0)
    closed, info_c = traced(n, call, 2)
    assert closed == recorded and info_c.levels == 0 and info_r.levels > 0
    assert info_c.fused == 1 and info_c.fusedSegments == info_r.fusedSegments == 64 * 63
    # the log-step templates, whose results are trees of six levels here
    for tree_alg in ("InsAllReduceNHR", "InsAllReduceRHD"):
        rec, info_rec = traced(n, lambda w: call(w, alg=tree_alg), 0)
        clo, info_clo = traced(n, lambda w: call(w, alg=tree_alg), 2)
        assert clo == rec and info_clo.levels == 0 and info_rec.levels > 0, tree_alg
        assert info_clo.fused == info_rec.fused == 1 and info_clo.fusedSegments == info_rec.fusedSegments
    # two ranks share an input buffer: the buffers do not lie apart, so the steps are recorded
    shared = [ins[0]] + ins[:-1]
    _, info = traced(n, lambda w: call(w, srcs=shared), 2)
    assert info.levels > 0


CLOSED_FORM_TEMPLATES = {
    api.CMD_ALLREDUCE: ["InsAllReduceMesh1DOneShot", "InsAllReduceMesh1DTwoShot", "InsAllReduceNHR",
                        "InsAllReduceAicpuReduceNHR", "InsAllReduceMesh1DTwoShotMeshChunk", "InsAllReduceRing",
                        "InsAllReduceRHD"],
    api.CMD_REDUCE_SCATTER: ["InsReduceScatterMesh1D", "InsReduceScatterNHR", "InsReduceScatterAicpuReduceNHR",
                             "InsReduceScatterMesh1DMeshChunk", "ReduceScatterOrderPreserved",
                             "ReduceScatterOrderPreservedGroup"],
}


@pytest.mark.parametrize("seed", range(32))
def test_closed_forms_equal_the_recorded_steps_over_seeded_random_shapes(seed):
    """A guard against the two statements of a template drifting apart: random communicators of 2..64 ranks, every
    template that has a closed form, counts drawn around the places where slices, 4 KiB chunk cuts and executor loops
    change (also with a scratch buffer so small that nearly every count takes several loops), three element sizes,
    in and out of place.  The trace of the closed form must be the trace of the recorded steps, line for line."""
    rng = np.random.default_rng(1000 + seed)
    cases = 0
    while cases < 64:
        n = int(rng.choice([2, 3, 4, 5, 6, 7, 8, 9, 11, 12, 13, 16, 17, 20, 24, 31, 32, 33, 40, 48, 63, 64],
                           p=None))
        if n > 33 and rng.random() < 0.6:
            continue                                   # the widest communicators cost the most: fewer of them
        cmd = api.CMD_ALLREDUCE if rng.random() < 0.55 else api.CMD_REDUCE_SCATTER
        alg = str(rng.choice(CLOSED_FORM_TEMPLATES[cmd]))
        dtype = [T.INT8, T.FP32, T.FP64][int(rng.integers(3))]
        esz = T.DTYPE_SIZE[dtype]
        ccl = SMALL_CCL if rng.random() < 0.5 else 1024 * 1024 + 128 * 64 + int(rng.integers(0, 4096)) * 8
        in_place = cmd == api.CMD_ALLREDUCE and rng.random() < 0.3
        # around a multiple of the rank count, of a 4 KiB chunk per rank, and of what one executor loop holds
        slot = max(1, (ccl - (1 << 20 if cmd == api.CMD_REDUCE_SCATTER else 0)) // n // 128 * 128 // esz)
        anchor = int(rng.choice([1, n, n * n, 4096 // esz, n * (4096 // esz), slot, 2 * slot, n * slot // 2 + 1]))
        count = max(1, anchor + int(rng.integers(-3, 4)))
        if cmd == api.CMD_REDUCE_SCATTER:
            count = max(1, count // n) if rng.random() < 0.5 else count
        loops = -(-count // slot)
        if loops > 4 or count * esz * (n if cmd == api.CMD_REDUCE_SCATTER else 1) > (6 << 20) or (n > 20 and loops > 2):
            continue                                   # keeps a dry case to milliseconds
        op = T.SUM if rng.random() < 0.7 else T.MAX
        ins, outs = fake_ptrs(n)

        def call(w):
            w.set_algorithm(cmd, alg)
            for r in range(n):
                dst = ins[r] if in_place else outs[r]
                if cmd == api.CMD_ALLREDUCE:
                    assert w.all_reduce(r, ins[r], dst, count, dtype, op, FAKE_STREAM) == 0
                else:
                    assert w.reduce_scatter(r, ins[r], dst, count, dtype, op, FAKE_STREAM) == 0
            return w.last_trace()

        def traced_with(closed_form):
            w = api.World(n, ccl_bytes=ccl, dry=True)
            try:
                w.set_closed_form(closed_form)
                return call(w), w.last_info()
            finally:
                w.close()

        recorded, info_r = traced_with(0)
        closed, info_c = traced_with(2)
        what = f"seed={seed} {alg} n={n} count={count} dtype={dtype} op={op} ccl={ccl} in_place={in_place}"
        assert info_r.levels > 0, what
        assert info_c.levels == 0, "the closed form was not used: " + what
        assert closed == recorded, what
        assert info_c.fused == info_r.fused and info_c.fusedSegments == info_r.fusedSegments, what
        cases += 1
