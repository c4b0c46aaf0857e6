"""CPU restatement of the reference's algorithm templates and executor chunk loops.

TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the library never does.

Every function below walks the same copy / reduce steps, in the same order and through the same scratch
("CCL") slots, as the reference template it names, for all N ranks of one communicator at once.  The
inter-rank handshakes of the reference only order those steps; here the order is the program order of
each function (all transfers of a phase, then the phase that consumes them).

Three element back-ends run the same schedules (SampledElems: the numeric one on a sample of the element
columns, for sizes where a dense run is too slow):
  * NumericElems  -- numpy buffers, reductions through oracle/elem_oracle.c (dst = src (+) dst);
  * SymbolicElems -- buffers of strings; a reduce builds "(src+dst)", a copy moves the string.  It shows
                     the association order of a template as text, e.g. "(x2+(x1+x0))".

Reference followed (paths relative to the reference tree, src/ops/...):
  allreduce_mesh_one_shot      all_reduce/template/aicpu/ins_temp_all_reduce_mesh_1D_one_shot.cc:67-199
  allreduce_mesh_two_shot      all_reduce/template/aicpu/ins_temp_all_reduce_mesh_1D_two_shot.cc:77-384
  allreduce_nhr                all_reduce/template/aicpu/ins_temp_all_reduce_nhr.cc:78-414
  allreduce_aicpu_reduce_nhr   all_reduce/template/aicpu/ins_temp_all_reduce_aicpu_reduce_nhr.cc:65-271
  reduce_scatter_mesh          reduce_scatter/template/aicpu/ins_temp_reduce_scatter_mesh_1D.cc:65-227
  reduce_scatter_nhr           reduce_scatter/template/aicpu/ins_temp_reduce_scatter_nhr.cc:77-425
  reduce_scatter_aicpu_reduce_nhr  reduce_scatter/template/aicpu/ins_temp_reduce_scatter_aicpu_reduce_nhr.cc:52-240
  reduce_scatter_order_preserved  reduce_scatter/template/aicpu/ins_temp_reduce_scatter_order_preserved_level1.cc:52-330,
                               executor reduce_scatter/executor/ins_v2_reduce_scatter_order_preserved_executor.cc:77-186;
                               the same result stands for ins_temp_reduce_scatter_order_preserved_group.cc, which
                               only changes which peer sends when (its sends are whole-slot copies)
  reduce_scatter_mesh_chunk    reduce_scatter/template/aicpu/ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:69-263
  allreduce_mesh_two_shot_mesh_chunk  all_reduce/template/aicpu/ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:49-336
  reduce_scatter_v_mesh        reduce_scatter_v/template/aicpu/ins_temp_reduce_scatter_v_mesh_1D.cc:50-179,
                               chunk loop reduce_scatter_v/executor/ins_v2_reduce_scatter_v_sole_executor.cc:75-170
  executor chunk loops         all_reduce/executor/ins_v2_all_reduce_sole_executor.cc:92-185,
                               reduce_scatter/executor/ins_v2_reduce_scatter_sole_executor.cc:123-170
  allreduce_ring, allreduce_rhd  no executable reference exists; defined from the prose of
                               docs/zh/user_guide/coll_algo_intro/Ring.md:5-15 and RHD.md:11-17
  allgather / allgatherv / alltoallv  the API contract (include/hccl.h:102-135, :183-204) as the
                               reference's semantics checkers state it
                               (test/st/algorithm/utils/src/hccl_verifier/semantics_check/
                               allgather_v_semantics_checker.cc:17-100, all2allv_semantics_checker.cc:19-95)

  moe_route / moe_pack / moe_combine  no reference code; the contract of include/hcclx.h (stable grouping by
                               destination rank, its inverse, fp32-accumulated combine)

What pins each function (tests/test_oracle_templates.py, fixtures in tests/golden/st_cases.json):
  * every template: the predicates of the reference's semantics checkers on the symbolic run (each output
    element reduces every rank exactly once at its own offset), equality with numpy folds on integers with
    executor chunking, two ranks = one pairwise op;
  * association order, as expression strings worked by hand from the cited lines: one-shot / two-shot /
    CPU-reduce NHR (self-first and chain orders), NHR (N = 5, 12 and the rank-0-of-12 step table), order-preserved
    tree (3, 8, 12 ranks), mesh-chunk ReduceScatter and AllReduce (N = 3, 4, every owner and chunk, and the
    4 KiB / by-element chunk cuts), ReduceScatter CPU-reduce NHR (N = 3, 5), ring (N = 3, 5, 8, every slice, plus
    the chain written out in fp32) and halving-doubling (p = 5, the document's own example, and p = 12, every
    slice, plus p = 5 written out in fp32).
  * ring and halving-doubling have no executable form in the reference (its AICPU templates are mesh and NHR);
    their step order follows Ring.md:5-15 and RHD.md:11-17, and where the prose leaves a choice (which half of
    its range a rank keeps, which operand is the source) the fixture states the rule used.
PARITY UNPINNED, by nature: the rounding of Ascend's inline reduce for 16-bit floats (external hardware; the
tests allow 1 ULP of an fp32-accumulated result) and NaN payloads (the reference's host FPU decides them; the
tests compare NaN positions).
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BFP16 = range(12)
SUM, PROD, MAX, MIN = range(4)
DTYPE_SIZE = [1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1]  # alg_param.h:43-45
NP_STORAGE = {INT8: np.int8, INT16: np.int16, INT32: np.int32, FP16: np.uint16, FP32: np.float32,
              INT64: np.int64, UINT64: np.uint64, UINT8: np.uint8, UINT16: np.uint16, UINT32: np.uint32,
              FP64: np.float64, BFP16: np.uint16}

CCL_BYTES_DEFAULT = 200 * 1024 * 1024  # test/st/algorithm/utils/inc/sim_common.h:36
HCCL_MIN_SLICE_ALIGN = 128              # src/ops/op_common/template/alg_template_base.h:35
UB_MAX_DATA_SIZE = 256 * 1024 * 1024    # src/ops/op_common/inc/alg_param.h:37

_lib = None


def lib():
    """ctypes handle of oracle/liboracle.so (built by oracle/Makefile)."""
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "liboracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle`")
        L = ctypes.CDLL(path)
        for name in ("orc_reduce", "orc_reduce_parallel"):
            fn = getattr(L, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_int]
        L.orc_fp16_to_fp32.restype = ctypes.c_float
        L.orc_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        L.orc_fp32_to_fp16.restype = ctypes.c_uint16
        L.orc_fp32_to_fp16.argtypes = [ctypes.c_float]
        L.orc_bf16_to_fp32.restype = ctypes.c_float
        L.orc_bf16_to_fp32.argtypes = [ctypes.c_uint16]
        L.orc_fp32_to_bf16.restype = ctypes.c_uint16
        L.orc_fp32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_widen16.restype = None
        L.orc_widen16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int]
        L.orc_narrow16.restype = None
        L.orc_narrow16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int]
        _lib = L
    return _lib


def widen16(bits, dtype):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().orc_widen16(out.ctypes.data, bits.ctypes.data, bits.size, dtype)
    return out


def narrow16(vals, dtype):
    vals = np.ascontiguousarray(vals, dtype=np.float32)
    out = np.empty(vals.shape, dtype=np.uint16)
    lib().orc_narrow16(out.ctypes.data, vals.ctypes.data, vals.size, dtype)
    return out


class NumericElems:
    """Buffers hold storage elements; reduce is the C restatement of AicpuReduceTemplate."""

    def __init__(self, dtype, op, parallel=False):
        self.dtype, self.op, self.parallel = dtype, op, parallel
        self.np_dtype = NP_STORAGE[dtype]

    def empty(self, n):
        return np.zeros(n, dtype=self.np_dtype)

    def copy(self, dst, doff, src, soff, n):
        if n:
            dst[doff:doff + n] = src[soff:soff + n]

    def reduce(self, dst, doff, src, soff, n):
        if not n:
            return
        d = dst[doff:doff + n]
        s = src[soff:soff + n]
        fn = lib().orc_reduce_parallel if self.parallel else lib().orc_reduce
        rc = fn(d.ctypes.data, s.ctypes.data, n, self.dtype, self.op)
        if rc != 0:
            raise ValueError(f"reduce unsupported: dtype {self.dtype} op {self.op}")


class SymbolicElems:
    """Buffers hold expression strings; "(a+b)" means dst=b, src=a."""

    def empty(self, n):
        a = np.empty(n, dtype=object)
        a[:] = "?"
        return a

    def copy(self, dst, doff, src, soff, n):
        if n:
            dst[doff:doff + n] = src[soff:soff + n]

    def reduce(self, dst, doff, src, soff, n):
        for i in range(n):
            if dst[doff + i] == "?" or src[soff + i] == "?":
                raise AssertionError("reduce reads an undefined element")
            dst[doff + i] = "(" + src[soff + i] + "+" + dst[doff + i] + ")"


class SampledBuf:
    """A buffer of which only some positions are known: sorted positions and their values."""

    def __init__(self, length, np_dtype, pos=None, val=None):
        self.n = length
        self.pos = np.empty(0, dtype=np.int64) if pos is None else np.asarray(pos, dtype=np.int64)
        self.val = np.empty(0, dtype=np_dtype) if val is None else np.ascontiguousarray(val, dtype=np_dtype)

    def __len__(self):
        return self.n

    def window(self, off, n):
        a, b = np.searchsorted(self.pos, [off, off + n])
        return a, b


class SampledElems:
    """Runs a schedule on a sample of the element columns only, so that a template can be followed at
    sizes (GiB per rank) where a dense CPU run would take minutes.  Every rank's input must be sampled at
    the same positions; copies move the samples that fall inside the copied range, reduces combine the
    samples of two ranges, which then sit at the same relative positions (both ranges derive from the same
    input range of different ranks).  Arithmetic is the same C loop as NumericElems."""

    def __init__(self, dtype, op):
        self.dtype, self.op = dtype, op
        self.np_dtype = NP_STORAGE[dtype]

    def empty(self, n):
        return SampledBuf(n, self.np_dtype)

    def sample(self, length, positions, values):
        return SampledBuf(length, self.np_dtype, positions, values)

    def copy(self, dst, doff, src, soff, n):
        if not n:
            return
        assert soff + n <= len(src) and doff + n <= len(dst), "copy outside a buffer"
        a, b = src.window(soff, n)
        c, d = dst.window(doff, n)
        dst.val = np.concatenate([dst.val[:c], src.val[a:b], dst.val[d:]])
        dst.pos = np.concatenate([dst.pos[:c], src.pos[a:b] - soff + doff, dst.pos[d:]])

    def reduce(self, dst, doff, src, soff, n):
        if not n:
            return
        assert soff + n <= len(src) and doff + n <= len(dst), "reduce outside a buffer"
        a, b = src.window(soff, n)
        c, d = dst.window(doff, n)
        if b - a != d - c or not np.array_equal(src.pos[a:b] - soff, dst.pos[c:d] - doff):
            raise AssertionError("reduce combines ranges with different samples")
        if b == a:
            return
        tmp = np.ascontiguousarray(dst.val[c:d])
        s = np.ascontiguousarray(src.val[a:b])
        rc = lib().orc_reduce(tmp.ctypes.data, s.ctypes.data, b - a, self.dtype, self.op)
        if rc != 0:
            raise ValueError(f"reduce unsupported: dtype {self.dtype} op {self.op}")
        dst.val[c:d] = tmp


class World:
    """N ranks; rank r owns inp[r], out[r] and a scratch buffer ccl[r] (element arrays)."""

    def __init__(self, elems, inputs, out_count, esz, ccl_bytes=CCL_BYTES_DEFAULT):
        self.e = elems
        self.n = len(inputs)
        self.inp = list(inputs)
        self.out = [elems.empty(out_count) for _ in range(self.n)]
        self.esz = esz
        self.ccl_bytes = ccl_bytes
        self.ccl = [None] * self.n

    def need_ccl(self, count):
        for r in range(self.n):
            if self.ccl[r] is None or len(self.ccl[r]) < count:
                self.ccl[r] = self.e.empty(count)


def round_up(a, b):
    return a // b + (1 if a % b else 0)


def nhr_step_num(n):
    """GetNHRStepNum, src/ops/op_common/template/template_utils.cc:27-35."""
    steps, tmp = 0, n - 1
    while tmp:
        tmp >>= 1
        steps += 1
    return steps


def split_data(count, n):
    """SplitData of the two-shot / NHR AllReduce templates (ins_temp_all_reduce_nhr.cc:137-163):
    (offset, count) per slice, ceil(count/n) each, the remainder short or empty."""
    slice_count = round_up(count, n)
    out, off = [], 0
    for _ in range(n):
        if count - off > slice_count:
            out.append((off, slice_count))
            off += slice_count
        else:
            out.append((off, count - off))
            off = count
    return out


def nhr_rs_steps(n, r):
    """GetReduceScatterStepInfoList, ins_temp_all_reduce_nhr.cc:325-364: per step (to, from, tx ids, rx ids)."""
    steps = []
    for s in range(nhr_step_num(n)):
        delta = 1 << s
        to, frm = (r + n - delta) % n, (r + delta) % n
        n_slices = (n - 1 + (1 << s)) // (1 << (s + 1))
        dsl = 1 << (s + 1)
        tx, rx, txs, rxs = to, r, [], []
        for _ in range(n_slices):
            txs.append(tx)
            rxs.append(rx)
            tx = (tx + n - dsl) % n
            rx = (rx + n - dsl) % n
        steps.append((to, frm, txs, rxs))
    return steps


def nhr_ag_steps(n, r):
    """GetAllGatherStepInfoList, ins_temp_all_reduce_nhr.cc:367-404 (same as GetStepInfo of the CPU-reduce
    NHR template, ins_temp_all_reduce_aicpu_reduce_nhr.cc:238-271)."""
    ns = nhr_step_num(n)
    steps = []
    for s in range(ns):
        delta = 1 << (ns - 1 - s)
        to, frm = (r + delta) % n, (r + n - delta) % n
        n_slices = (n - 1 + (1 << (ns - 1 - s))) // (1 << (ns - s))
        dsl = 1 << (ns - s)
        tx, rx, txs, rxs = r, (r - (1 << (ns - 1 - s)) + n) % n, [], []
        for _ in range(n_slices):
            txs.append(tx)
            rxs.append(rx)
            tx = (tx + n - dsl) % n
            rx = (rx + n - dsl) % n
        steps.append((to, frm, txs, rxs))
    return steps


# ------------------------------------------------------------------------------------------------
# AllReduce templates: one call handles one executor chunk [base, base+count) of every rank
# ------------------------------------------------------------------------------------------------

def allreduce_mesh_one_shot(w, base, count):
    n, e = w.n, w.e
    w.need_ccl(count * n)
    for r in range(n):                                   # RunAllReduce :101-161
        e.copy(w.out[r], base, w.inp[r], base, count)    # own data first
        for q in range(1, n):
            peer = (r + q) % n
            e.copy(w.ccl[peer], r * count, w.inp[r], base, count)   # slot r of the peer's scratch
    for r in range(n):                                   # PostLocalReduce :163-199
        for k in range(n):
            if k != r:
                e.reduce(w.out[r], base, w.ccl[r], k * count, count)


def allreduce_mesh_two_shot(w, base, count):
    n, e = w.n, w.e
    sl = split_data(count, n)
    w.need_ccl(max(c for _, c in sl) * n if count else 0)
    for r in range(n):                                   # ScatterData :191-266
        for k in range(n):
            off, c = sl[k]
            e.copy(w.ccl[k], r * c, w.inp[r], base + off, c)   # my slice k -> slot r of rank k
    for r in range(n):                                   # ReduceData :268-294 ("sequential, deterministic")
        _, c = sl[r]
        for s in range(1, n):
            e.reduce(w.ccl[r], 0, w.ccl[r], s * c, c)
    for r in range(n):                                   # GatherData :310-384
        for k in range(n):
            off, c = sl[k]
            e.copy(w.out[r], base + off, w.ccl[k], 0, c)


def allreduce_nhr(w, base, count):
    n, e = w.n, w.e
    if count == 0:
        return
    sl = split_data(count, n)
    w.need_ccl(count)
    for r in range(n):                                   # PreCopy :165-181
        e.copy(w.ccl[r], 0, w.inp[r], base, count)
    for s in range(nhr_step_num(n)):                     # RunReduceScatter :183-243
        sends = []
        for r in range(n):
            to, _, txs, _ = nhr_rs_steps(n, r)[s]
            for idx in txs:
                off, c = sl[idx]
                sends.append((to, r, off, c))
        # within a step no slice is both sent and received by one rank, so order inside the step is free
        for to, r, off, c in sends:
            e.reduce(w.ccl[to], off, w.ccl[r], off, c)
    for s in range(nhr_step_num(n)):                     # RunAllGather :245-304
        for r in range(n):
            to, _, txs, _ = nhr_ag_steps(n, r)[s]
            for idx in txs:
                off, c = sl[idx]
                e.copy(w.ccl[to], off, w.ccl[r], off, c)
    for r in range(n):                                   # PostCopy :306-322
        e.copy(w.out[r], base, w.ccl[r], 0, count)


def allreduce_aicpu_reduce_nhr(w, base, count):
    n, e = w.n, w.e
    w.need_ccl(count * n)
    for r in range(n):                                   # PreCopy :151-162
        e.copy(w.ccl[r], r * count, w.inp[r], base, count)
    for s in range(nhr_step_num(n)):                     # RunGather :164-210: all-gather of whole inputs
        for r in range(n):
            to, _, txs, _ = nhr_ag_steps(n, r)[s]
            for idx in txs:
                e.copy(w.ccl[to], idx * count, w.ccl[r], idx * count, count)
    for r in range(n):                                   # RunReduce :212-236
        e.copy(w.out[r], base, w.ccl[r], r * count, count)
        for k in range(n):
            if k != r:
                e.reduce(w.out[r], base, w.ccl[r], k * count, count)


def allreduce_ring(w, base, count):
    """Ring.md:5-15: one lap of reduce-scatter (each step a rank passes one block downstream and the
    receiver folds it in), one lap of all-gather.  Blocks are the SplitData slices; at step t rank r
    sends slice (r - t) mod n to rank r + 1."""
    n, e = w.n, w.e
    if count == 0:
        return
    sl = split_data(count, n)
    w.need_ccl(count)
    for r in range(n):
        e.copy(w.ccl[r], 0, w.inp[r], base, count)
    for t in range(n - 1):
        for r in range(n):
            off, c = sl[(r - t) % n]
            e.reduce(w.ccl[(r + 1) % n], off, w.ccl[r], off, c)
    for t in range(n - 1):
        for r in range(n):
            off, c = sl[(r + 1 - t) % n]                 # the slice rank r completed, then what it received
            e.copy(w.ccl[(r + 1) % n], off, w.ccl[r], off, c)
    for r in range(n):
        e.copy(w.out[r], base, w.ccl[r], 0, count)


def rhd_block(n):
    """RHD.md:17: r = p - 2^floor(log p); the first 2r ranks fold pairwise (odd into even); the block of
    p - r ranks that runs halving-doubling is [0, 2, .., 2r-2, 2r, 2r+1, .., p-1]."""
    p2 = 1 << (n.bit_length() - 1)
    extra = n - p2
    return extra, [2 * i for i in range(extra)] + list(range(2 * extra, n))


def allreduce_rhd(w, base, count):
    """RHD.md:11-17, AllReduce variant :26: fold, reduce-scatter by vector halving / distance doubling
    (partner b XOR 2^s; each keeps the half its own bit selects), all-gather in reverse, copy back."""
    n, e = w.n, w.e
    if count == 0:
        return
    extra, block = rhd_block(n)
    p2 = len(block)
    sl = split_data(count, p2)
    w.need_ccl(count)
    for r in range(n):
        e.copy(w.ccl[r], 0, w.inp[r], base, count)
    for i in range(extra):                               # fold rank 2i+1 into rank 2i
        e.reduce(w.ccl[2 * i], 0, w.ccl[2 * i + 1], 0, count)
    steps = p2.bit_length() - 1
    own = [(0, p2)] * p2                                 # slice range each block rank still works on
    for s in range(steps):
        nxt, ops = list(own), []
        for b in range(p2):
            lo, hi = own[b]
            mid = (lo + hi) // 2
            keep = (lo, mid) if not (b >> s) & 1 else (mid, hi)
            give = (mid, hi) if not (b >> s) & 1 else (lo, mid)
            nxt[b] = keep
            ops.append((b ^ (1 << s), b, give))
        for dst_b, src_b, (lo, hi) in ops:
            for k in range(lo, hi):
                off, c = sl[k]
                e.reduce(w.ccl[block[dst_b]], off, w.ccl[block[src_b]], off, c)
        own = nxt
    for s in reversed(range(steps)):                     # all-gather: send back what was kept
        ops = []
        for b in range(p2):
            ops.append((b ^ (1 << s), b, own[b]))
        for dst_b, src_b, (lo, hi) in ops:
            for k in range(lo, hi):
                off, c = sl[k]
                e.copy(w.ccl[block[dst_b]], off, w.ccl[block[src_b]], off, c)
        own = [(min(own[b][0], own[b ^ (1 << s)][0]), max(own[b][1], own[b ^ (1 << s)][1])) for b in range(p2)]
    for i in range(extra):                               # restore the folded ranks
        e.copy(w.ccl[2 * i + 1], 0, w.ccl[2 * i], 0, count)
    for r in range(n):
        e.copy(w.out[r], base, w.ccl[r], 0, count)


def chunk_distance(step, chunk, n):
    """Mesh-chunk rotation: in step `step`, chunk `chunk` of a shard is written by the rank this many places
    above the owner: step + chunk + 1, skipping the multiples of n
    (ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:187-191, ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:176-181)."""
    d = step + chunk + 1
    if d >= n:
        d += 1
    return d % n


def split_even(count, parts):
    """count elements in `parts` chunks, the first count % parts one longer (two_shot_mesh_chunk.cc:131-142)."""
    return [count // parts + (1 if i < count % parts else 0) for i in range(parts)]


def allreduce_mesh_two_shot_mesh_chunk(w, base, count):
    """Two-shot mesh for large messages: the owner's slice sits in its scratch buffer at the slice's own offset
    and every peer reduce-writes its chunks straight onto it, chunk c in step s coming from the rank
    chunk_distance(s, c) above the owner; then every rank reads every owner's slice."""
    n, e = w.n, w.e
    if count == 0:
        return
    sl = split_data(count, n)
    w.need_ccl(count)
    for r in range(n):                                   # PreCopy :313-336
        off, c = sl[r]
        e.copy(w.ccl[r], off, w.inp[r], base + off, c)
    for step in range(n - 1):                            # RunReduceScatter :122-238
        for owner in range(n):
            off, c = sl[owner]
            sizes = split_even(c, n - 1)
            pos = 0
            for ch in range(n - 1):
                src = (owner + chunk_distance(step, ch, n)) % n
                e.reduce(w.ccl[owner], off + pos, w.inp[src], base + off + pos, sizes[ch])
                pos += sizes[ch]
    for r in range(n):                                   # RunAllgather :240-311
        for k in range(n):
            off, c = sl[k]
            e.copy(w.out[r], base + off, w.ccl[k], off, c)


ALLREDUCE_TEMPLATES = {
    # name -> (function, scratch multiple as CalcScratchMultiple returns it)
    "InsAllReduceMesh1DOneShot": (allreduce_mesh_one_shot, lambda n: n),      # one_shot.cc:42-48
    "InsAllReduceMesh1DTwoShot": (allreduce_mesh_two_shot, lambda n: 2),      # two_shot.cc:20-27
    "InsAllReduceNHR": (allreduce_nhr, lambda n: 1),                           # nhr.cc:20-26
    "InsAllReduceAicpuReduceNHR": (allreduce_aicpu_reduce_nhr, lambda n: n),  # aicpu_reduce_nhr.cc:22-28
    "InsAllReduceMesh1DTwoShotMeshChunk": (allreduce_mesh_two_shot_mesh_chunk, lambda n: 2),   # mesh_chunk.cc:17-24
    "InsAllReduceRing": (allreduce_ring, lambda n: 1),
    "InsAllReduceRHD": (allreduce_rhd, lambda n: 1),
}


def chunk_counts(total, ccl_bytes, scratch_multiple, esz, transport_bound):
    """The executors' chunk rule: maxDataSizePerLoop = min(transportBound, ccl/mult/128*128)
    (ins_v2_all_reduce_sole_executor.cc:129-152)."""
    if scratch_multiple:
        bound = ccl_bytes // scratch_multiple // HCCL_MIN_SLICE_ALIGN * HCCL_MIN_SLICE_ALIGN
        max_bytes = min(transport_bound, bound)
    else:
        max_bytes = transport_bound
    max_count = max_bytes // esz
    if max_count == 0:
        raise ValueError("maxDataCountPerLoop is 0")
    loops = total // max_count + (1 if total % max_count else 0)
    out, done = [], 0
    for i in range(loops):
        cur = total - done if i == loops - 1 else max_count
        out.append((done, cur))
        done += cur
    return out


def run_allreduce(elems, inputs, count, esz, alg, ccl_bytes=CCL_BYTES_DEFAULT):
    """HcclAllReduce through the sole executor and template `alg`; returns the per-rank outputs."""
    fn, mult = ALLREDUCE_TEMPLATES[alg]
    w = World(elems, inputs, count, esz, ccl_bytes)
    for base, cur in chunk_counts(count, ccl_bytes, mult(w.n), esz, ccl_bytes):
        fn(w, base, cur)
    return w.out


# ------------------------------------------------------------------------------------------------
# ReduceScatter
# ------------------------------------------------------------------------------------------------

def reduce_scatter_mesh(w, base, count, stride):
    """One chunk: rank r's slice k lives at inp[r][k*stride + base .. +count); out[r][base .. +count)."""
    n, e = w.n, w.e
    w.need_ccl(count * n)
    for r in range(n):                                   # RunReduceScatter :160-227
        for q in range(1, n):
            k = (r + q) % n
            e.copy(w.ccl[k], r * count, w.inp[r], k * stride + base, count)
    for r in range(n):                                   # PostCopy :103-158
        e.copy(w.out[r], base, w.inp[r], r * stride + base, count)
        for k in range(n):
            if k != r:
                e.reduce(w.out[r], base, w.ccl[r], k * count, count)


def reduce_scatter_nhr(w, base, count, stride):
    """ins_temp_reduce_scatter_nhr.cc: slices are the ranks' shards; the NHR steps of the AllReduce NHR
    reduce-scatter phase run over scratch slots (slot k = shard k); step-0 sends go straight from the
    input (:98-101, :329-332), which changes no value."""
    n, e = w.n, w.e
    w.need_ccl(count * n)
    for r in range(n):                                   # LocalDataCopy :168-208
        for k in range(n):
            e.copy(w.ccl[r], k * count, w.inp[r], k * stride + base, count)
    for s in range(nhr_step_num(n)):                     # RunNHR :255-367
        sends = []
        for r in range(n):
            to, _, txs, _ = nhr_rs_steps(n, r)[s]
            for idx in txs:
                sends.append((to, r, idx))
        for to, r, idx in sends:
            e.reduce(w.ccl[to], idx * count, w.ccl[r], idx * count, count)
    for r in range(n):                                   # PostLocalCopy :210-253
        e.copy(w.out[r], base, w.ccl[r], r * count, count)


def reduce_scatter_aicpu_reduce_nhr(w, base, count, stride):
    """ins_temp_reduce_scatter_aicpu_reduce_nhr.cc:52-80: one round per shard k: every rank copies its shard k
    into slot <own rank> of its scratch (:82-113), the NHR all-gather steps spread the slots (:180-240), and rank
    k folds: own input to the output (:115-138), then the other ranks' slots ascending (:140-178)."""
    n, e = w.n, w.e
    w.need_ccl(count * n)
    for k in range(n):
        for r in range(n):
            e.copy(w.ccl[r], r * count, w.inp[r], k * stride + base, count)
        e.copy(w.out[k], base, w.inp[k], k * stride + base, count)
        for s in range(nhr_step_num(n)):
            for r in range(n):
                to, _, txs, _ = nhr_ag_steps(n, r)[s]
                for idx in txs:
                    e.copy(w.ccl[to], idx * count, w.ccl[r], idx * count, count)
        for q in range(n):
            if q != k:
                e.reduce(w.out[k], base, w.ccl[k], q * count, count)


def reduce_scatter_mesh_chunk(w, base, count, stride):
    """Mesh ReduceScatter for large shards: the own shard is copied to the scratch buffer and the peers reduce-
    write their chunks onto it in the chunk_distance rotation; N-1 chunks, all but the last rounded down to
    4 KiB, shards too small for that cut evenly (meshchunk.cc:139-162)."""
    n, e = w.n, w.e
    w.need_ccl(max(count, 1))
    for r in range(n):                                   # PreCopy :110-123
        e.copy(w.ccl[r], 0, w.inp[r], r * stride + base, count)
    if n > 1:
        parts = n - 1
        aligned = (count * w.esz // parts) // 4096 * 4096
        if parts >= 2 and aligned > 0:
            sizes = [aligned // w.esz] * (parts - 1) + [count - (aligned // w.esz) * (parts - 1)]
        else:
            sizes = split_even(count, parts)
        for step in range(n - 1):                        # DoMeshChunk :171-243
            for owner in range(n):
                pos = 0
                for ch in range(n - 1):
                    src = (owner + chunk_distance(step, ch, n)) % n
                    e.reduce(w.ccl[owner], pos, w.inp[src], owner * stride + base + pos, sizes[ch])
                    pos += sizes[ch]
    for r in range(n):                                   # PostCopy :245-263
        e.copy(w.out[r], base, w.ccl[r], 0, count)


def reduce_scatter_order_preserved(w, base, count, stride):
    """Strict determinism: all-to-all of the shards into scratch slots (the block from rank k sits in slot
    (k + r) % n of rank r), then a tree that is the same on every rank: with m the largest power of two below
    the number of remaining blocks, block v >= m is folded into block v % m
    (ins_temp_reduce_scatter_order_preserved_level1.cc:170-330)."""
    n, e = w.n, w.e
    w.need_ccl(max(count, 1) * n)
    for r in range(n):                                   # PreLocalCopy + RunAllToAll
        for k in range(n):
            e.copy(w.ccl[k], ((r + k) % n) * count, w.inp[r], k * stride + base, count)
    for r in range(n):                                   # RunLocalReduce
        remaining = n
        while remaining > 1:
            m = 1
            while m * 2 < remaining:
                m *= 2
            for v in range(m, remaining):
                e.reduce(w.ccl[r], ((v % m + r) % n) * count, w.ccl[r], ((v + r) % n) * count, count)
            remaining = m
        e.copy(w.out[r], base, w.ccl[r], (r % n) * count, count)    # PostCopy: block 0


REDUCE_SCATTER_TEMPLATES = {
    "InsReduceScatterMesh1D": (reduce_scatter_mesh, lambda n: n),   # mesh_1D.cc:59-63
    "InsReduceScatterNHR": (reduce_scatter_nhr, lambda n: n),       # nhr.cc:369-377
    "InsReduceScatterAicpuReduceNHR": (reduce_scatter_aicpu_reduce_nhr, lambda n: n),  # aicpu_reduce_nhr.cc:242-249
    "InsReduceScatterMesh1DMeshChunk": (reduce_scatter_mesh_chunk, lambda n: n - 1),   # meshchunk.cc:46-52
    "ReduceScatterOrderPreserved": (reduce_scatter_order_preserved, lambda n: n),      # level1.cc:46-50
    # ins_temp_reduce_scatter_order_preserved_group.cc: the same slots and tree; only the order in which the
    # all-to-all sends go out (:236-262) and the thread count differ, which changes no value
    "ReduceScatterOrderPreservedGroup": (reduce_scatter_order_preserved, lambda n: n),
}


def run_reduce_scatter(elems, inputs, recv_count, esz, alg, ccl_bytes=CCL_BYTES_DEFAULT):
    fn, mult = REDUCE_SCATTER_TEMPLATES[alg]
    w = World(elems, inputs, recv_count, esz, ccl_bytes)
    usable = ccl_bytes - 1024 * 1024          # ins_v2_reduce_scatter_sole_executor.cc:126-128
    bound = usable
    if alg.startswith("ReduceScatterOrderPreserved"):  # its own executor: whole buffer, 256 MiB transport bound
        usable, bound = ccl_bytes, UB_MAX_DATA_SIZE   # ins_v2_reduce_scatter_order_preserved_executor.cc:108-119
    for base, cur in chunk_counts(recv_count, usable, mult(w.n), esz, bound):
        fn(w, base, cur, recv_count)          # inputSliceStride = recvCount * esz (:160)
    return w.out


def reduce_scatter_v_mesh(w, done, sizes, displs, slot):
    """One chunk of the ragged mesh ReduceScatter: rank k's part is inp[*][displs[k] + done .. +sizes[k]);
    rank r writes its part for k into slot r of ccl[k] (slots `slot` elements apart); rank k copies its own
    part to out[k][done ..) and folds the other slots in, ranks ascending."""
    n, e = w.n, w.e
    slot = min(slot, max(sizes))      # where a slot sits in the scratch changes no value: keep the buffers small
    w.need_ccl(slot * n)
    for r in range(n):                                   # RunReduceScatterV :131-179
        for q in range(n - 1):
            k = (r + 1 + q) % n
            e.copy(w.ccl[k], r * slot, w.inp[r], displs[k] + done, sizes[k])
    for r in range(n):                                   # PostCopy :79-129
        e.copy(w.out[r], done, w.inp[r], displs[r] + done, sizes[r])
        for k in range(n):
            if k != r:
                e.reduce(w.out[r], done, w.ccl[r], k * slot, sizes[r])


def run_reduce_scatter_v(elems, inputs, counts, displs, esz, ccl_bytes=CCL_BYTES_DEFAULT):
    """HcclReduceScatterV through its sole executor: every loop takes up to maxDataCountPerLoop elements of
    every rank's part, all parts advancing by the same offset (sole_executor.cc:133-166)."""
    n = len(inputs)
    w = World(elems, inputs, 0, esz, ccl_bytes)
    w.out = [elems.empty(counts[r]) for r in range(n)]
    max_bytes = min(UB_MAX_DATA_SIZE, ccl_bytes // n // HCCL_MIN_SLICE_ALIGN * HCCL_MIN_SLICE_ALIGN)
    max_count = max_bytes // esz
    if max_count == 0:
        raise ValueError("maxDataCountPerLoop is 0")
    biggest = max(counts)
    if biggest == 0:
        return w.out
    done = 0
    for _ in range(1 + (biggest - 1) // max_count):
        sizes = [min(max_count, c - done) if done < c else 0 for c in counts]
        reduce_scatter_v_mesh(w, done, sizes, displs, max_count)
        done += max(sizes)
    return w.out


# ------------------------------------------------------------------------------------------------
# Copies and permutes: the contract
# ------------------------------------------------------------------------------------------------

def run_allgather(inputs, send_count):
    cat = np.concatenate([np.asarray(x[:send_count]) for x in inputs])
    return [cat.copy() for _ in inputs]


def run_allgatherv(inputs, counts, displs, out_len, fill):
    """out_j[displs[i] .. +counts[i]) = in_i[0 .. counts[i]) for all i, j; other positions keep `fill`."""
    outs = []
    for _ in inputs:
        o = fill.copy() if isinstance(fill, np.ndarray) else np.full(out_len, fill, dtype=inputs[0].dtype)
        for i, x in enumerate(inputs):
            o[displs[i]:displs[i] + counts[i]] = x[:counts[i]]
        outs.append(o)
    return outs


def run_alltoallv(inputs, send_counts, sdispls, recv_counts, rdispls, out_lens, fill=0):
    """out_j[rdispls[j][i] .. +recv_counts[j][i]) = in_i[sdispls[i][j] .. +send_counts[i][j]); other positions keep
    `fill` (one value, or per rank the array that was there before)."""
    n = len(inputs)
    outs = []
    for j in range(n):
        o = fill[j].copy() if isinstance(fill, list) else np.full(out_lens[j], fill, dtype=inputs[0].dtype)
        for i in range(n):
            c = send_counts[i][j]
            if c != recv_counts[j][i]:
                raise ValueError("sendCounts[i][j] != recvCounts[j][i]")
            o[rdispls[j][i]:rdispls[j][i] + c] = inputs[i][sdispls[i][j]:sdispls[i][j] + c]
        outs.append(o)
    return outs


# ------------------------------------------------------------------------------------------------
# The caller side of an MoE AlltoAllV (no reference code: defined by its contract)
# ------------------------------------------------------------------------------------------------
MOE_DROPPED = 0xFFFFFFFF


def moe_route(dests, n, row_elems):
    """dests[i]: destination rank per routing entry of rank i.  Entries are grouped by destination, entry
    order kept inside a group; destinations outside 0..n-1 are dropped.  Returns send_counts, sdispls,
    recv_counts, rdispls (n x n lists, in elements) and perm[i] (row of the packed buffer per entry)."""
    counts = [[0] * n for _ in range(n)]
    perms = []
    for i in range(n):
        d = np.asarray(dests[i], dtype=np.int64)
        ok = (d >= 0) & (d < n)
        for j in range(n):
            counts[i][j] = int(np.count_nonzero(d == j))
        starts = np.concatenate([[0], np.cumsum(counts[i])[:-1]])
        perm = np.full(d.size, MOE_DROPPED, dtype=np.uint32)
        kept = np.nonzero(ok)[0]
        order = kept[np.argsort(d[kept], kind="stable")]      # kept entries, grouped by destination, stable
        perm[order] = np.arange(order.size, dtype=np.uint32)
        perms.append(perm)
        del starts
    send_counts = [[c * row_elems for c in row] for row in counts]
    sdispls = [[sum(row[:j]) for j in range(n)] for row in send_counts]
    recv_counts = [[send_counts[i][j] for i in range(n)] for j in range(n)]
    rdispls = [[sum(recv_counts[j][:i]) for i in range(n)] for j in range(n)]
    return send_counts, sdispls, recv_counts, rdispls, perms


def moe_pack(tokens, perm, topk, out_rows):
    """tokens: (rows, width) array; packed[perm[e]] = tokens[e // topk]."""
    packed = np.zeros((out_rows, tokens.shape[1]), dtype=tokens.dtype)
    for e, p in enumerate(perm):
        if p != MOE_DROPPED:
            packed[p] = tokens[e // topk]
    return packed


def moe_combine(packed, perm, topk, dtype):
    """out[t] = sum_j packed[perm[t*topk + j]], j ascending from the first kept entry; 16-bit floats in fp32 with
    one narrowing; topk == 1 moves rows as they are."""
    tokens = len(perm) // topk
    out = np.zeros((tokens, packed.shape[1]), dtype=packed.dtype)
    for t in range(tokens):
        rows = [packed[p] for p in perm[t * topk:(t + 1) * topk] if p != MOE_DROPPED]
        if not rows:
            continue
        if topk == 1:
            out[t] = rows[0]
            continue
        wide = dtype in (FP16, BFP16)
        acc = widen16(rows[0], dtype) if wide else rows[0].astype(np.float32).copy()
        e = NumericElems(FP32, SUM)
        for r in rows[1:]:
            x = widen16(r, dtype) if wide else np.ascontiguousarray(r, dtype=np.float32)
            e.reduce(acc, 0, x, 0, acc.size)
        out[t] = narrow16(acc, dtype) if wide else acc
    return out


def alltoallvc_to_v(matrix, rank):
    """ConvertAlltoAllVCParam, src/ops/all_to_all_v/all_to_all_v_op.cc:396-430: row = what `rank` sends,
    column = what it receives, displacements are the running sums."""
    n = len(matrix)
    sc = [matrix[rank][j] for j in range(n)]
    rc = [matrix[i][rank] for i in range(n)]
    sd = [sum(sc[:j]) for j in range(n)]
    rd = [sum(rc[:i]) for i in range(n)]
    return sc, sd, rc, rd
