#!/usr/bin/env python3
"""Benchmark of the collective hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already resident in HBM:
by default the ReduceScatter SUM bf16 of 8 virtual ranks x 33,554,432 elements (64 MiB per rank), mesh
template order, each output shard a fused 8-way reduce in one HBM pass.  `value` is the effective HBM
bandwidth: algorithmic bytes (every input byte read once + every output byte written once) divided by
the time of a step.

Output: the LAST line of stdout is the benchmark line, one compact JSON object (under 2000 bytes: metric, value,
roofline, cpu_baseline and one percentage per op).  The tables behind it (per-op rows, the 12-rank size sweep,
small-message and planning times from C++) are printed before it, one JSON object per line, and written to the
file DETAILS_FILE names.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-ops] [--no-sweep]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
METRIC = "effective HBM GB/s (and % of peak) per op at 64MB/rank, 8 virtual ranks"
LINE_LIMIT = 2000      # bytes: the benchmark line must survive a reader that keeps the last 2000 characters


def profile_traffic(path, allow_missing=False):
    """HBM bytes per step of a workload as its rocprofv3 summary under profiles/ states them (FETCH_SIZE and
    WRITE_SIZE, scaled by the copy calibration; the summary says how).  The file must exist and hold the line
    `traffic_bytes_per_step: N`."""
    if path is None:
        return None
    full = os.path.join(ROOT, path)
    if not os.path.exists(full):
        if allow_missing:
            return None
        raise SystemExit("bench.py: %s is missing (the roofline's traffic figure is read from it)" % path)
    for line in open(full):
        if line.startswith("traffic_bytes_per_step:"):
            return int(line.split(":")[1].split()[0])
    if allow_missing:
        return None
    raise SystemExit("bench.py: %s has no traffic_bytes_per_step line" % path)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="reduce_scatter_sum_bf16_mesh_8x64MiB")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-ops", action="store_true", help="skip the per-op table")
    ap.add_argument("--no-sweep", action="store_true", help="skip the 12-rank AllReduce size sweep")
    ap.add_argument("--allow-missing-profile", action="store_true",
                    help="report traffic as null instead of stopping when the workload's profiles/ summary is absent "
                         "(the profiling runs that write those summaries use this)")
    return ap.parse_args()


# ----------------------------------------------------------------------------------------------------
# workloads: each builds device buffers once; step() = one collective through the HCCL entry points
# (one call per virtual rank; the last call launches)
# ----------------------------------------------------------------------------------------------------

class Workload:
    name = ""
    dtype = ""
    kernel = ""          # name of the dominant kernel as rocprofv3 prints it (prefix)
    # rocprofv3 summary of this workload under profiles/: kernel times, and the HBM bytes per step from
    # --pmc FETCH_SIZE / WRITE_SIZE scaled by what the same counters read on a plain 1 GiB copy
    profile = None

    def __init__(self, torch, api, T, n):
        self.torch, self.api, self.T, self.n = torch, api, T, n
        self.stream_obj = torch.cuda.Stream()
        self.stream = self.stream_obj.cuda_stream
        self.world = api.World(n)

    def step(self):
        raise NotImplementedError

    def algo_bytes(self):
        raise NotImplementedError

    def pins_bytes(self):
        """The least that must cross the HBM pins: equal to the algorithmic bytes except where one read serves
        several deliveries (AllGather)."""
        return self.algo_bytes()

    def info(self):
        i = self.world.last_info()
        return {"algorithm": i.algName.decode(), "fused": bool(i.fused), "launches": i.launches,
                "plan_cache_hit": bool(i.planCacheHit)}


def _randn_bits16(torch, n, seed, dt):
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    return torch.randn(n, device="cuda:0", generator=g, dtype=torch.float32).to(dt)


class ReduceScatterMesh(Workload):
    """benchmark configuration 2: HcclReduceScatter SUM bf16, 8 ranks x 33,554,432 elements in (64 MiB per rank).
    The selector picks the mesh template; output shard r folds slice r of every rank starting from rank
    r's own data, then ranks ascending (ins_temp_reduce_scatter_mesh_1D.cc:132-154), as one fused pass of the
    chain kernel that moves four vectors per thread (eight sources, one destination per segment)."""
    dtype = "bf16"
    kernel = "hcclx::k_fold_wide<11, 0, 0, 4>"
    profile = "profiles/k_fold_wide_reduce_scatter_bf16_8x64MiB.txt"

    def __init__(self, torch, api, T, n=8, recv=4 * 1024 * 1024):
        super().__init__(torch, api, T, n)
        if (n, recv) != (8, 4 * 1024 * 1024):
            self.profile, self.kernel = None, "hcclx::k_fold_wide<11, 0, 0, 4>"
        self.name = "reduce_scatter_sum_bf16_mesh_%dx%dMiB" % (n, n * recv * 2 >> 20)
        self.recv = recv
        self.x = [_randn_bits16(torch, n * recv, 1000 + r, torch.bfloat16) for r in range(n)]
        self.out = [torch.empty(recv, device="cuda:0", dtype=torch.bfloat16) for _ in range(n)]
        self.sp = [t.data_ptr() for t in self.x]
        self.rp = [t.data_ptr() for t in self.out]

    def step(self):
        w, T = self.world, self.T
        for r in range(self.n):
            rc = w.reduce_scatter(r, self.sp[r], self.rp[r], self.recv, T.BFP16, T.SUM, self.stream)
            assert rc == 0, rc

    def algo_bytes(self):
        return (self.n + 1) * self.n * self.recv * 2

    def cpu_baseline(self, parallel):
        """The oracle's restatement of the same template on the same shape, timed on the host."""
        import numpy as np
        from oracle import templates as T     # the only use of the oracle in this script: the thing timed here
        rng = np.random.default_rng(0)
        xs = [T.narrow16(rng.standard_normal(self.n * self.recv, dtype=np.float32), T.BFP16) for _ in range(self.n)]
        best = None
        runs = 6    # about 5 s on one core
        for _ in range(runs):
            t0 = time.perf_counter()
            T.run_reduce_scatter(T.NumericElems(T.BFP16, T.SUM, parallel=parallel), xs, self.recv, 2,
                                 "InsReduceScatterMesh1D")
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return self.algo_bytes() / best / 1e9, ("the full workload (8 ranks x 64 MiB bf16, one ReduceScatter) through the "
                                                "oracle's C loop in the mesh template's order, best of %d runs" % runs)


class AllReduce(Workload):
    """HcclAllReduce, by default SUM fp32 among 8 ranks x 16,777,216 elements (64 MiB per rank).  At that size the
    selector takes the two-shot mesh template: every slice is the fold x7 (+) (... (x1 (+) x0)), the same on all
    ranks.  One launch folds each slice into the first output (eight inputs read once), a second copies it to the
    other seven, one output at a time."""
    dtype = "f32"
    kernel = "hcclx::k_fold_wide<4, 0, 0, 4> + hcclx::(anonymous namespace)::k_phased_copy"
    profile = "profiles/k_fold_wide_k_phased_copy_all_reduce_fp32_8x64MiB.txt"

    def __init__(self, torch, api, T, n=8, count=16 * 1024 * 1024, alg=None, step_mode=False, dtype=None, op=None,
                 profile=None, kernel=None):
        super().__init__(torch, api, T, n)
        self.dt = T.FP32 if dtype is None else dtype
        self.op = T.SUM if op is None else op
        opname = {T.SUM: "sum", T.PROD: "prod", T.MAX: "max", T.MIN: "min"}[self.op]
        self.name = "all_reduce_%s_%s_%dx%dMiB" % (opname, "int32" if self.dt == T.INT32 else "fp32", n, count * 4 >> 20)
        if alg:
            self.world.set_algorithm(api.CMD_ALLREDUCE, alg)
            self.name += "_" + alg
        if step_mode:
            self.world.set_mode(api.EXEC_STEP)
            self.name += "_step_by_step"
        if (n, count, alg, step_mode, dtype, op) != (8, 16 * 1024 * 1024, None, False, None, None):
            self.profile, self.kernel = profile, kernel or ""
        self.dtype = "i32" if self.dt == T.INT32 else "f32"
        self.count = count
        g = torch.Generator(device="cuda:0")
        g.manual_seed(7)
        if self.dt == T.INT32:
            self.x = [torch.randint(-2**31, 2**31 - 1, (count,), device="cuda:0", generator=g, dtype=torch.int32)
                      for _ in range(n)]
            self.out = [torch.empty(count, device="cuda:0", dtype=torch.int32) for _ in range(n)]
        else:
            lo, hi = (0.9, 1.1) if self.op == T.PROD else (-1.0, 1.0)
            self.x = [torch.rand(count, device="cuda:0", generator=g) * (hi - lo) + lo for _ in range(n)]
            self.out = [torch.empty(count, device="cuda:0") for _ in range(n)]
        self.sp = [t.data_ptr() for t in self.x]
        self.rp = [t.data_ptr() for t in self.out]

    def step(self):
        w = self.world
        for r in range(self.n):
            rc = w.all_reduce(r, self.sp[r], self.rp[r], self.count, self.dt, self.op, self.stream)
            assert rc == 0, rc

    def algo_bytes(self):
        return 2 * self.n * self.count * 4


class AllGather(Workload):
    """HcclAllGather fp16, 8 ranks x 33,554,432 elements (64 MiB per rank): every block lands in every
    output; each source byte is read once and written eight times."""
    dtype = "u8"
    kernel = "hcclx::(anonymous namespace)::k_phased_copy_inline"
    profile = "profiles/k_phased_copy_all_gather_fp16_8x64MiB.txt"

    def __init__(self, torch, api, T, n=8, count=32 * 1024 * 1024):
        super().__init__(torch, api, T, n)
        self.name = "all_gather_fp16_%dx%dMiB" % (n, count * 2 >> 20)
        self.count = count
        self.x = [torch.randint(-32768, 32767, (count,), device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.out = [torch.empty(n * count, device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.sp = [t.data_ptr() for t in self.x]
        self.rp = [t.data_ptr() for t in self.out]

    def step(self):
        w, T = self.world, self.T
        for r in range(self.n):
            rc = w.all_gather(r, self.sp[r], self.rp[r], self.count, T.FP16, self.stream)
            assert rc == 0, rc

    def algo_bytes(self):
        return 2 * self.n * self.n * self.count * 2

    def pins_bytes(self):
        return (1 + self.n) * self.n * self.count * 2


class AllGatherV(Workload):
    """benchmark configuration 3: HcclAllGatherV fp16, 16 ranks, per-rank counts uniform in [0, 8,388,608] from a
    seed, displacements their prefix sum (so most blocks start at addresses that are only 2-byte aligned)."""
    dtype = "u8"
    kernel = "hcclx::(anonymous namespace)::k_phased_copy_inline"
    profile = "profiles/k_phased_copy_all_gather_v_fp16_16_ranks_ragged.txt"

    def __init__(self, torch, api, T, n=16, seed=3):
        import numpy as np
        super().__init__(torch, api, T, n)
        self.name = "all_gather_v_fp16_16_ranks_ragged"
        rng = np.random.default_rng(seed)
        self.counts = [int(c) for c in rng.integers(0, 8388608, size=n, endpoint=True)]
        self.displs = [int(d) for d in np.concatenate([[0], np.cumsum(self.counts)[:-1]])]
        total = sum(self.counts)
        self.x = [torch.randint(-32768, 32767, (max(c, 1),), device="cuda:0", dtype=torch.int16) for c in self.counts]
        self.out = [torch.empty(total, device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.sp = [t.data_ptr() for t in self.x]
        self.rp = [t.data_ptr() for t in self.out]
        self.ct, self.dt = api.u64_table(self.counts), api.u64_table(self.displs)

    def step(self):
        w, T = self.world, self.T
        for r in range(self.n):
            rc = w.all_gather_v(r, self.sp[r], self.counts[r], self.rp[r], self.ct, self.dt, T.FP16, self.stream)
            assert rc == 0, rc

    def algo_bytes(self):
        return 2 * self.n * sum(self.counts) * 2

    def pins_bytes(self):
        return (1 + self.n) * sum(self.counts) * 2


class AllToAllV(Workload):
    """benchmark configuration 4: HcclAlltoAllV bf16, MoE dispatch: 8 ranks x 4096 tokens x hidden 7168,
    destination rank per token Zipf(s=1.2), tokens grouped by destination."""
    dtype = "u8"
    kernel = "hcclx::(anonymous namespace)::k_alltoallv_direct<2>"

    def __init__(self, torch, api, T, n=8, tokens=4096, hidden=7168, seed=0):
        import numpy as np
        super().__init__(torch, api, T, n)
        self.name = "all_to_all_v_bf16_moe_%dx%dx%d" % (n, tokens, hidden)
        self.profile = "profiles/k_alltoallv_bf16_moe_%dx%dx%d.txt" % (n, tokens, hidden)
        rng = np.random.default_rng(seed)
        w = 1.0 / np.arange(1, n + 1) ** 1.2
        w /= w.sum()
        tok = np.stack([np.bincount(rng.choice(n, size=tokens, p=w), minlength=n) for _ in range(n)])
        m = tok * hidden
        # rank r sends row r and receives column r; displacements are the exclusive running sums (what
        # HcclAlltoAllVC derives from the same matrix)
        excl = lambda a: [int(x) for x in np.concatenate([[0], np.cumsum(a)[:-1]])]
        self.v = [([int(x) for x in m[r]], excl(m[r]), [int(x) for x in m[:, r]], excl(m[:, r])) for r in range(n)]
        self.tabs = [[api.u64_table(t) for t in self.v[r]] for r in range(n)]   # converted once
        self.payload = int(m.sum()) * 2
        self.send = [torch.randint(-32768, 32767, (tokens * hidden,), device="cuda:0", dtype=torch.int16)
                     for _ in range(n)]
        self.recv = [torch.empty(max(1, sum(self.v[j][2])), device="cuda:0", dtype=torch.int16) for j in range(n)]
        self.sp = [t.data_ptr() for t in self.send]
        self.rp = [t.data_ptr() for t in self.recv]

    def step(self):
        w, T = self.world, self.T
        for r in range(self.n):
            sc, sd, rc_, rd = self.tabs[r]
            rc = w.all_to_all_v(r, self.sp[r], sc, sd, self.rp[r], rc_, rd, T.BFP16, self.stream)
            assert rc == 0, rc

    def algo_bytes(self):
        return 2 * self.payload


class _NoWorld:
    def close(self):
        pass


class MoeDispatchPack(Workload):
    """The caller side of benchmark configuration 4, timed on its own: per-token destinations (Zipf 1.2) -> AlltoAllV
    tables and the stable row permutation (hcclx_moe_route), then the row gather that packs the send buffers
    (hcclx_moe_pack); 8 ranks x 4096 tokens x hidden 7168 bf16.  Algorithmic bytes: every token row read once
    and written once."""
    dtype = "u8"
    kernel = "k_moe_rows<true>"

    def __init__(self, torch, api, T, n=8, tokens=4096, hidden=7168, seed=0, combine=False, one_pass=False):
        import numpy as np
        from hccl_amd import hcclx
        self.torch, self.T, self.n, self.hx = torch, T, n, hcclx
        self.stream_obj = torch.cuda.Stream()
        self.stream = self.stream_obj.cuda_stream
        self.world = _NoWorld()
        self.combine = combine
        self.one_pass = one_pass    # route + dispatch straight into the receive buffers / combine straight out of them
        self.name = ("moe_combine_bf16_%dx%dx%d" if combine else "moe_dispatch_pack_bf16_%dx%dx%d") % (n, tokens, hidden)
        if one_pass:
            self.name = ("moe_gather_combine_bf16_%dx%dx%d" if combine else "moe_route_dispatch_bf16_%dx%dx%d") % (n, tokens, hidden)
            self.kernel = "k_moe_gather_long" if combine else "k_moe_scatter_rows<2>"
            self.profile = "profiles/%s_bf16_%dx%dx%d.txt" % ("k_moe_gather_long_combine" if combine
                                                              else "k_moe_scatter_rows_dispatch", n, tokens, hidden)
        self.tokens, self.hidden = tokens, hidden
        rng = np.random.default_rng(seed)
        w = 1.0 / np.arange(1, n + 1) ** 1.2
        w /= w.sum()
        self.dest = [torch.from_numpy(rng.choice(n, size=tokens, p=w).astype(np.int32)).to("cuda:0") for _ in range(n)]
        self.tok = [torch.randint(-32768, 32767, (tokens * hidden,), device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.packed = [torch.empty(tokens * hidden, device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.out = [torch.empty(tokens * hidden, device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.tabs = [torch.zeros(n * n, dtype=torch.int64, device="cuda:0") for _ in range(4)]
        self.perm = [torch.empty(tokens, dtype=torch.int32, device="cuda:0") for _ in range(n)]
        self.ws = torch.empty(hcclx.moe_workspace_bytes(n, tokens), dtype=torch.uint8, device="cuda:0")
        self.p = lambda ts: [t.data_ptr() for t in ts]
        self._route()
        self.hx.moe_pack(self.p(self.tok), self.p(self.perm), tokens, 1, hidden * 2, self.p(self.packed), stream=self.stream)
        if one_pass:
            # receive buffers sized for the worst case: every token of every rank
            self.recv = [torch.empty(n * tokens * hidden, device="cuda:0", dtype=torch.int16) for _ in range(n)]
            self._dispatch()

    def _dispatch(self):
        t = self.tabs
        self.hx.moe_dispatch(self.p(self.tok), self.p(self.dest), self.p(self.perm), self.tokens, 1, self.hidden, self.T.BFP16,
                             t[1].data_ptr(), t[3].data_ptr(), self.p(self.recv), stream=self.stream)

    def _route(self):
        t = self.tabs
        self.hx.moe_route(self.p(self.dest), self.tokens, self.hidden, t[0].data_ptr(), t[1].data_ptr(), t[2].data_ptr(),
                          t[3].data_ptr(), self.p(self.perm), self.ws.data_ptr(), stream=self.stream)

    def step(self):
        if self.one_pass:
            if self.combine:
                t = self.tabs
                self.hx.moe_gather_combine(self.p(self.recv), self.p(self.dest), self.p(self.perm), self.tokens, 1, self.hidden,
                                           self.T.BFP16, t[1].data_ptr(), t[3].data_ptr(), self.p(self.out), stream=self.stream)
            else:
                self._route()
                self._dispatch()
        elif self.combine:
            self.hx.moe_combine(self.p(self.packed), self.p(self.perm), self.tokens, 1, self.hidden, self.T.BFP16,
                                self.p(self.out), stream=self.stream)
        else:
            self._route()
            self.hx.moe_pack(self.p(self.tok), self.p(self.perm), self.tokens, 1, self.hidden * 2, self.p(self.packed),
                             stream=self.stream)

    def algo_bytes(self):
        return 2 * self.n * self.tokens * self.hidden * 2

    def info(self):
        if self.one_pass:
            what = "AlltoAllV back + combine in one pass" if self.combine else "route + pack + AlltoAllV in one pass"
        else:
            what = "moe combine (top-1)" if self.combine else "moe route + pack"
        return {"algorithm": what, "fused": True, "launches": 1 if self.combine else 3, "plan_cache_hit": False}


class CopyCalibration(Workload):
    """A plain device copy of 1 GiB through the fold kernel's copy instantiation: a kernel of known size,
    used to scale the HBM traffic counters of a profiler run.  Not part of the per-op table."""
    dtype = "u8"
    kernel = "hcclx::k_fold<0, 0, 1, 0>"
    profile = "profiles/k_fold_copy_1GiB_counter_calibration.txt"

    def __init__(self, torch, api, T, nbytes=1 << 30):
        from hccl_amd import hcclx
        self.torch, self.n = torch, 1
        self.stream_obj = torch.cuda.Stream()
        self.stream = self.stream_obj.cuda_stream
        self.world = None
        self.name = "copy_calibration_%dMiB" % (nbytes >> 20)
        self.nbytes = nbytes
        self.a = torch.empty(nbytes, device="cuda:0", dtype=torch.uint8).random_(0, 255)
        self.b = torch.empty(nbytes, device="cuda:0", dtype=torch.uint8)
        self.plan = hcclx.Plan([(nbytes, [self.a.data_ptr()], [self.b.data_ptr()])], T.UINT8)

    def step(self):
        self.plan.launch(self.stream)

    def algo_bytes(self):
        return 2 * self.nbytes

    def info(self):
        return {"algorithm": "copy", "fused": True, "launches": 1, "plan_cache_hit": True}


WORKLOADS = {
    "reduce_scatter_sum_bf16_mesh_8x64MiB": lambda *a: ReduceScatterMesh(*a),
    "all_reduce_sum_fp32_8x64MiB": lambda *a: AllReduce(*a),
    "all_gather_fp16_8x64MiB": lambda *a: AllGather(*a),
    "all_to_all_v_bf16_moe_8x4096x7168": lambda *a: AllToAllV(*a),
    # the same routing with 4608 tokens per rank: 66 MB sent per rank, the size the AlltoAllV target is stated for
    "all_to_all_v_bf16_moe_8x4608x7168": lambda *a: AllToAllV(*a, tokens=4608),
    "all_gather_v_fp16_16_ranks_ragged": lambda *a: AllGatherV(*a),
    # benchmark configuration 1 (8 x 1,048,576 fp32): what the selector takes at this size (the one-shot mesh
    # template: eight outputs in eight different orders, one pass), the ring template as one fused pass, and every
    # step of the ring launched through the scratch buffers (the step-faithful variant, with the ring's own larger
    # traffic)
    "all_reduce_sum_fp32_8x4MiB": lambda *a: AllReduce(
        *a, count=1048576, kernel="hcclx::k_fold<4, 0, 8, 1>",
        profile="profiles/k_fold_self_first_all_reduce_fp32_8x4MiB.txt"),
    "all_reduce_sum_fp32_8x4MiB_ring": lambda *a: AllReduce(
        *a, count=1048576, alg="InsAllReduceRing", kernel="hcclx::k_fold<4, 0, 8, 0>",
        profile="profiles/k_fold_all_reduce_ring_fp32_8x4MiB.txt"),
    "all_reduce_sum_fp32_8x4MiB_ring_step_by_step": lambda *a: AllReduce(*a, count=1048576, alg="InsAllReduceRing",
                                                                         step_mode=True),
    "all_reduce_sum_fp32_8x64MiB_two_shot_step_by_step": lambda *a: AllReduce(*a, step_mode=True),
    # communicators of more than 16 ranks: the wide chain kernel (two-shot mesh) and the wide tree kernel (NHR)
    "all_reduce_sum_fp32_32x16MiB": lambda *a: AllReduce(
        *a, n=32, count=4 * 1024 * 1024, kernel="hcclx::k_fold_wide<4, 0, 0, 4> + k_phased_copy",
        profile="profiles/k_fold_wide_k_phased_copy_all_reduce_fp32_32x16MiB.txt"),
    "all_reduce_sum_fp32_32x16MiB_nhr": lambda *a: AllReduce(
        *a, n=32, count=4 * 1024 * 1024, alg="InsAllReduceNHR", kernel="hcclx::k_fold_wide<4, 0, 2, 1> + k_phased_copy",
        profile="profiles/k_fold_wide_tree_k_phased_copy_all_reduce_nhr_fp32_32x16MiB.txt"),
    # benchmark configuration 5 at two of its sizes (the sweep below has all ten): 12 ranks, int32 MAX through the NHR
    # template and fp32 PROD through the CPU-reduce NHR template, which is what the selector takes for PROD
    "all_reduce_max_int32_12x64MiB_nhr": lambda *a: AllReduce(
        *a, n=12, count=16 * 1024 * 1024, dtype=a[2].INT32, op=a[2].MAX, alg="InsAllReduceNHR",
        kernel="hcclx::k_fold_wide<2, 2, 0, 4> + k_phased_copy",
        profile="profiles/k_fold_wide_k_phased_copy_all_reduce_nhr_int32_max_12x64MiB.txt"),
    "all_reduce_prod_fp32_12x64MiB_aicpu_nhr": lambda *a: AllReduce(
        *a, n=12, count=16 * 1024 * 1024, op=a[2].PROD, alg="InsAllReduceAicpuReduceNHR",
        kernel="hcclx::k_fold_waves<4, 1, 1, 12>",
        profile="profiles/k_fold_waves_all_reduce_aicpu_nhr_fp32_prod_12x64MiB.txt"),
    # benchmark configuration 5 names the halving-doubling template: the same two collectives through it (for fp32 its
    # schedule is a tree per slice, folded by the tree kernel, then handed out one output at a time)
    "all_reduce_max_int32_12x64MiB_rhd": lambda *a: AllReduce(
        *a, n=12, count=16 * 1024 * 1024, dtype=a[2].INT32, op=a[2].MAX, alg="InsAllReduceRHD",
        kernel="hcclx::k_fold_wide<2, 2, 0, 4> + k_phased_copy",
        profile="profiles/k_fold_wide_k_phased_copy_all_reduce_rhd_int32_max_12x64MiB.txt"),
    "all_reduce_prod_fp32_12x64MiB_rhd": lambda *a: AllReduce(
        *a, n=12, count=16 * 1024 * 1024, op=a[2].PROD, alg="InsAllReduceRHD",
        kernel="hcclx::k_fold<4, 1, 16, 2> + k_phased_copy",
        profile="profiles/k_fold_tree_k_phased_copy_all_reduce_rhd_fp32_prod_12x64MiB.txt"),
    # the same template among 8 ranks: eight orders from one pass, on the kernel that gives every wavefront one store
    "all_reduce_prod_fp32_8x64MiB_aicpu_nhr": lambda *a: AllReduce(
        *a, n=8, count=16 * 1024 * 1024, op=a[2].PROD, alg="InsAllReduceAicpuReduceNHR",
        kernel="hcclx::k_fold_waves<4, 1, 1, 8>",
        profile="profiles/k_fold_waves_all_reduce_aicpu_nhr_fp32_prod_8x64MiB.txt"),
    "reduce_scatter_sum_bf16_mesh_32x32MiB": lambda *a: ReduceScatterMesh(*a, n=32, recv=512 * 1024),
    "moe_dispatch_pack_bf16_8x4096x7168": lambda *a: MoeDispatchPack(*a),
    "moe_combine_bf16_8x4096x7168": lambda *a: MoeDispatchPack(*a, combine=True),
    "moe_route_dispatch_bf16_8x4096x7168": lambda *a: MoeDispatchPack(*a, one_pass=True),
    "moe_gather_combine_bf16_8x4096x7168": lambda *a: MoeDispatchPack(*a, combine=True, one_pass=True),
}
# not in the per-op table (the 12-rank sweep times the 1 GiB size too); profiled on their own
EXTRA_WORKLOADS = {
    "copy_calibration_1024MiB": lambda *a: CopyCalibration(*a),
    "all_reduce_max_int32_12x1GiB_nhr": lambda *a: AllReduce(
        *a, n=12, count=256 * 1024 * 1024, dtype=a[2].INT32, op=a[2].MAX, alg="InsAllReduceNHR",
        kernel="hcclx::k_fold_wide<2, 2, 0, 4> + k_phased_copy",
        profile="profiles/k_fold_wide_k_phased_copy_all_reduce_nhr_int32_max_12x1GiB.txt"),
    "all_reduce_prod_fp32_12x1GiB_aicpu_nhr": lambda *a: AllReduce(
        *a, n=12, count=256 * 1024 * 1024, op=a[2].PROD, alg="InsAllReduceAicpuReduceNHR",
        kernel="hcclx::k_fold_waves<4, 1, 1, 12>",
        profile="profiles/k_fold_waves_all_reduce_aicpu_nhr_fp32_prod_12x1GiB.txt"),
}


def sweep_allreduce_12_ranks(torch, api, T, steps):
    """benchmark configuration 5: AllReduce on 12 ranks, 4 KiB ... 1 GiB per rank in powers of 4; int32 MAX through the
    NHR and halving-doubling templates, fp32 PROD through the CPU-reduce NHR template (what the selector
    takes for PROD) and halving-doubling.  Small sizes are bound by the launch, so microseconds are reported
    beside GB/s (algorithmic bytes = 2 * 12 * size); up to 1 MiB per rank also the time per collective when 20 of
    them are replayed from one HIP graph."""
    n = 12
    cases = [("int32_max_nhr", T.INT32, T.MAX, "InsAllReduceNHR"), ("int32_max_rhd", T.INT32, T.MAX, "InsAllReduceRHD"),
             ("fp32_prod_aicpu_nhr", T.FP32, T.PROD, "InsAllReduceAicpuReduceNHR"),
             ("fp32_prod_rhd", T.FP32, T.PROD, "InsAllReduceRHD")]
    stream_obj = torch.cuda.Stream()
    out = {}
    big = 1 << 30
    # One arena for the inputs and one for the outputs, reused at every size.  The ranks' buffers start 1 GiB apart
    # (what twelve 1 GiB allocations in a row give); at the largest size the collectives are also timed with the
    # buffers 1 GiB + 8 KiB apart: at strides that are a multiple of 1 GiB the same offset of every buffer falls
    # into the same HBM channel and bank, which costs the kernels that read and write all buffers at once 10-25 %.
    stagger = 8192
    arena_in = torch.rand(n * (big + stagger) // 4, device="cuda:0") * 0.2 + 0.9
    arena_out = torch.empty(n * (big + stagger) // 4, device="cuda:0")
    for k in range(10):
        nbytes = 4096 * 4 ** k
        count = nbytes // 4
        row = {}
        for name, dt, op, alg in cases:
            w = api.World(n)
            w.set_algorithm(api.CMD_ALLREDUCE, alg)

            class Step:
                stream_obj_ = stream_obj
                stride = big

                def step(self_inner):
                    for r in range(n):
                        rc = w.all_reduce(r, arena_in.data_ptr() + r * self_inner.stride,
                                          arena_out.data_ptr() + r * self_inner.stride, count, dt, op,
                                          stream_obj.cuda_stream)
                        assert rc == 0, rc
            st = Step()
            st.stream_obj = stream_obj
            reps = max(3, min(steps, (1 << 32) // max(nbytes * n, 1)))
            # bandwidth-bound sizes are run in like the rows of the per-op table (see time_steps)
            busy = OPS_BUSY_MS if nbytes >= (1 << 24) else 0.0
            _, ms = time_steps(torch, st, reps, 2, busy_ms=busy)
            info = w.last_info()
            row[name] = {"us": round(ms * 1e3, 1), "GB/s": round(2 * n * nbytes / (ms * 1e-3) / 1e9, 1),
                         "fused": bool(info.fused), "launches": info.launches}
            if nbytes == big:
                st.stride = big + stagger
                _, ms = time_steps(torch, st, reps, 2, busy_ms=busy)
                row[name]["us_buffers_1GiB_plus_8KiB_apart"] = round(ms * 1e3, 1)
                row[name]["GB/s_buffers_1GiB_plus_8KiB_apart"] = round(2 * n * nbytes / (ms * 1e-3) / 1e9, 1)
                st.stride = big
            if nbytes <= (1 << 20):
                # launch-bound sizes: the warm collective captured 20 times into one HIP graph, so that the
                # twelve host calls per collective drop out of the replayed time
                g = torch.cuda.CUDAGraph()
                with torch.cuda.stream(stream_obj):
                    g.capture_begin()
                    for _ in range(20):
                        st.step()
                    g.capture_end()
                g.replay()
                torch.cuda.synchronize()
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(5):
                    g.replay()
                e1.record()
                torch.cuda.synchronize()
                row[name]["us_in_a_graph"] = round(e0.elapsed_time(e1) * 1e3 / 100, 2)
                del g
            w.close()
        out["%d" % nbytes] = row
    del arena_in, arena_out
    torch.cuda.empty_cache()
    return out


def small_messages_from_cpp():
    """The time per warm collective for 4 KiB ... 1 MiB per rank when a C++ caller issues the ranks' calls (the
    library's own overhead, without the Python call layer): hccl_amd/lib/latency_virtual_ranks run as a child
    process, outside every timed region of this script."""
    import subprocess
    exe = os.path.join(ROOT, "hccl_amd", "lib", "latency_virtual_ranks")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe, "300"], capture_output=True, text=True, timeout=120)
        return json.loads(out.stdout) if out.returncode == 0 else {"error": out.stderr[-300:]}
    except Exception as e:      # the figure is an extra: never let it take the benchmark line down
        return {"error": repr(e)}


def planning_from_cpp():
    """What a collective costs the host the first time (templates run, steps ordered and traced, or the template's
    closed form; tables built), on other buffers (the first plan moved there) and from then on, for every AllReduce
    and ReduceScatter template among 8, 16 and 32 ranks: hccl_amd/lib/first_call_virtual_ranks as a child process."""
    import subprocess
    exe = os.path.join(ROOT, "hccl_amd", "lib", "first_call_virtual_ranks")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe, "32"], capture_output=True, text=True, timeout=120)
        return json.loads(out.stdout) if out.returncode == 0 else {"error": out.stderr[-300:]}
    except Exception as e:      # an extra, like the small-message timings
        return {"error": repr(e)}


OPS_BUSY_MS = 30.0   # untimed run-in of every row of the per-op table


def time_steps(torch, wl, steps, warmup, busy_ms=0.0):
    """W untimed steps, then K steps bracketed by synchronisation; events sit on the launch stream.

    busy_ms (the per-op table only, never the benchmark line's workload): keep stepping untimed until the GPU has
    been busy with this workload for that long.  A train of launches that starts on an idle GPU runs its first few
    milliseconds at boost clocks and the next ten or so under the power controller's correction (the twelve-order
    fold: 265 us per launch, then up to 330, then back to 270 over forty launches); a table row of 25 steps would
    report that transient instead of the kernel."""
    import gc
    gc.collect()
    gc.disable()   # a full collection of the interpreter's heap would show up as a 40 ms step, or as an idle gap
    torch.cuda.synchronize()
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    if busy_ms > 0:   # flows into the timed steps with no more than one synchronisation between them
        t_busy = time.perf_counter()
        while (time.perf_counter() - t_busy) * 1e3 < busy_ms:
            for _ in range(10):
                wl.step()
            torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(wl.stream_obj)
    for _ in range(steps):
        wl.step()
    e1.record(wl.stream_obj)
    torch.cuda.synchronize()
    gc.enable()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps
    return wall_ms, ev_ms


# short names of the workloads for the one-number-per-op summary of the benchmark line
SHORT = {
    "reduce_scatter_sum_bf16_mesh_8x64MiB": "rs_bf16_8x64M",
    "all_reduce_sum_fp32_8x64MiB": "ar_f32_8x64M",
    "all_gather_fp16_8x64MiB": "ag_f16_8x64M",
    "all_to_all_v_bf16_moe_8x4096x7168": "a2av_moe_4096",
    "all_to_all_v_bf16_moe_8x4608x7168": "a2av_moe_4608",
    "all_gather_v_fp16_16_ranks_ragged": "agv_f16_16r",
    "all_reduce_sum_fp32_8x4MiB": "ar_f32_8x4M_oneshot",
    "all_reduce_sum_fp32_8x4MiB_ring": "ar_f32_8x4M_ring",
    "all_reduce_sum_fp32_8x4MiB_ring_step_by_step": "ar_f32_8x4M_ring_steps",
    "all_reduce_sum_fp32_8x64MiB_two_shot_step_by_step": "ar_f32_8x64M_steps",
    "all_reduce_sum_fp32_32x16MiB": "ar_f32_32x16M",
    "all_reduce_sum_fp32_32x16MiB_nhr": "ar_f32_32x16M_nhr",
    "all_reduce_max_int32_12x64MiB_nhr": "ar_i32max_12x64M_nhr",
    "all_reduce_prod_fp32_12x64MiB_aicpu_nhr": "ar_f32prod_12x64M",
    "all_reduce_prod_fp32_8x64MiB_aicpu_nhr": "ar_f32prod_8x64M",
    "all_reduce_max_int32_12x64MiB_rhd": "ar_i32max_12x64M_rhd",
    "all_reduce_prod_fp32_12x64MiB_rhd": "ar_f32prod_12x64M_rhd",
    "reduce_scatter_sum_bf16_mesh_32x32MiB": "rs_bf16_32x32M",
    "moe_dispatch_pack_bf16_8x4096x7168": "moe_pack",
    "moe_combine_bf16_8x4096x7168": "moe_combine",
    "moe_route_dispatch_bf16_8x4096x7168": "moe_route_dispatch",
    "moe_gather_combine_bf16_8x4096x7168": "moe_gather_combine",
}


def benchmark_line(args, wl, wall_ms, ev_ms, traffic, cpu=None, ops=None, small=None):
    """The benchmark line as a string: one compact JSON object that stays under LINE_LIMIT bytes.

    wl: what the headline workload is (name, dtype, n, algo_bytes, kernel, profile, info); wall_ms / ev_ms: host clock
    and HIP-event time per step; traffic: HBM bytes per step from the profile (or None); cpu: the cpu_baseline
    object; ops: {workload name: percent of the 8 TB/s peak}; small: latency-bound collectives in microseconds,
    from Python and from C++ side by side."""
    gbs = wl["algo_bytes"] / (ev_ms * 1e-3) / 1e9
    line = {
        "metric": METRIC,
        "value": round(wl["algo_bytes"] / (wall_ms * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl["dtype"],
        "data": "synthetic",
        "config": {"workload": wl["name"], "virtual_ranks": wl["n"], "algorithm": wl["info"].get("algorithm"),
                   "launches": wl["info"].get("launches"), "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 1)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "algorithmic_bytes": wl["algo_bytes"], "kernel": wl["kernel"], "kernel_us": round(ev_ms * 1e3, 2)},
    }
    if cpu is not None:
        line["cpu_baseline"] = cpu
    if ops:
        line["ops_pct_of_peak"] = {SHORT.get(k, k): v for k, v in ops.items()}
    if small:
        line["small_us"] = small
    text = json.dumps(line, separators=(",", ":"))
    if len(text.encode()) >= LINE_LIMIT:
        # never let an extra push the figures a reader needs out of its window: drop the extras, longest first
        for key in ("ops_pct_of_peak", "small_us"):
            line.pop(key, None)
            text = json.dumps(line, separators=(",", ":"))
            if len(text.encode()) < LINE_LIMIT:
                break
    assert len(text.encode()) < LINE_LIMIT, "benchmark line too long"
    return text


DETAILS_FILE = os.path.join(ROOT, "gpurun_out", "bench_details.json")


def emit_details(details):
    """The tables behind the benchmark line: one JSON object per line on stdout (before the benchmark line) and
    the whole of it in DETAILS_FILE when its folder can be written."""
    for key, val in details.items():
        print(json.dumps({"detail": key, "data": val}))
    try:
        os.makedirs(os.path.dirname(DETAILS_FILE), exist_ok=True)
        with open(DETAILS_FILE, "w") as f:
            json.dump(details, f, indent=1)
    except OSError:
        pass


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the virtual ranks all live in one MI355X's HBM; "
              "run it with --gpus 1 (no multi-GPU figure exists for this build)", file=sys.stderr)
        sys.exit(2)
    import torch
    from hccl_amd import api, hcclx
    from hccl_amd import types as T

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    hcclx.init()
    makers = dict(WORKLOADS, **EXTRA_WORKLOADS)
    if args.workload not in makers:
        print("unknown workload; choose one of: " + ", ".join(makers), file=sys.stderr)
        sys.exit(2)

    wl = makers[args.workload](torch, api, T)
    wall_ms, ev_ms = time_steps(torch, wl, args.steps, args.warmup)
    head = {"name": wl.name, "dtype": wl.dtype, "n": wl.n, "algo_bytes": wl.algo_bytes(), "kernel": wl.kernel,
            "info": wl.info()}
    traffic = profile_traffic(wl.profile, args.allow_missing_profile)
    details = {"headline": dict(head, wall_ms=wall_ms, event_ms=ev_ms, traffic_source=wl.profile)}

    ops_pct, small = None, None
    if not args.no_ops:
        ops = {}
        for name, make in WORKLOADS.items():
            if name == args.workload:
                w2, ms = wl, ev_ms
            else:
                w2 = make(torch, api, T)
                _, ms = time_steps(torch, w2, max(5, args.steps // 2), args.warmup, busy_ms=OPS_BUSY_MS)
            # GB/s: algorithmic bytes (what the op delivers, read + written) per second; pins_GB/s: the least that has to
            # cross the HBM pins per second, which is what the percentage of the 8 TB/s peak is taken from (the two
            # differ for AllGather, where one read serves n deliveries)
            g = w2.algo_bytes() / (ms * 1e-3) / 1e9
            pins = w2.pins_bytes() / (ms * 1e-3) / 1e9
            ops[name] = dict({"GB/s": round(g, 1), "pins_GB/s": round(pins, 1),
                              "pct_of_peak": round(pins / HBM_PEAK_GBS * 100, 1), "us": round(ms * 1e3, 1),
                              "profile": w2.profile if w2.profile and os.path.exists(os.path.join(ROOT, w2.profile))
                              else None}, **w2.info())
            if w2 is not wl:
                w2.world.close()
                del w2
                torch.cuda.empty_cache()
        details["ops"] = ops
        ops_pct = {k: v["pct_of_peak"] for k, v in ops.items()}
    if not args.no_ops and not args.no_sweep:
        sweep = sweep_allreduce_12_ranks(torch, api, T, args.steps)
        details["allreduce_12_ranks_sweep"] = sweep
        cpp = small_messages_from_cpp()
        if cpp is not None:
            details["small_messages_from_cpp"] = cpp
            for row in cpp.get("rows", []):
                size = sweep.get(str(row["bytes_per_rank"]), {})
                if row["ranks"] == 12 and row["case"] in size:
                    size[row["case"]]["us_from_cpp"] = row["us"]
            # benchmark configuration 1 (8 x 4 MiB fp32) is bound by launch latency: microseconds per collective
            # issued from Python (twelve ctypes calls around a 10 us kernel) next to the same collective from C++
            small = {}
            for key, case, wname in (("ar_f32_8x4M_oneshot", "fp32_sum_default", "all_reduce_sum_fp32_8x4MiB"),
                                     ("ar_f32_8x4M_ring", "fp32_sum_ring", "all_reduce_sum_fp32_8x4MiB_ring")):
                row = [r for r in cpp.get("rows", []) if r["case"] == case and r["ranks"] == 8
                       and r["bytes_per_rank"] == 4 << 20]
                if row and wname in details.get("ops", {}):
                    small[key] = {"py": details["ops"][wname]["us"], "cpp": row[0]["us"]}
        planning = planning_from_cpp()
        if planning is not None:
            details["planning_from_cpp"] = planning

    cpu = None
    if not args.no_cpu and hasattr(wl, "cpu_baseline"):
        v1, sample = wl.cpu_baseline(parallel=False)
        vp, _ = wl.cpu_baseline(parallel=True)
        cores = int(os.environ.get("OMP_NUM_THREADS") or os.cpu_count())
        cpu = {"value": round(v1, 3), "unit": "GB/s", "cores": 1, "kind": "port", "sample": sample,
               "all_cores": {"value": round(vp, 3), "cores": cores}}
        details["cpu_baseline"] = cpu
    emit_details(details)
    sys.stdout.flush()
    print(benchmark_line(args, head, wall_ms, ev_ms, traffic, cpu, ops_pct, small))


if __name__ == "__main__":
    main()
