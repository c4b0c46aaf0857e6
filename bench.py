#!/usr/bin/env python3
"""Benchmark of the collective hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input that is already resident in HBM:
by default the ReduceScatter SUM bf16 of 8 virtual ranks x 33,554,432 elements (64 MiB per rank), mesh
template order, each output shard a fused 8-way reduce in one HBM pass.  `value` is the effective HBM
bandwidth: algorithmic bytes (every input byte read once + every output byte written once) divided by
the time of a step.  One JSON line is printed.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-ops]
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


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="reduce_scatter_sum_bf16_mesh_8x64MiB")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-ops", action="store_true", help="skip the per-op table")
    return ap.parse_args()


# ----------------------------------------------------------------------------------------------------
# workloads: each builds device buffers once and exposes step() = one launch of the hot path
# ----------------------------------------------------------------------------------------------------

class Workload:
    name = ""
    dtype = ""
    kernel = ""          # name of the dominant kernel as rocprofv3 prints it (prefix)

    def __init__(self, torch, hcclx, T):
        self.torch, self.hcclx, self.T = torch, hcclx, T
        self.stream = torch.cuda.current_stream().cuda_stream

    def step(self):
        raise NotImplementedError

    def algo_bytes(self):
        raise NotImplementedError


def _randn_bits16(torch, n, seed, dt):
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    return torch.randn(n, device="cuda:0", generator=g, dtype=torch.float32).to(dt)


class ReduceScatterMesh(Workload):
    """BASELINE config 2: ReduceScatter SUM bf16, mesh template, N ranks x (N * recv) elements in.
    Output shard r folds slice r of every rank starting from rank r's own data, then ranks ascending
    (ins_temp_reduce_scatter_mesh_1D.cc:132-154), fused into one pass."""
    dtype = "bf16"
    kernel = "hcclx::k_fold<11, 0, 8, 0>"

    def __init__(self, torch, hcclx, T, n=8, recv=4 * 1024 * 1024):
        super().__init__(torch, hcclx, T)
        self.name = "reduce_scatter_sum_bf16_mesh_%dx%dMiB" % (n, n * recv * 2 >> 20)
        self.n, self.recv = n, recv
        self.x = [_randn_bits16(torch, n * recv, 1000 + r, torch.bfloat16) for r in range(n)]
        self.out = [torch.empty(recv, device="cuda:0", dtype=torch.bfloat16) for _ in range(n)]
        segs = []
        for r in range(n):
            order = [r] + [k for k in range(n) if k != r]
            segs.append((recv, [self.x[k].data_ptr() + r * recv * 2 for k in order], [self.out[r].data_ptr()]))
        self.plan = hcclx.Plan(segs, T.BFP16, T.SUM)

    def step(self):
        self.plan.launch(self.stream)

    def algo_bytes(self):
        return (self.n + 1) * self.n * self.recv * 2

    def cpu_baseline(self, parallel):
        """The oracle's restatement of the same template on the same shape, timed on the host."""
        import numpy as np
        T = self.T
        rng = np.random.default_rng(0)
        xs = [T.narrow16(rng.standard_normal(self.n * self.recv, dtype=np.float32), T.BFP16) for _ in range(self.n)]
        best = None
        for _ in range(2):
            t0 = time.perf_counter()
            T.run_reduce_scatter(T.NumericElems(T.BFP16, T.SUM, parallel=parallel), xs, self.recv, 2,
                                 "InsReduceScatterMesh1D")
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return self.algo_bytes() / best / 1e9, "full workload (8 ranks x 64 MiB bf16), best of 2 runs"


class AllReduceOneShotOrder(Workload):
    """AllReduce SUM fp32, N ranks: every rank's output is the fold that starts from its own data
    (one-shot mesh order, ins_temp_all_reduce_mesh_1D_one_shot.cc:182-197); inputs read once."""
    dtype = "f32"

    def __init__(self, torch, hcclx, T, n=8, count=16 * 1024 * 1024):
        super().__init__(torch, hcclx, T)
        self.name = "all_reduce_sum_fp32_%dx%dMiB" % (n, count * 4 >> 20)
        self.n, self.count = n, count
        g = torch.Generator(device="cuda:0")
        g.manual_seed(7)
        self.x = [torch.rand(count, device="cuda:0", generator=g) * 2 - 1 for _ in range(n)]
        self.out = [torch.empty(count, device="cuda:0") for _ in range(n)]
        self.plan = hcclx.Plan([(count, [t.data_ptr() for t in self.x], [t.data_ptr() for t in self.out])],
                               T.FP32, T.SUM, hcclx.FOLD_SELF_FIRST)

    def step(self):
        self.plan.launch(self.stream)

    def algo_bytes(self):
        return 2 * self.n * self.count * 4


class AllGather(Workload):
    """AllGather fp16: every rank's block lands in every output; read once, written N times."""
    dtype = "u8"

    def __init__(self, torch, hcclx, T, n=8, count=32 * 1024 * 1024):
        super().__init__(torch, hcclx, T)
        self.name = "all_gather_fp16_%dx%dMiB" % (n, count * 2 >> 20)
        self.n, self.count = n, count
        self.x = [torch.randint(-32768, 32767, (count,), device="cuda:0", dtype=torch.int16) for _ in range(n)]
        self.out = [torch.empty(n * count, device="cuda:0", dtype=torch.int16) for _ in range(n)]
        segs = [(count, [self.x[i].data_ptr()], [o.data_ptr() + i * count * 2 for o in self.out]) for i in range(n)]
        self.plan = hcclx.Plan(segs, T.FP16)

    def step(self):
        self.plan.launch(self.stream)

    def algo_bytes(self):
        return 2 * self.n * self.n * self.count * 2


class AllToAllV(Workload):
    """BASELINE config 4 shape: MoE dispatch, N ranks x tokens x hidden bf16, destinations Zipf(1.2),
    tokens grouped by destination; count/displacement tables resident on the device."""
    dtype = "u8"

    def __init__(self, torch, hcclx, T, n=8, tokens=4096, hidden=7168, seed=0):
        import numpy as np
        super().__init__(torch, hcclx, T)
        self.name = "all_to_all_v_bf16_moe_%dx%dx%d" % (n, tokens, hidden)
        rng = np.random.default_rng(seed)
        w = 1.0 / np.arange(1, n + 1) ** 1.2
        w /= w.sum()
        tok = np.stack([np.bincount(rng.choice(n, size=tokens, p=w), minlength=n) for _ in range(n)])
        sc = (tok * hidden).astype(np.uint64)
        sd = np.zeros_like(sc)
        sd[:, 1:] = np.cumsum(sc, 1)[:, :-1]
        rc = sc.T.copy()
        rd = np.zeros_like(rc)
        rd[:, 1:] = np.cumsum(rc, 1)[:, :-1]
        self.n = n
        self.payload = int(sc.sum()) * 2
        self.send = [torch.randint(-32768, 32767, (tokens * hidden,), device="cuda:0", dtype=torch.int16)
                     for _ in range(n)]
        self.recv = [torch.empty(max(1, int(rc[j].sum())), device="cuda:0", dtype=torch.int16) for j in range(n)]
        self.tab = torch.from_numpy(np.concatenate([sc.ravel(), sd.ravel(), rd.ravel()]).astype(np.int64)).to("cuda:0")
        self.sp = [t.data_ptr() for t in self.send]
        self.rp = [t.data_ptr() for t in self.recv]

    def step(self):
        p, nn = self.tab.data_ptr(), self.n * self.n * 8
        self.hcclx.alltoallv(self.sp, self.rp, p, p + nn, p + 2 * nn, self.T.BFP16, on_device=True,
                             stream=self.stream)

    def algo_bytes(self):
        return 2 * self.payload


WORKLOADS = {
    "reduce_scatter_sum_bf16_mesh_8x64MiB": lambda *a: ReduceScatterMesh(*a),
    "all_reduce_sum_fp32_8x64MiB": lambda *a: AllReduceOneShotOrder(*a),
    "all_gather_fp16_8x64MiB": lambda *a: AllGather(*a),
    "all_to_all_v_bf16_moe_8x4096x7168": lambda *a: AllToAllV(*a),
}


def time_steps(torch, wl, steps, warmup):
    for _ in range(warmup):
        wl.step()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        wl.step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps
    return wall_ms, ev_ms


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the virtual ranks all live in one MI355X's HBM; "
              "run it with --gpus 1 (no multi-GPU figure exists for this build)", file=sys.stderr)
        sys.exit(2)
    import torch
    from hccl_amd import hcclx
    from oracle import templates as T   # cpu_baseline leg only

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    hcclx.init()
    if args.workload not in WORKLOADS:
        print("unknown workload; choose one of: " + ", ".join(WORKLOADS), file=sys.stderr)
        sys.exit(2)

    wl = WORKLOADS[args.workload](torch, hcclx, T)
    wall_ms, ev_ms = time_steps(torch, wl, args.steps, args.warmup)
    gbs = wl.algo_bytes() / (ev_ms * 1e-3) / 1e9
    line = {
        "metric": "effective HBM GB/s (and % of peak) per op at 64MB/rank, 8 virtual ranks",
        "value": round(wl.algo_bytes() / (wall_ms * 1e-3) / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl.dtype,
        "data": "synthetic",
        "config": {"workload": wl.name, "virtual_ranks": 8, "algorithmic_bytes": wl.algo_bytes(),
                   "pct_of_hbm_peak": round(gbs / HBM_PEAK_GBS * 100, 1)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": wl.kernel,
                     "kernel_us": round(ev_ms * 1e3, 2)},
    }

    if not args.no_ops:
        ops = {}
        for name, make in WORKLOADS.items():
            if name == args.workload:
                w2, ms = wl, ev_ms
            else:
                w2 = make(torch, hcclx, T)
                _, ms = time_steps(torch, w2, max(5, args.steps // 2), args.warmup)
            g = w2.algo_bytes() / (ms * 1e-3) / 1e9
            ops[name] = {"GB/s": round(g, 1), "pct_of_peak": round(g / HBM_PEAK_GBS * 100, 1), "us": round(ms * 1e3, 1)}
            if w2 is not wl:
                del w2
                torch.cuda.empty_cache()
        line["ops"] = ops

    if not args.no_cpu and hasattr(wl, "cpu_baseline"):
        v1, sample = wl.cpu_baseline(parallel=False)
        vp, _ = wl.cpu_baseline(parallel=True)
        line["cpu_baseline"] = {"value": round(v1, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                                "sample": sample,
                                "all_cores": {"value": round(vp, 3), "cores": os.cpu_count()}}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
