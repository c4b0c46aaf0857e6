"""The benchmark line must stay one compact JSON object: a reader that keeps only the last 2000 characters of the
benchmark's output still has to find the metric, the roofline and the CPU baseline in it."""
import argparse
import json
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402


def canned():
    args = argparse.Namespace(steps=20, warmup=5)
    head = {"name": "reduce_scatter_sum_bf16_mesh_8x64MiB", "dtype": "bf16", "n": 8, "algo_bytes": 603979776,
            "kernel": "hcclx::k_fold_wide<11, 0, 0, 4>",
            "info": {"algorithm": "InsReduceScatterMesh1D", "fused": True, "launches": 1, "plan_cache_hit": True}}
    cpu = {"value": 0.749, "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": "the full workload (8 ranks x 64 MiB bf16, one ReduceScatter) through the oracle's C loop in the "
                     "mesh template's order, best of 6 runs",
           "all_cores": {"value": 5.77, "cores": 16}}
    ops = {name: 12345.6 for name in bench.WORKLOADS}       # the widest a percentage can print
    small = {"ar_f32_8x4M_oneshot": {"py": 1234.5, "cpp": 1234.56}, "ar_f32_8x4M_ring": {"py": 1234.5, "cpp": 1234.56}}
    return args, head, cpu, ops, small


def test_the_line_is_short_and_carries_what_the_driver_reads():
    args, head, cpu, ops, small = canned()
    text = bench.benchmark_line(args, head, 0.09591, 0.09494, 604204032, cpu, ops, small)
    assert "\n" not in text and len(text.encode()) < 2000, len(text.encode())
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["metric"] == json.load(open(os.path.join(ROOT, "BASELINE.json")))["metric"]
    assert line["config"]["workload"] == head["name"] and line["vs_baseline"] is None
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(roof["achieved"] - 603979776 / 0.09494e-3 / 1e9) < 0.1      # event time, not the host clock
    assert abs(line["value"] - 603979776 / 0.09591e-3 / 1e9) < 0.1          # host clock around the K steps
    assert roof["traffic"] == 604204032
    assert line["cpu_baseline"]["kind"] == "port" and line["cpu_baseline"]["cores"] == 1
    assert len(line["ops_pct_of_peak"]) == len(bench.WORKLOADS)             # every op has a short name


def test_every_workload_has_a_distinct_short_name():
    assert set(bench.SHORT) == set(bench.WORKLOADS)
    assert len(set(bench.SHORT.values())) == len(bench.SHORT)


def test_extras_are_dropped_before_the_line_grows_past_the_limit():
    args, head, cpu, _, small = canned()
    ops = {"a_workload_with_a_very_long_name_%03d" % i: 99.9 for i in range(60)}
    text = bench.benchmark_line(args, head, 0.1, 0.1, None, cpu, ops, small)
    assert len(text.encode()) < 2000
    line = json.loads(text)
    assert "ops_pct_of_peak" not in line and "roofline" in line and "cpu_baseline" in line


def test_the_oracle_is_only_imported_inside_the_cpu_baseline_leg():
    src = open(os.path.join(ROOT, "bench.py")).read()
    uses = [m.start() for m in re.finditer(r"^\s*(from|import)\s+oracle\b", src, re.M)]
    assert len(uses) == 1
    # the enclosing function of that import is cpu_baseline
    before = src[:uses[0]]
    assert re.findall(r"^\s*def (\w+)\(", before, re.M)[-1] == "cpu_baseline"
