"""Guards on the layout: the product never reaches into the CPU oracle or the scratch folder, and the benchmark refuses
to pretend there is more than one GPU."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def product_files():
    for base, _, names in os.walk(os.path.join(ROOT, "hccl_amd")):
        if os.sep + "lib" in base:
            continue
        for name in names:
            if name.endswith((".py", ".h", ".hip", ".cc", ".cpp")) or name == "Makefile":
                yield os.path.join(base, name)


def test_the_library_and_its_python_face_never_touch_the_oracle():
    offenders = []
    for path in product_files():
        text = open(path, encoding="utf-8").read()
        if re.search(r"^\s*(from|import)\s+oracle\b", text, re.M) or "liboracle" in text or "elem_oracle" in text:
            offenders.append(os.path.relpath(path, ROOT))
    assert not offenders, "product code reaches into oracle/: " + ", ".join(offenders)


def test_nothing_committed_reads_the_scratch_folder():
    offenders = []
    tracked = subprocess.run(["git", "-C", ROOT, "ls-files"], capture_output=True, text=True).stdout.split()
    for rel in tracked:
        if not rel.endswith((".py", ".h", ".hip", ".cc", ".cpp", ".c", ".sh")) and os.path.basename(rel) != "Makefile":
            continue
        if rel == os.path.relpath(__file__, ROOT):
            continue
        path = os.path.join(ROOT, rel)
        if os.path.exists(path) and "_work/" in open(path, encoding="utf-8").read():
            offenders.append(rel)
    assert not offenders, "committed files name _work/: " + ", ".join(offenders)


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0
    assert "one GPU" in out.stderr and out.stdout.strip() == ""
