"""The host runtime (templates, executors, recording, ordering, tracing, closed forms, plan building for dry worlds)
under AddressSanitizer and UndefinedBehaviorSanitizer: `make sanitize` builds host/*.cc with the host compiler and
both sanitizers into a library of its own plus a driver of dry collectives (tests/sanitize_dry_collectives.cpp); the
driver must finish without a sanitizer report and without a failed collective.  No GPU is involved."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hccl_amd", "csrc")
DRIVER = os.path.join(ROOT, "build", "csrc", "san", "sanitize_dry_collectives")


def test_dry_collectives_of_every_template_run_clean_under_asan_and_ubsan():
    build = subprocess.run(["make", "-C", CSRC, "-j", "8", "sanitize"], capture_output=True, text=True)
    assert build.returncode == 0, build.stdout[-3000:] + build.stderr[-3000:]
    env = dict(os.environ,
               ASAN_OPTIONS="abort_on_error=0:detect_leaks=1:halt_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    run = subprocess.run([DRIVER], capture_output=True, text=True, env=env, timeout=900, cwd=os.path.dirname(DRIVER))
    report = run.stdout[-2000:] + run.stderr[-6000:]
    assert "ERROR: AddressSanitizer" not in run.stderr and "runtime error:" not in run.stderr, report
    assert "ERROR: LeakSanitizer" not in run.stderr, report
    assert run.returncode == 0, report
    m = re.search(r"collectives: (\d+) failed: (\d+)", run.stdout)
    assert m and int(m.group(2)) == 0 and int(m.group(1)) >= 1000, run.stdout[-500:]
