"""The C++ example (hccl_amd/examples/allreduce_virtual_ranks.cpp, built beside the library) calls the public API the way
an application of the reference does; it checks its own result."""
import os
import subprocess

import pytest

from hccl_amd import _lib

pytestmark = pytest.mark.gpu
EXE = os.path.join(os.path.dirname(_lib.LIB_PATH), "allreduce_virtual_ranks")


@pytest.mark.parametrize("ranks,mib", [(8, 4), (12, 1), (32, 2)])
def test_cpp_caller_of_the_public_api(ranks, mib):
    assert os.path.exists(EXE), f"{EXE} is missing: build it with `make -C hccl_amd/csrc`"
    out = subprocess.run([EXE, str(ranks), str(mib)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "-- OK" in out.stdout and "one pass, 1 launch(es)" in out.stdout, out.stdout
