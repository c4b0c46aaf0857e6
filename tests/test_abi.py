"""The C-ABI library loads without a GPU and exports every function the headers under include/ declare."""
import ctypes
import glob
import os
import re

from hccl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)          # comments
        text = re.sub(r"//[^\n]*", " ", text)
        text = re.sub(r"^\s*#[^\n]*(\\\n[^\n]*)*", " ", text, flags=re.M)   # preprocessor lines
        text = re.sub(r"typedef\s+(struct|enum)\s*\w*\s*\{.*?\}\s*\w+\s*;", " ", text, flags=re.S)
        for m in re.finditer(r"\b([A-Za-z_]\w*)\s*\(([^;{}()]|\([^()]*\))*\)\s*;", text):
            name = m.group(1)
            if name in ("defined", "sizeof", "__attribute__"):
                continue
            names[name] = os.path.basename(path)
    return names


def test_every_declared_function_is_exported():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    # the headers declare the public ops, the communicator calls, the primitives and the kernel layer
    for expected in ("HcclAllReduce", "HcclReduceScatter", "HcclReduceScatterV", "HcclAllGather", "HcclAllGatherV",
                     "HcclAlltoAll", "HcclAlltoAllV", "HcclAlltoAllVC", "HcclCommInitAll", "hcclxCommInitAll",
                     "hcclxCommSetCheck", "HcommLocalCopyOnThread", "HcommLocalReduceOnThread", "HcommWriteReduceOnThread",
                     "HcommChannelNotifyWaitOnThread", "HcommThreadJoin", "hcclx_fold", "hcclx_plan_create",
                     "hcclx_alltoallv", "hcclx_allgatherv", "hcclx_moe_route", "hcclx_moe_pack", "hcclx_moe_combine"):
        assert expected in names, f"{expected} is not declared in include/"
    missing = [f"{n} ({h})" for n, h in sorted(names.items()) if not hasattr(lib, n)]
    assert not missing, "declared but not exported: " + ", ".join(missing)
    assert len(names) >= 45


def test_no_compute_entry_point_runs_without_a_gpu_silently():
    """Without a GPU the kernel layer reports an error instead of falling back to anything."""
    import torch
    if torch.cuda.is_available():
        return
    lib = _lib.load()
    assert lib.hcclx_init() != 0
    assert lib.hcclx_last_error() != b""
    assert lib.hcclx_dtype_size(11) == 2 and lib.hcclx_dtype_size(99) == 0      # pure host helpers still work
