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
                     "hcclx_alltoallv", "hcclx_allgatherv", "hcclx_moe_route", "hcclx_moe_pack", "hcclx_moe_combine",
                     "hcclx_fold_wide", "hcclx_plan_create_wide", "hcclx_plan_table_bytes", "hcclx_moe_dispatch",
                     "hcclx_moe_gather_combine", "hcclx_displs_from_counts"):
        assert expected in names, f"{expected} is not declared in include/"
    missing = [f"{n} ({h})" for n, h in sorted(names.items()) if not hasattr(lib, n)]
    assert not missing, "declared but not exported: " + ", ".join(missing)
    assert len(names) >= 50


C_PROGRAM = r'''
#include <stdio.h>
#include <stdint.h>
#include "hccl.h"
#include "hccl_comm.h"
#include "hcclx.h"
#include "hcomm_primitives.h"
int main(void)
{
    HcclComm comm[4];
    uint32_t n = 0, id = 9;
    char trace[4096];
    hcclxLastOpInfo info;
    hcclxCheckReport rep;
    if (hcclxCommInitAll(4, 0, 1, comm) != HCCL_SUCCESS) return 1;
    if (HcclGetRankSize(comm[2], &n) != HCCL_SUCCESS || n != 4) return 2;
    if (HcclGetRankId(comm[2], &id) != HCCL_SUCCESS || id != 2) return 3;
    hcclxCommSetCheck(comm[0], 1);
    hcclxCommSetTrace(comm[0], 1);
    for (int r = 0; r < 4; ++r) {
        void *in = (void *)(uintptr_t)(0x100000000000ull + (uint64_t)r * 0x1000000000ull);
        void *out = (void *)(uintptr_t)(0x200000000000ull + (uint64_t)r * 0x1000000000ull);
        if (HcclAllReduce(in, out, 1000, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm[r], (aclrtStream)1) != HCCL_SUCCESS) return 4;
    }
    hcclxCommGetLastOpInfo(comm[0], &info);
    hcclxCommGetLastCheck(comm[0], &rep);
    hcclxCommGetLastTrace(comm[0], trace, sizeof(trace));
    printf("%s fused=%d steps=%u races=%u semantic=%u\n%.60s\n", info.algName, info.fused, rep.steps, rep.races, rep.semanticErrors, trace);
    if (HcclAllReduce(0, 0, 1000, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm[0], (aclrtStream)1) != HCCL_E_PTR) return 5;
    {
        /* the kernel layer's structures as a C caller fills them; without a GPU the call reports an error */
        hcclx_wide_seg_t wide = {0};
        hcclx_seg_t seg = {0};
        wide.count = 4; wide.nsrc = 20; wide.ndst = 1;
        seg.count = 4; seg.nsrc = 2; seg.ndst = 1;
        if (sizeof(wide.src) / sizeof(wide.src[0]) != HCCLX_MAX_WIDE_FAN || sizeof(seg.dst) / sizeof(seg.dst[0]) != HCCLX_MAX_FAN) return 7;
        if (hcclx_plan_table_bytes(0) != 0 || hcclx_plan_bytes(0) != 0) return 8;
    }
    for (int r = 0; r < 4; ++r) HcclCommDestroy(comm[r]);
    return (rep.races == 0 && rep.semanticErrors == 0) ? 0 : 6;
}
'''


def test_headers_are_plain_c_and_a_c_program_drives_a_dry_world(tmp_path):
    """gcc -std=c99 -pedantic -Werror on all four headers; the program makes a dry world of four ranks, runs a
    checked and traced HcclAllReduce, and reads the reports back."""
    import subprocess
    c = tmp_path / "c_abi.c"
    c.write_text(C_PROGRAM)
    exe = tmp_path / "c_abi"
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                           str(c), "-o", str(exe), "-L", lib_dir, "-lhccl_amd", "-Wl,-rpath," + lib_dir])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "InsAllReduceMesh1DOneShot fused=1" in out.stdout and "races=0 semantic=0" in out.stdout
    assert "rank 0 out[0,4000) = (x3@0+(x2@0+(x1@0+x0@0)))" in out.stdout


def test_no_compute_entry_point_runs_without_a_gpu_silently():
    """Without a GPU the kernel layer reports an error instead of falling back to anything."""
    import torch
    if torch.cuda.is_available():
        return
    lib = _lib.load()
    assert lib.hcclx_init() != 0
    assert lib.hcclx_last_error() != b""
    assert lib.hcclx_dtype_size(11) == 2 and lib.hcclx_dtype_size(99) == 0      # pure host helpers still work
