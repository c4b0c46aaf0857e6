"""The bottom boundary by symbol lookup: a template compiled outside the library reaches every data-plane
primitive the way the reference does -- dlopen, then dlsym by name
(src/common/hcomm_dlsym/hcomm_dlsym.cc:62-70, hcomm_primitives_dl.cc:100-125) -- and drives a world without a GPU
through the function pointers, the batch descriptor call included."""
import ctypes
import os
import re
import subprocess

import pytest

from oracle import templates as T
from hccl_amd import api, _lib

from host_util import FAKE_STREAM, fake_ptrs, parse_trace

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SMALL_CCL = 1024 * 1024 + 64 * 1024

# every function include/hcomm_primitives.h declares: the names a loader has to find
HEADER = open(os.path.join(ROOT, "include", "hcomm_primitives.h")).read()
NAMES = sorted(set(re.findall(r"\b(Hcomm[A-Za-z]+)\s*\(", HEADER)))

PLUGIN = r'''
// A mesh one-shot AllReduce written against function pointers only: every primitive is found with dlsym.
#include <dlfcn.h>
#include <cstdio>
#include "host/data_move_templates.h"
#include "host/sole_executors.h"
using namespace ops_hccl;

namespace {
struct Table {
    int32_t (*LocalCopy)(ThreadHandle, void *, const void *, uint64_t) = nullptr;
    int32_t (*LocalReduce)(ThreadHandle, void *, const void *, uint64_t, HcommDataType, HcommReduceOp) = nullptr;
    int32_t (*Write)(ThreadHandle, ChannelHandle, void *, const void *, uint64_t) = nullptr;
    int32_t (*Read)(ThreadHandle, ChannelHandle, void *, const void *, uint64_t) = nullptr;
    int32_t (*WriteReduce)(ThreadHandle, ChannelHandle, void *, const void *, uint64_t, HcommDataType, HcommReduceOp) = nullptr;
    int32_t (*ReadReduce)(ThreadHandle, ChannelHandle, void *, const void *, uint64_t, HcommDataType, HcommReduceOp) = nullptr;
    int32_t (*ChannelRecord)(ThreadHandle, ChannelHandle, uint32_t) = nullptr;
    int32_t (*ChannelWait)(ThreadHandle, ChannelHandle, uint32_t, uint32_t) = nullptr;
    int32_t (*ThreadRecord)(ThreadHandle, ThreadHandle, uint32_t) = nullptr;
    int32_t (*ThreadWait)(ThreadHandle, uint32_t, uint32_t) = nullptr;
    int32_t (*Batch)(ThreadHandle, ChannelHandle, const HcclHcommBatchTransferDesc *, uint32_t) = nullptr;
    int32_t (*BatchModeStart)(const char *) = nullptr;
    int32_t (*BatchModeEnd)(const char *) = nullptr;
    int32_t (*ThreadJoin)(ThreadHandle, uint32_t) = nullptr;
    // the process-wide time-out and the waits that use it, which the reference's wrapper tries first
    // (hcomm_primitives_dl.h:95-105)
    int32_t (*SetNotifyWaitTimeOut)(uint32_t) = nullptr;
    int32_t (*ThreadResAcquireTimeOut)(uint32_t) = nullptr;
    int32_t (*ThreadWaitDefault)(ThreadHandle, uint32_t) = nullptr;
    int32_t (*ChannelWaitDefault)(ThreadHandle, ChannelHandle, uint32_t) = nullptr;
    int32_t (*WriteWithNotify)(ThreadHandle, ChannelHandle, void *, const void *, uint64_t, uint32_t) = nullptr;
    int32_t (*ChannelFence)(ThreadHandle, ChannelHandle) = nullptr;
    int missing = -1;
};
Table g;

template <typename F> void Find(void *lib, const char *name, F *slot)
{
    *slot = reinterpret_cast<F>(dlsym(lib, name));
    if (*slot == nullptr) {
        std::fprintf(stderr, "dlsym(%s) failed\n", name);
        g.missing++;
    }
}
}  // namespace

// Called by the test with the path of the library: the loader of the reference, pointed at this backend.
extern "C" int LoadPrimitives(const char *path)
{
    void *lib = dlopen(path, RTLD_NOW);
    if (lib == nullptr) return -1;
    g.missing = 0;
    Find(lib, "HcommLocalCopyOnThread", &g.LocalCopy);
    Find(lib, "HcommLocalReduceOnThread", &g.LocalReduce);
    Find(lib, "HcommWriteOnThread", &g.Write);
    Find(lib, "HcommReadOnThread", &g.Read);
    Find(lib, "HcommWriteReduceOnThread", &g.WriteReduce);
    Find(lib, "HcommReadReduceOnThread", &g.ReadReduce);
    Find(lib, "HcommChannelNotifyRecordOnThread", &g.ChannelRecord);
    Find(lib, "HcommChannelNotifyWaitOnThread", &g.ChannelWait);
    Find(lib, "HcommThreadNotifyRecordOnThread", &g.ThreadRecord);
    Find(lib, "HcommThreadNotifyWaitOnThread", &g.ThreadWait);
    Find(lib, "HcommBatchTransferOnThread", &g.Batch);
    Find(lib, "HcommBatchModeStart", &g.BatchModeStart);
    Find(lib, "HcommBatchModeEnd", &g.BatchModeEnd);
    Find(lib, "HcommThreadJoin", &g.ThreadJoin);
    Find(lib, "HcommSetNotifyWaitTimeOut", &g.SetNotifyWaitTimeOut);
    Find(lib, "HcommThreadResAcquireTimeOut", &g.ThreadResAcquireTimeOut);
    Find(lib, "HcommThreadNotifyWaitOnThreadWithDefaultTimeout", &g.ThreadWaitDefault);
    Find(lib, "HcommChannelNotifyWaitOnThreadWithDefaultTimeout", &g.ChannelWaitDefault);
    Find(lib, "HcommWriteWithNotifyNbiOnThread", &g.WriteWithNotify);
    Find(lib, "HcommChannelFenceOnThread", &g.ChannelFence);
    if (g.missing == 0 && (g.SetNotifyWaitTimeOut(1800) != 0 || g.ThreadResAcquireTimeOut(1800) != 0)) return -2;
    return g.missing;
}

// Own data to the output; the own input written into slot <own rank> of every peer's scratch buffer through the batch
// call, between the ACK / DATA_SIGNAL handshakes; then the peers' slots folded in, ranks ascending.  One thread.
HCCL_DECLARE_TEMPLATE(DlsymOneShot, "one-shot mesh through dlsym'ed primitives", templateRankSize_, 1);
HcclResult DlsymOneShot::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    if (g.missing != 0) return HCCL_E_INTERNAL;
    const u32 n = templateRankSize_;
    const u64 size = p.sliceSize;
    const u64 count = size / DATATYPE_SIZE_TABLE[param.DataDes.dataType];
    const ThreadHandle t = res.threads[0];
    char *in = static_cast<char *>(p.buffInfo.inputPtr) + p.buffInfo.inBuffBaseOff;
    char *out = static_cast<char *>(p.buffInfo.outputPtr) + p.buffInfo.outBuffBaseOff;
    char *ccl = static_cast<char *>(p.buffInfo.hcclBuff.addr);
    if (g.BatchModeStart(param.algTag.c_str()) != 0) return HCCL_E_INTERNAL;
    if (g.LocalCopy(t, out, in, size) != 0) return HCCL_E_INTERNAL;
    for (u32 k = 0; k < n; ++k) {
        if (k == myRank_) continue;
        const ChannelInfo &link = res.channels.at(k)[0];
        if (g.ChannelRecord(t, link.handle, NOTIFY_IDX_ACK) != 0) return HCCL_E_INTERNAL;       // my slot is free
        if (g.ChannelWaitDefault(t, link.handle, NOTIFY_IDX_ACK) != 0) return HCCL_E_INTERNAL;   // so is the peer's
        if (k % 2 == 1) {
            // odd peers: the write that records its notify, behind a fence; then the wait with the default time-out
            if (g.ChannelFence(t, link.handle) != 0) return HCCL_E_INTERNAL;
            if (g.WriteWithNotify(t, link.handle, static_cast<char *>(link.remoteCclMem.addr) + myRank_ * size, in, size,
                                  NOTIFY_IDX_DATA_SIGNAL) != 0) return HCCL_E_INTERNAL;
            if (g.ChannelWaitDefault(t, link.handle, NOTIFY_IDX_DATA_SIGNAL) != 0) return HCCL_E_INTERNAL;
            continue;
        }
        HcclHcommBatchTransferDesc d[2] = {};
        d[0].transType = HCCL_HCOMM_TRANSFER_TYPE_WRITE;
        d[0].transferInfo.write.len = size;
        d[0].transferInfo.write.dst = static_cast<char *>(link.remoteCclMem.addr) + myRank_ * size;
        d[0].transferInfo.write.src = in;
        d[1].transType = HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_RECORD;
        d[1].transferInfo.notifyRecord.notifyIdx = NOTIFY_IDX_DATA_SIGNAL;
        if (g.Batch(t, link.handle, d, 2) != 0) return HCCL_E_INTERNAL;
        if (g.ChannelWait(t, link.handle, NOTIFY_IDX_DATA_SIGNAL, 1800) != 0) return HCCL_E_INTERNAL;
    }
    if (g.BatchModeEnd(param.algTag.c_str()) != 0 || g.ThreadJoin(t, 1800) != 0) return HCCL_E_INTERNAL;
    for (u32 k = 0; k < n; ++k) {
        if (k == myRank_) continue;
        if (g.LocalReduce(t, out, ccl + k * size, count, param.DataDes.dataType, param.reduceType) != 0) return HCCL_E_INTERNAL;
    }
    return HCCL_SUCCESS;
}
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, TestDlsymOneShot, InsV2AllReduceSoleExecutor, TopoMatch1D, DlsymOneShot);
'''


@pytest.fixture(scope="module")
def plugin(tmp_path_factory):
    d = tmp_path_factory.mktemp("dlsym_plugin")
    src = d / "dlsym_template.cc"
    src.write_text(PLUGIN)
    so = d / "libdlsym_template.so"
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    # -lhccl_amd only for the executor / template base classes and the registry; the primitives are NOT linked:
    # the template calls them through dlsym'ed pointers
    cmd = ["g++", "-std=c++17", "-shared", "-fPIC", "-O1", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "hccl_amd", "csrc"), str(src), "-o", str(so), "-L", lib_dir, "-lhccl_amd", "-ldl",
           "-Wl,-rpath," + lib_dir]
    subprocess.check_call(cmd)
    _lib.load()
    lib = ctypes.CDLL(str(so), mode=ctypes.RTLD_GLOBAL)
    lib.LoadPrimitives.argtypes = [ctypes.c_char_p]
    lib.LoadPrimitives.restype = ctypes.c_int
    return lib, str(so)


def test_every_declared_primitive_is_found_by_name(plugin):
    lib, so = plugin
    assert lib.LoadPrimitives(_lib.LIB_PATH.encode()) == 0
    # the template's own object has no undefined reference to a primitive: it can only reach them through dlsym
    undefined = subprocess.run(["nm", "-D", "--undefined-only", so], capture_output=True, text=True, check=True).stdout
    assert not re.search(r"\bHcomm[A-Za-z]+OnThread\b", undefined), undefined
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in NAMES:
        assert hasattr(handle, name), name
    assert "HcommBatchTransferOnThread" in NAMES and "HcommChannelNotifyWaitOnThreadWithDefaultTimeout" in NAMES
    assert len(NAMES) == 20


@pytest.mark.parametrize("n", [2, 3, 5])
def test_a_template_on_dlsymed_primitives_runs_a_checked_dry_world(plugin, n):
    lib, _ = plugin
    assert lib.LoadPrimitives(_lib.LIB_PATH.encode()) == 0
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_check(True)
        w.set_algorithm(api.CMD_ALLREDUCE, "TestDlsymOneShot")
        ins, outs = fake_ptrs(n)
        count = 1000
        for r in range(n):
            assert w.all_reduce(r, ins[r], outs[r], count, T.FP32, T.SUM, FAKE_STREAM) == 0
        rep = w.last_check()
        assert rep.races == 0 and rep.semanticErrors == 0, rep.firstProblem
        assert rep.copies == n * n and rep.reduces == n * (n - 1)     # one copy to the output + n-1 writes per rank
        assert w.last_info().fused == 1
        rows = parse_trace(w.last_trace())
        assert len(rows) == n
        for rank, off, length, expr in rows:
            assert (off, length) == (0, count * 4)
            want = f"x{rank}@0"
            for k in range(n):
                if k != rank:
                    want = f"(x{k}@0+{want})"
            assert expr == want, (rank, expr)
    finally:
        w.close()
