"""The schedule check (race + semantics) on every built-in template, and on a deliberately broken template that
is added through the plugin API from a separately compiled shared object."""
import ctypes
import os
import subprocess

import pytest

from oracle import templates as T
from hccl_amd import api, _lib

from host_util import FAKE_STREAM, fake_ptrs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SMALL_CCL = 1024 * 1024 + 64 * 1024


def checked_world(n):
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    w.set_check(True)
    return w


@pytest.mark.parametrize("n", [2, 3, 5, 8, 12, 16])
@pytest.mark.parametrize("alg", list(T.ALLREDUCE_TEMPLATES))
def test_allreduce_templates_pass_the_check(alg, n):
    w = checked_world(n)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        ins, outs = fake_ptrs(n)
        for count, dtype in ((n * 1000 + 3, T.FP32), (7, T.INT8), (90001, T.BFP16)):
            for r in range(n):
                assert w.all_reduce(r, ins[r], outs[r], count, dtype, T.SUM, FAKE_STREAM) == 0
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0, rep.firstProblem
            assert rep.steps == rep.copies + rep.reduces and rep.steps > 0 and rep.exhaustive == 1
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 3, 8, 12])
@pytest.mark.parametrize("alg", list(T.ALLREDUCE_TEMPLATES))
def test_in_place_allreduce_passes_the_check(alg, n):
    """sendBuf == recvBuf: the template's first step copies the input onto itself, which changes no byte and so
    races with no reader; every other pair of steps on the shared buffer must still be ordered."""
    w = checked_world(n)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, alg)
        ins, _ = fake_ptrs(n)
        for count, dtype, op in ((n * 1000 + 3, T.FP32, T.SUM), (7, T.INT32, T.MAX)):
            for r in range(n):
                assert w.all_reduce(r, ins[r], ins[r], count, dtype, op, FAKE_STREAM) == 0, (alg, count)
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0, rep.firstProblem
    finally:
        w.close()


@pytest.mark.parametrize("n", [2, 4, 7, 8, 13])
def test_the_other_collectives_pass_the_check(n):
    w = checked_world(n)
    try:
        ins, outs = fake_ptrs(n)
        for alg in T.REDUCE_SCATTER_TEMPLATES:
            w.set_algorithm(api.CMD_REDUCE_SCATTER, alg)
            for r in range(n):
                assert w.reduce_scatter(r, ins[r], outs[r], 30011, T.FP32, T.SUM, FAKE_STREAM) == 0
            rep = w.last_check()
            assert rep.races == 0 and rep.semanticErrors == 0, (alg, rep.firstProblem)
        counts = [(7 * k + 3) % 11 * 1000 for k in range(n)]
        displs = [sum(counts[:k]) + k for k in range(n)]
        for r in range(n):
            assert w.reduce_scatter_v(r, ins[r], counts, displs, outs[r], counts[r], T.INT32, T.MAX, FAKE_STREAM) == 0
        assert w.last_check().races == 0 and w.last_check().semanticErrors == 0, w.last_check().firstProblem
        for alg in ("InsAllGatherMesh1D", "InsAllGatherNHR"):
            w.set_algorithm(api.CMD_ALLGATHER, alg)
            for r in range(n):
                assert w.all_gather(r, ins[r], outs[r], 20001, T.FP16, FAKE_STREAM) == 0
            assert w.last_check().races == 0 and w.last_check().semanticErrors == 0, (alg, w.last_check().firstProblem)
        for r in range(n):
            assert w.all_gather_v(r, ins[r], counts[r], outs[r], counts, displs, T.FP16, FAKE_STREAM) == 0
        assert w.last_check().races == 0 and w.last_check().semanticErrors == 0, w.last_check().firstProblem
        m = [[(3 * i + 5 * j) % 7 * 500 for j in range(n)] for i in range(n)]
        v = [T.alltoallvc_to_v(m, r) for r in range(n)]
        for r in range(n):
            sc, sd, rc, rd = v[r]
            assert w.all_to_all_v(r, ins[r], sc, sd, outs[r], rc, rd, T.BFP16, FAKE_STREAM) == 0
        assert w.last_check().races == 0 and w.last_check().semanticErrors == 0, w.last_check().firstProblem
    finally:
        w.close()


PLUGIN = r'''
// Two deliberately broken AllReduce templates, registered from outside the library through the plugin macros.
#include <algorithm>
#include "host/all_reduce_templates.h"
#include "host/data_move_templates.h"
#include "host/sole_executors.h"
using namespace ops_hccl;

// "Racy": the mesh one-shot schedule, except that the fold into the output is not ordered after the receives
// (the threads are never joined), so the reduce steps race with the peers' writes.
HCCL_DECLARE_TEMPLATE(RacyOneShot, "racy", (templateRankSize_ > 1 ? templateRankSize_ : 1), templateRankSize_);
HcclResult RacyOneShot::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    const u32 n = templateRankSize_;
    const u64 size = p.sliceSize;
    const u64 esz = DATATYPE_SIZE_TABLE[param.DataDes.dataType];
    CHK_RET(LocalCopy(res.threads[0], DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, size),
                      DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size)));
    for (u32 k = 0; k < n; ++k) {
        if (k == myRank_) continue;
        const ChannelInfo &link = res.channels.at(k)[0];
        DataSlice txSrc(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, size, size / esz);
        DataSlice txDst(link.remoteCclMem.addr, myRank_ * size, size, size / esz);
        DataSlice rxSrc(link.remoteCclMem.addr, p.buffInfo.inBuffBaseOff, size, size / esz);
        DataSlice rxDst(p.buffInfo.hcclBuff.addr, k * size, size, size / esz);
        SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, param.DataDes.dataType};
        CHK_RET(SendRecvWrite(info, res.threads[k]));     // on the sub threads, with no sync back to thread 0
    }
    for (u32 k = 0; k < n; ++k) {
        if (k == myRank_) continue;
        CHK_RET(LocalReduce(res.threads[0], DataSlice(p.buffInfo.hcclBuff.addr, k * size, size, size / esz),
                            DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size, size / esz),
                            param.DataDes.dataType, param.reduceType));
    }
    return HCCL_SUCCESS;
}

// "Forgetful": every rank only adds its right-hand neighbour: ordered, race-free, and wrong.
HCCL_DECLARE_TEMPLATE(ForgetfulPair, "forgetful", 1, templateRankSize_);
HcclResult ForgetfulPair::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    const u32 n = templateRankSize_;
    const u64 size = p.sliceSize;
    const u64 esz = DATATYPE_SIZE_TABLE[param.DataDes.dataType];
    const u32 right = (myRank_ + 1) % n;
    const u32 left = (myRank_ + n - 1) % n;
    CHK_RET(LocalCopy(res.threads[0], DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, size),
                      DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size)));
    const ChannelInfo &to = res.channels.at(left)[0];
    const ChannelInfo &from = res.channels.at(right)[0];
    DataSlice txSrc(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, size, size / esz);
    DataSlice txDst(to.remoteCclMem.addr, 0, size, size / esz);
    DataSlice rxSrc(from.remoteCclMem.addr, p.buffInfo.inBuffBaseOff, size, size / esz);
    DataSlice rxDst(p.buffInfo.hcclBuff.addr, 0, size, size / esz);
    SendRecvInfo info{{to, from}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, param.DataDes.dataType};
    CHK_RET(SendRecvWrite(info, res.threads[0]));
    return LocalReduce(res.threads[0], DataSlice(p.buffInfo.hcclBuff.addr, 0, size, size / esz),
                       DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size, size / esz),
                       param.DataDes.dataType, param.reduceType);
}

// "Overreaching": the one-shot template with a closed form that names a piece beyond the end of the input.
class OverreachingOneShot : public InsTempAllReduceMesh1DOneShot {
public:
    using InsTempAllReduceMesh1DOneShot::InsTempAllReduceMesh1DOneShot;
    bool ClosedForm(const TemplateDataParams &p, u64, std::vector<ClosedFold> &out) const override
    {
        ClosedFold f;
        f.bytes = p.sliceSize;
        f.src.push_back({0, p.buffInfo.inBuffBaseOff + 64});
        f.src.push_back({1, p.buffInfo.inBuffBaseOff});
        f.dst.push_back({0, p.buffInfo.outBuffBaseOff});
        out.push_back(f);
        return true;
    }
};

// "Misstated": the two-shot template with a closed form that folds every slice in the opposite order: the right
// contributions, the wrong association.
class MisstatedTwoShot : public InsTempAllReduceMesh1DTwoShot {
public:
    using InsTempAllReduceMesh1DTwoShot::InsTempAllReduceMesh1DTwoShot;
    bool ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const override
    {
        const size_t first = out.size();
        if (!InsTempAllReduceMesh1DTwoShot::ClosedForm(p, esz, out)) return false;
        for (size_t i = first; i < out.size(); ++i) std::reverse(out[i].src.begin(), out[i].src.end());
        return true;
    }
};
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, TestMisstatedTwoShot, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 MisstatedTwoShot);

REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, TestOverreachingOneShot, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 OverreachingOneShot);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, TestRacyOneShot, InsV2AllReduceSoleExecutor, TopoMatch1D, RacyOneShot);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, TestForgetfulPair, InsV2AllReduceSoleExecutor, TopoMatch1D, ForgetfulPair);
'''


@pytest.fixture(scope="module")
def plugin(tmp_path_factory):
    d = tmp_path_factory.mktemp("plugin")
    src = d / "broken_templates.cc"
    src.write_text(PLUGIN)
    so = d / "libbroken_templates.so"
    lib_dir = os.path.dirname(_lib.LIB_PATH)
    cmd = ["g++", "-std=c++17", "-shared", "-fPIC", "-O1", "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "hccl_amd", "csrc"), str(src), "-o", str(so), "-L", lib_dir, "-lhccl_amd",
           "-Wl,-rpath," + lib_dir]
    subprocess.check_call(cmd)
    _lib.load()
    return ctypes.CDLL(str(so), mode=ctypes.RTLD_GLOBAL)


def test_a_racy_template_is_caught_before_launch(plugin):
    w = checked_world(4)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "TestRacyOneShot")
        ins, outs = fake_ptrs(4)
        rcs = [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(4)]
        assert rcs[-1] == 4                       # HCCL_E_INTERNAL from the call that would have launched
        rep = w.last_check()
        assert rep.races > 0 and b"race" in rep.firstProblem
    finally:
        w.close()


def test_a_wrong_template_is_caught_by_the_semantics_check(plugin):
    w = checked_world(4)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "TestForgetfulPair")
        ins, outs = fake_ptrs(4)
        rcs = [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(4)]
        assert rcs[-1] == 4
        rep = w.last_check()
        assert rep.races == 0 and rep.semanticErrors > 0 and b"not the reduction of every rank" in rep.firstProblem
        # without the check the schedule is taken as it is
        w.set_check(False)
        assert [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(4)][-1] == 0
    finally:
        w.close()


def test_a_closed_form_that_reaches_beyond_the_buffers_is_not_used(plugin):
    """A template may state its result in closed form; a statement that names bytes outside the call's buffers is
    dropped and the recorded steps are planned instead (here they are the one-shot template's)."""
    def trace(alg, closed_form):
        w = api.World(4, ccl_bytes=SMALL_CCL, dry=True)
        try:
            w.set_closed_form(closed_form)
            w.set_algorithm(api.CMD_ALLREDUCE, alg)
            ins, outs = fake_ptrs(4)
            for r in range(4):
                assert w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) == 0
            return w.last_trace(), w.last_info().levels
        finally:
            w.close()

    want, _ = trace("InsAllReduceMesh1DOneShot", 0)
    got, levels = trace("TestOverreachingOneShot", 2)
    assert levels > 0 and got == want


def test_a_closed_form_that_misstates_the_order_is_caught_by_the_check(plugin):
    """A template's closed form is trusted for plain launches; with the check on it is held against the recorded
    steps: the same contributions folded in another order are a different result for floats, and are rejected."""
    n = 4
    ins, outs = fake_ptrs(n)
    w = checked_world(n)
    try:
        w.set_algorithm(api.CMD_ALLREDUCE, "TestMisstatedTwoShot")
        rcs = [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(n)]
        assert rcs[-1] == 4
        rep = w.last_check()
        assert rep.races == 0 and rep.semanticErrors == 1 and b"closed form" in rep.firstProblem, rep.firstProblem
        assert b"(x0@0+(x1@0+(x2@0+x3@0)))" in rep.firstProblem       # what it states for the first piece
        # the built-in template states what it does: accepted under the same check
        w.set_algorithm(api.CMD_ALLREDUCE, "InsAllReduceMesh1DTwoShot")
        assert [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(n)][-1] == 0
        assert w.last_check().semanticErrors == 0
        # the comparison is of the statement itself, whatever the type: an integer fold would come out the same in
        # either order, the statement is still not the template's
        w.set_algorithm(api.CMD_ALLREDUCE, "TestMisstatedTwoShot")
        assert [w.all_reduce(r, ins[r], outs[r], 1000, T.INT32, T.MAX, FAKE_STREAM) for r in range(n)][-1] == 4
    finally:
        w.close()
    # unchecked and traced from its closed form, the misstatement is what would run
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        w.set_closed_form(2)
        w.set_algorithm(api.CMD_ALLREDUCE, "TestMisstatedTwoShot")
        assert [w.all_reduce(r, ins[r], outs[r], 1000, T.FP32, T.SUM, FAKE_STREAM) for r in range(n)][-1] == 0
        assert "(x0@0+(x1@0+(x2@0+x3@0)))" in w.last_trace() and w.last_info().levels == 0
    finally:
        w.close()


def run_ar(n, count, dtype, op):
    w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
    try:
        ins, outs = fake_ptrs(n)
        for r in range(n):
            assert w.all_reduce(r, ins[r], outs[r], count, dtype, op, FAKE_STREAM) == 0
        return w.last_info().algName.decode()
    finally:
        w.close()


def test_hccl_algo_environment_override(monkeypatch):
    """HCCL_ALGO with the reference's grammar (alg_env_config.cc:330-590) picks the template of the flat level."""
    monkeypatch.setenv("HCCL_ALGO", "level0:NA;level1:ring")
    assert run_ar(8, 1000, T.FP32, T.SUM) == "InsAllReduceRing"
    monkeypatch.setenv("HCCL_ALGO", " level0:NA ; level1:H-D_R ")
    assert run_ar(12, 1000, T.INT32, T.MAX) == "InsAllReduceRHD"
    monkeypatch.setenv("HCCL_ALGO", "allreduce=level0:NA;level1:NHR/allgather=level0:fullmesh")
    assert run_ar(8, 1000, T.FP32, T.SUM) == "InsAllReduceNHR"
    assert run_ar(8, 1000, T.FP32, T.PROD) == "InsAllReduceAicpuReduceNHR"
    monkeypatch.setenv("HCCL_ALGO", "others=level0:NA;level1:ring/allreduce=level0:fullmesh")
    assert run_ar(8, 1000, T.FP32, T.SUM) == "InsAllReduceMesh1DOneShot"       # fullmesh: the selector's mesh choice
    monkeypatch.setenv("HCCL_ALGO", "reducescatter=level0:NA;level1:ring")
    assert run_ar(8, 1000, T.FP32, T.SUM) == "InsAllReduceMesh1DOneShot"       # other ops are not affected
    for bad in ("level0:ring;level0:NHR", "level9:ring", "level0:fast", "level0:ring/allreduce=level0:ring",
                "level0:ring/level1:NHR", "allreduce=", "=level0:ring", "allreduce=level0:null", "transpose=level0:ring",
                "level0:ring;", "allreduce=level0:ring//allgather=level0:ring", "level0"):
        monkeypatch.setenv("HCCL_ALGO", bad)
        with pytest.raises(_lib.HcclError) as e:
            api.World(2, ccl_bytes=SMALL_CCL, dry=True)
        assert e.value.code == 1, bad
    monkeypatch.setenv("HCCL_ALGO", "  ")
    assert run_ar(8, 1000, T.FP32, T.SUM) == "InsAllReduceMesh1DOneShot"


def test_strict_determinism_selects_the_order_preserved_reduce_scatter(monkeypatch):
    """HCCL_DETERMINISTIC=strict (alg_env_config.cc:948-990): floating-point SUM / PROD among more than two ranks
    take the order-preserved template (reduce_scatter_auto_selector.cc:337-347, order_preserved_common.h:63-76)."""
    def pick_rs(n, dtype, op):
        w = api.World(n, ccl_bytes=SMALL_CCL, dry=True)
        try:
            ins, outs = fake_ptrs(n)
            rc = 0
            for r in range(n):
                rc = w.reduce_scatter(r, ins[r], outs[r], 1000, dtype, op, FAKE_STREAM)
            return rc, w.last_info().algName.decode()
        finally:
            w.close()

    monkeypatch.setenv("HCCL_DETERMINISTIC", "Strict")
    assert pick_rs(8, T.BFP16, T.SUM) == (0, "ReduceScatterOrderPreserved")
    assert pick_rs(5, T.FP64, T.PROD) == (0, "ReduceScatterOrderPreserved")
    assert pick_rs(8, T.FP32, T.MAX) == (0, "InsReduceScatterMesh1D")          # max / min need no order
    assert pick_rs(8, T.INT32, T.SUM) == (0, "InsReduceScatterMesh1D")         # integers neither
    assert pick_rs(2, T.FP32, T.SUM) == (0, "InsReduceScatterMesh1D")          # two ranks: one pairwise op
    assert pick_rs(32, T.FP32, T.SUM) == (0, "ReduceScatterOrderPreserved")
    assert pick_rs(33, T.FP32, T.SUM) == (0, "ReduceScatterOrderPreservedGroup")   # more than 32 ranks
    monkeypatch.setenv("HCCL_DETERMINISTIC", "true")
    assert pick_rs(8, T.BFP16, T.SUM) == (0, "InsReduceScatterMesh1D")
    monkeypatch.setenv("HCCL_DETERMINISTIC", "sometimes")
    with pytest.raises(_lib.HcclError) as e:
        api.World(2, ccl_bytes=SMALL_CCL, dry=True)
    assert e.value.code == 1
