// AllReduce algorithm templates.
//
// Restated from the reference (src/ops/all_reduce/template/aicpu/):
//   InsTempAllReduceMesh1DOneShot    ins_temp_all_reduce_mesh_1D_one_shot.cc:67-199
//   InsTempAllReduceMesh1DTwoShot    ins_temp_all_reduce_mesh_1D_two_shot.cc:77-384
//   InsTempAllReduceNHR              ins_temp_all_reduce_nhr.cc:78-414
//   InsTempAllReduceAicpuReduceNHR   ins_temp_all_reduce_aicpu_reduce_nhr.cc:65-271
// Added, defined from documentation prose because the reference has no executable form of them:
//   InsTempAllReduceRing             docs/zh/user_guide/coll_algo_intro/Ring.md:5-15
//   InsTempAllReduceRHD              docs/zh/user_guide/coll_algo_intro/RHD.md:11-17, :26
// Each class emits, for its own rank, the same copies, reduces, sends and handshakes in the same order
// and through the same scratch slots as the reference's KernelRun.
#include "all_reduce_templates.h"

namespace ops_hccl {

namespace {
bool NeedsCpuReduce(HcclDataType dt, HcclReduceOp op)
{
    return dt == HCCL_DATA_TYPE_INT64 || dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64 ||
           op == HCCL_REDUCE_PROD;
}

HcclResult JoinAll(const OpParam &param, const std::vector<ThreadHandle> &threads)
{
    // the CPU reduce path flushes the task batch and joins every thread first
    CHK_RET(HcommBatchModeEnd(param.algTag.c_str()));
    CHK_RET(HcommBatchModeStart(param.algTag.c_str()));
    for (ThreadHandle t : threads) CHK_RET(HcommThreadJoin(t, CUSTOM_TIMEOUT));
    return HCCL_SUCCESS;
}
}  // namespace

// ---------------------------------------------------------------------------------------------------
// one-shot mesh: everybody writes its whole input into a slot of everybody's scratch; each rank then
// folds the slots into its output, starting from its own data
// ---------------------------------------------------------------------------------------------------
HcclResult InsTempAllReduceMesh1DOneShot::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                    TemplateResource &res)
{
    threadNum_ = static_cast<u32>(res.threads.size());
    const u64 processSize = p.sliceSize;
    const u64 count = p.count;
    dataType_ = param.DataDes.dataType;
    CHK_PRT_RET(threadNum_ != templateRankSize_, HCCL_ERROR("[OneShot] thread num is invalid"), HCCL_E_INTERNAL);

    CHK_RET(PreSync(res.threads));
    DataSlice usrIn(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, processSize, count);
    DataSlice usrOut(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, processSize, count);
    CHK_RET(LocalCopy(res.threads[0], usrIn, usrOut));
    if (templateRankSize_ > 1) {
        for (u32 q = 1; q < threadNum_; ++q) {
            const u32 peer = subCommRanks_[0][(myRank_ + q) % templateRankSize_];
            const ChannelInfo &link = res.channels.at(peer)[0];
            // slot k of a scratch buffer holds rank k's data: offset k * processSize
            DataSlice txDst(link.remoteCclMem.addr, myRank_ * processSize + p.buffInfo.hcclBuffBaseOff, processSize,
                            count);
            DataSlice rxDst(link.remoteCclMem.addr, peer * processSize + p.buffInfo.hcclBuffBaseOff, processSize,
                            count);
            SendRecvInfo info{{link, link}, {{{usrIn}, {txDst}}, {{usrIn}, {rxDst}}}, dataType_};
            CHK_RET(SendRecvBatchWrite(info, res.threads[q]));
        }
    }
    CHK_RET(PostSync(res.threads));

    if (templateRankSize_ == 1) return HCCL_SUCCESS;
    if (NeedsCpuReduce(dataType_, param.reduceType)) CHK_RET(JoinAll(param, res.threads));
    for (u32 k = 0; k < templateRankSize_; ++k) {
        if (k == myRank_) continue;
        DataSlice src(p.buffInfo.hcclBuff.addr, k * processSize + p.buffInfo.hcclBuffBaseOff, processSize, count);
        CHK_RET(LocalReduce(res.threads[0], src, usrOut, dataType_, reduceOp_));
    }
    return HCCL_SUCCESS;
}

// Every rank's output is its own data with the others' reduced onto it, ranks ascending: what the steps of the
// one-shot mesh template, and of the gather-then-fold NHR template, amount to.
static bool OwnDataThenTheOthersAscending(u32 n, const TemplateDataParams &p, std::vector<ClosedFold> &out)
{
    if (n < 2) return false;
    if (p.sliceSize == 0) return true;
    for (u32 r = 0; r < n; ++r) {
        ClosedFold f;
        f.bytes = p.sliceSize;
        f.src.push_back({r, p.buffInfo.inBuffBaseOff});
        for (u32 k = 0; k < n; ++k) {
            if (k != r) f.src.push_back({k, p.buffInfo.inBuffBaseOff});
        }
        f.dst.push_back({r, p.buffInfo.outBuffBaseOff});
        out.push_back(std::move(f));
    }
    return true;
}

bool InsTempAllReduceMesh1DOneShot::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    return OwnDataThenTheOthersAscending(templateRankSize_, p, out);
}

// ---------------------------------------------------------------------------------------------------
// two-shot mesh: scatter slice k of every rank to rank k, reduce there in slot order, gather back
// ---------------------------------------------------------------------------------------------------
HcclResult InsTempAllReduceMesh1DTwoShot::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                    TemplateResource &res)
{
    threadNum_ = static_cast<u32>(res.threads.size());
    CHK_PRT_RET(threadNum_ != templateRankSize_, HCCL_ERROR("[TwoShot] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    if (p.count == 0) return HCCL_SUCCESS;
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, templateRankSize_, esz);
    const u32 me = myRank_;
    void *in = p.buffInfo.inputPtr;
    void *out = p.buffInfo.outputPtr;
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 inBase = p.buffInfo.inBuffBaseOff;
    const u64 outBase = p.buffInfo.outBuffBaseOff;
    const u64 cclBase = p.buffInfo.hcclBuffBaseOff;

    // --- scatter
    CHK_RET(PreSync(res.threads));
    for (u32 k = 0; k < templateRankSize_; ++k) {
        const SliceInfo &send = sl[k];
        const SliceInfo &recv = sl[me];
        if (send.size == 0 && recv.size == 0) continue;
        if (k == me) {
            CHK_RET(LocalCopy(res.threads[k], DataSlice(in, inBase + send.offset, send.size, send.count),
                              DataSlice(ccl, cclBase + k * recv.size, recv.size, recv.count)));
            continue;
        }
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][k])[0];
        DataSlice txSrc(in, inBase + send.offset, send.size, send.count);
        DataSlice txDst(link.remoteCclMem.addr, cclBase + me * send.size, send.size, send.count);
        DataSlice rxSrc(link.remoteCclMem.addr, inBase + recv.offset, recv.size, recv.count);
        DataSlice rxDst(ccl, cclBase + k * recv.size, recv.size, recv.count);
        if (send.size == 0) {
            CHK_RET(RecvWrite(DataInfo(link, {{rxSrc}, {rxDst}}), res.threads[k]));
        } else if (recv.size == 0) {
            CHK_RET(SendBatchWrite(DataInfo(link, {{txSrc}, {txDst}}, dataType_), res.threads[k]));
        } else {
            SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_};
            CHK_RET(SendRecvBatchWrite(info, res.threads[k]));
        }
    }
    CHK_RET(PostSync(res.threads));
    if (NeedsCpuReduce(dataType_, param.reduceType)) CHK_RET(JoinAll(param, res.threads));

    // --- reduce into slot 0, slot after slot ("deterministic, sequential")
    if (sl[me].size != 0) {
        DataSlice dst(ccl, cclBase, sl[me].size, sl[me].count);
        for (u32 s = 1; s < templateRankSize_; ++s) {
            DataSlice src(ccl, cclBase + s * sl[me].size, sl[me].size, sl[me].count);
            CHK_RET(LocalReduce(res.threads[0], src, dst, dataType_, reduceOp_));
        }
    }

    // --- gather: everybody reads everybody's slot 0
    CHK_RET(PreSync(res.threads));
    for (u32 k = 0; k < templateRankSize_; ++k) {
        const SliceInfo &send = sl[me];
        const SliceInfo &recv = sl[k];
        if (send.size == 0 && recv.size == 0) continue;
        if (k == me) {
            CHK_RET(LocalCopy(res.threads[k], DataSlice(ccl, cclBase, send.size, send.count),
                              DataSlice(out, outBase + recv.offset, recv.size, recv.count)));
            continue;
        }
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][k])[0];
        DataSlice txSrc(ccl, cclBase, send.size, send.count);
        DataSlice txDst(link.remoteCclMem.addr, outBase + send.offset, send.size, send.count);
        DataSlice rxSrc(link.remoteCclMem.addr, cclBase, recv.size, recv.count);
        DataSlice rxDst(out, outBase + recv.offset, recv.size, recv.count);
        if (send.size == 0) {
            CHK_RET(RecvBatchRead(DataInfo(link, {{rxSrc}, {rxDst}}, dataType_), res.threads[k]));
        } else if (recv.size == 0) {
            CHK_RET(SendRead(DataInfo(link, {{txSrc}, {txDst}}, dataType_), res.threads[k]));
        } else {
            SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_};
            CHK_RET(SendRecvBatchRead(info, res.threads[k]));
        }
    }
    CHK_RET(PostSync(res.threads));
    return HCCL_SUCCESS;
}

// What the steps above amount to: slice k is the ranks' slices k folded in rank order (slot 0 first, the slots
// after it one by one), and every rank gets it.
bool InsTempAllReduceMesh1DTwoShot::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n < 2) return false;
    if (p.count == 0) return true;
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    for (u32 k = 0; k < n; ++k) {
        if (sl[k].size == 0) continue;
        ClosedFold f;
        f.bytes = sl[k].size;
        for (u32 s = 0; s < n; ++s) f.src.push_back({s, p.buffInfo.inBuffBaseOff + sl[k].offset});
        for (u32 r = 0; r < n; ++r) f.dst.push_back({r, p.buffInfo.outBuffBaseOff + sl[k].offset});
        out.push_back(std::move(f));
    }
    return true;
}

// ---------------------------------------------------------------------------------------------------
// shared by the log-step templates: one NHR step over slices that sit at the same offset in every
// rank's scratch buffer
// ---------------------------------------------------------------------------------------------------
namespace {
struct StepSlices {
    std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
};

void BuildSameOffsetStep(const NHRStepInfo &st, const std::vector<SliceInfo> &sl, void *localCcl, u64 base,
                         const ChannelInfo &send, const ChannelInfo &recv, StepSlices &o)
{
    for (u32 i = 0; i < st.nSlices; ++i) {
        const SliceInfo &t = sl[st.txSliceIdxs[i]];
        const SliceInfo &r = sl[st.rxSliceIdxs[i]];
        o.txSrc.emplace_back(localCcl, base + t.offset, t.size, t.count);
        o.txDst.emplace_back(send.remoteCclMem.addr, base + t.offset, t.size, t.count);
        o.rxSrc.emplace_back(recv.remoteCclMem.addr, base + r.offset, r.size, r.count);
        o.rxDst.emplace_back(localCcl, base + r.offset, r.size, r.count);
    }
}
}  // namespace

HcclResult InsTempAllReduceNHR::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    threadNum_ = static_cast<u32>(res.threads.size());
    CHK_PRT_RET(threadNum_ != 1, HCCL_ERROR("[NHR] thread num is invalid, need 1"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    if (p.count == 0) return HCCL_SUCCESS;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, templateRankSize_, esz);
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 base = p.buffInfo.hcclBuffBaseOff;

    // over PCIe links the receiver fetches (read mode): the same slices at the same offsets, the other verb
    // (ins_temp_all_reduce_nhr.cc:105-106, :231-239, :292-300)
    const bool dmaRead = IsPcieProtocol(res.channels);
    CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, p.sliceSize, p.count),
                      DataSlice(ccl, base, p.sliceSize, p.count)));
    if (templateRankSize_ > 1) {
        std::vector<NHRStepInfo> steps;
        GetNHRReduceScatterSteps(templateRankSize_, me, steps);
        for (const NHRStepInfo &st : steps) {
            const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
            const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
            StepSlices s;
            BuildSameOffsetStep(st, sl, ccl, base, send, recv, s);
            SendRecvReduceInfo info{{send, recv}, {{s.txSrc, s.txDst}, {s.rxSrc, s.rxDst}}, dataType_, reduceOp_};
            CHK_RET(dmaRead ? SendRecvReadReduce(info, th) : SendRecvBatchWriteReduce(info, th));
        }
        GetNHRAllGatherSteps(templateRankSize_, me, steps);
        for (const NHRStepInfo &st : steps) {
            const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
            const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
            StepSlices s;
            BuildSameOffsetStep(st, sl, ccl, base, send, recv, s);
            SendRecvInfo info{{send, recv}, {{s.txSrc, s.txDst}, {s.rxSrc, s.rxDst}}};
            CHK_RET(dmaRead ? SendRecvRead(info, th) : SendRecvWrite(info, th));
        }
    }
    return LocalCopy(th, DataSlice(ccl, base, p.sliceSize, p.count),
                     DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, p.sliceSize, p.count));
}

// What the steps above amount to: the reduce-scatter rounds replayed on what every rank holds of every slice (whose
// data, in which tree), then the all-gather rounds; every rank must end up with the same value of every slice.
bool InsTempAllReduceNHR::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n < 2) return false;
    if (p.count == 0) return true;
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    std::vector<SliceValues> slice(n, SliceValues(n));
    std::vector<std::vector<NHRStepInfo>> steps(n);
    for (int gather = 0; gather < 2; ++gather) {
        for (u32 r = 0; r < n; ++r) {
            if (gather) {
                GetNHRAllGatherSteps(n, r, steps[r]);
            } else {
                GetNHRReduceScatterSteps(n, r, steps[r]);
            }
        }
        for (size_t s = 0; s < steps[0].size(); ++s) {
            for (u32 r = 0; r < n; ++r) {
                const NHRStepInfo &st = steps[r][s];
                for (u32 i = 0; i < st.nSlices; ++i) {
                    if (gather) {
                        slice[st.txSliceIdxs[i]].Copy(st.toRank, r);
                    } else {
                        slice[st.txSliceIdxs[i]].Reduce(st.toRank, r);
                    }
                }
            }
            for (SliceValues &v : slice) v.EndRound();
        }
    }
    for (u32 k = 0; k < n; ++k) {
        if (sl[k].size == 0) continue;
        ClosedFold f;
        slice[k].Emit(0, p.buffInfo.inBuffBaseOff + sl[k].offset, f);
        f.bytes = sl[k].size;
        for (u32 r = 0; r < n; ++r) {
            if (!slice[k].Same(0, r)) return false;
            f.dst.push_back({r, p.buffInfo.outBuffBaseOff + sl[k].offset});
        }
        out.push_back(std::move(f));
    }
    return true;
}

// ---------------------------------------------------------------------------------------------------
// CPU-reduce NHR: all-gather the whole inputs into scratch slots with NHR steps, then fold the slots
// into the output, own data first (the reference runs this fold on the CPU for PROD and 64-bit types)
// ---------------------------------------------------------------------------------------------------
HcclResult InsTempAllReduceAicpuReduceNHR::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                     TemplateResource &res)
{
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[AicpuReduceNHR] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u64 sliceSize = p.sliceSize;
    const u64 count = sliceSize / esz;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 base = p.buffInfo.hcclBuffBaseOff;

    std::vector<SliceInfo> slots;  // CalcSlice :122-149: slot k = [k * chunk, +chunk)
    for (u32 k = 0; k < templateRankSize_; ++k) slots.emplace_back(k * sliceSize, sliceSize, count);

    CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, sliceSize),
                      DataSlice(ccl, base + me * sliceSize, sliceSize)));
    if (templateRankSize_ > 1) {
        std::vector<NHRStepInfo> steps;
        GetNHRAllGatherSteps(templateRankSize_, me, steps);
        for (const NHRStepInfo &st : steps) {
            const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
            const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
            StepSlices s;
            BuildSameOffsetStep(st, slots, ccl, base, send, recv, s);
            SendRecvInfo info{{send, recv}, {{s.txSrc, s.txDst}, {s.rxSrc, s.rxDst}}};
            CHK_RET(SendRecvWrite(info, th));
        }
    }
    DataSlice dst(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, sliceSize, count);
    CHK_RET(LocalCopy(th, DataSlice(ccl, base + me * sliceSize, sliceSize, count), dst));
    CHK_RET(JoinAll(param, {th}));
    for (u32 k = 0; k < templateRankSize_; ++k) {
        if (k == myRank_) continue;
        CHK_RET(LocalReduce(th, DataSlice(ccl, base + k * sliceSize, sliceSize, count), dst, dataType_, reduceOp_));
    }
    return HCCL_SUCCESS;
}

// The slots are folded in the one-shot template's order (own data, then the others ascending).
bool InsTempAllReduceAicpuReduceNHR::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    return OwnDataThenTheOthersAscending(templateRankSize_, p, out);
}

// ---------------------------------------------------------------------------------------------------
// ring (from the documentation): one lap of reduce-scatter, one lap of all-gather
// ---------------------------------------------------------------------------------------------------
HcclResult InsTempAllReduceRing::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[Ring] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    if (p.count == 0) return HCCL_SUCCESS;
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 base = p.buffInfo.hcclBuffBaseOff;

    CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, p.sliceSize, p.count),
                      DataSlice(ccl, base, p.sliceSize, p.count)));
    if (n > 1) {
        const ChannelInfo &next = res.channels.at(subCommRanks_[0][(me + 1) % n]).at(0);
        const ChannelInfo &prev = res.channels.at(subCommRanks_[0][(me + n - 1) % n]).at(0);
        for (u32 t = 0; t + 1 < n; ++t) {  // step t: pass slice (me - t) downstream, fold in slice (me - 1 - t)
            const SliceInfo &tx = sl[(me + n - t % n) % n];
            const SliceInfo &rx = sl[(me + 2 * n - 1 - t) % n];
            SendRecvReduceInfo info{{next, prev},
                                    {{{DataSlice(ccl, base + tx.offset, tx.size, tx.count)},
                                      {DataSlice(next.remoteCclMem.addr, base + tx.offset, tx.size, tx.count)}},
                                     {{DataSlice(prev.remoteCclMem.addr, base + rx.offset, rx.size, rx.count)},
                                      {DataSlice(ccl, base + rx.offset, rx.size, rx.count)}}},
                                    dataType_, reduceOp_};
            CHK_RET(SendRecvWriteReduce(info, th));
        }
        for (u32 t = 0; t + 1 < n; ++t) {  // rank r finished slice r + 1; pass it on, then what arrives
            const SliceInfo &tx = sl[(me + 1 + n - t % n) % n];
            const SliceInfo &rx = sl[(me + 2 * n - t) % n];
            SendRecvInfo info{{next, prev},
                              {{{DataSlice(ccl, base + tx.offset, tx.size, tx.count)},
                                {DataSlice(next.remoteCclMem.addr, base + tx.offset, tx.size, tx.count)}},
                               {{DataSlice(prev.remoteCclMem.addr, base + rx.offset, rx.size, rx.count)},
                                {DataSlice(ccl, base + rx.offset, rx.size, rx.count)}}},
                              dataType_};
            CHK_RET(SendRecvWrite(info, th));
        }
    }
    return LocalCopy(th, DataSlice(ccl, base, p.sliceSize, p.count),
                     DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, p.sliceSize, p.count));
}

// What the two laps amount to: slice c starts as rank c's data, goes round the ring once with every rank's data
// reduced in as it passes (the partial result arrives and is the source operand), and ends up on every rank.
bool InsTempAllReduceRing::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n < 2) return false;
    if (p.count == 0) return true;
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    for (u32 c = 0; c < n; ++c) {
        if (sl[c].size == 0) continue;
        ClosedFold f;
        f.bytes = sl[c].size;
        f.accIsSource = true;
        for (u32 k = 0; k < n; ++k) f.src.push_back({(c + k) % n, p.buffInfo.inBuffBaseOff + sl[c].offset});
        for (u32 r = 0; r < n; ++r) f.dst.push_back({r, p.buffInfo.outBuffBaseOff + sl[c].offset});
        out.push_back(std::move(f));
    }
    return true;
}

// ---------------------------------------------------------------------------------------------------
// recursive halving-doubling (from the documentation), any rank count
// ---------------------------------------------------------------------------------------------------
void RhdBlock(u32 n, u32 &extra, std::vector<u32> &block)
{
    u32 p2 = 1;
    while (p2 * 2 <= n) p2 *= 2;
    extra = n - p2;
    block.clear();
    for (u32 i = 0; i < extra; ++i) block.push_back(2 * i);
    for (u32 r = 2 * extra; r < n; ++r) block.push_back(r);
}

HcclResult InsTempAllReduceRHD::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[RHD] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    if (p.count == 0) return HCCL_SUCCESS;
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    u32 extra = 0;
    std::vector<u32> block;
    RhdBlock(n, extra, block);
    const u32 p2 = static_cast<u32>(block.size());
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, p2, esz);
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 base = p.buffInfo.hcclBuffBaseOff;
    auto chan = [&](u32 algRank) -> const ChannelInfo & { return res.channels.at(subCommRanks_[0][algRank]).at(0); };
    DataSlice whole(ccl, base, p.sliceSize, p.count);

    CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, p.sliceSize, p.count), whole));

    const bool folded = me < 2 * extra && (me & 1);  // odd rank of a fold pair: hands its data over and waits
    if (folded) {
        const ChannelInfo &c = chan(me - 1);
        DataSlice dst(c.remoteCclMem.addr, base, p.sliceSize, p.count);
        CHK_RET(HcommChannelNotifyWaitOnThread(th, c.handle, NOTIFY_IDX_ACK, CUSTOM_TIMEOUT));
        CHK_RET(HcommWriteReduceOnThread(th, c.handle, GetSliceAddr(dst), GetSliceAddr(whole), p.count, dataType_,
                                         reduceOp_));
        CHK_RET(HcommChannelNotifyRecordOnThread(th, c.handle, NOTIFY_IDX_DATA_SIGNAL));
        CHK_RET(RecvWrite(DataInfo(c, {{dst}, {whole}}), th));  // the result comes back at the end
    } else {
        if (me < 2 * extra) CHK_RET(RecvWrite(DataInfo(chan(me + 1), {{whole}, {whole}}), th));
        u32 b = 0;
        for (u32 i = 0; i < p2; ++i) {
            if (block[i] == me) b = i;
        }
        u32 steps = 0;
        while ((1u << steps) < p2) ++steps;
        u32 lo = 0;
        u32 hi = p2;  // slice range this block rank still owns
        std::vector<std::pair<u32, u32>> kept;
        for (u32 s = 0; s < steps; ++s) {
            const u32 mid = (lo + hi) / 2;
            const bool upper = (b >> s) & 1;
            const u32 giveLo = upper ? lo : mid;
            const u32 giveHi = upper ? mid : hi;
            const u32 keepLo = upper ? mid : lo;
            const u32 keepHi = upper ? hi : mid;
            const ChannelInfo &c = chan(block[b ^ (1u << s)]);
            StepSlices x;
            for (u32 k = giveLo; k < giveHi; ++k) {
                x.txSrc.emplace_back(ccl, base + sl[k].offset, sl[k].size, sl[k].count);
                x.txDst.emplace_back(c.remoteCclMem.addr, base + sl[k].offset, sl[k].size, sl[k].count);
            }
            for (u32 k = keepLo; k < keepHi; ++k) {
                x.rxSrc.emplace_back(c.remoteCclMem.addr, base + sl[k].offset, sl[k].size, sl[k].count);
                x.rxDst.emplace_back(ccl, base + sl[k].offset, sl[k].size, sl[k].count);
            }
            SendRecvReduceInfo info{{c, c}, {{x.txSrc, x.txDst}, {x.rxSrc, x.rxDst}}, dataType_, reduceOp_};
            CHK_RET(SendRecvWriteReduce(info, th));
            kept.emplace_back(lo, hi);
            lo = keepLo;
            hi = keepHi;
        }
        for (u32 s = steps; s-- > 0;) {  // all-gather: send what I hold, receive the partner's part
            const ChannelInfo &c = chan(block[b ^ (1u << s)]);
            const u32 fullLo = kept[s].first;
            const u32 fullHi = kept[s].second;
            StepSlices x;
            for (u32 k = lo; k < hi; ++k) {
                x.txSrc.emplace_back(ccl, base + sl[k].offset, sl[k].size, sl[k].count);
                x.txDst.emplace_back(c.remoteCclMem.addr, base + sl[k].offset, sl[k].size, sl[k].count);
            }
            for (u32 k = fullLo; k < fullHi; ++k) {
                if (k >= lo && k < hi) continue;
                x.rxSrc.emplace_back(c.remoteCclMem.addr, base + sl[k].offset, sl[k].size, sl[k].count);
                x.rxDst.emplace_back(ccl, base + sl[k].offset, sl[k].size, sl[k].count);
            }
            SendRecvInfo info{{c, c}, {{x.txSrc, x.txDst}, {x.rxSrc, x.rxDst}}, dataType_};
            CHK_RET(SendRecvWrite(info, th));
            lo = fullLo;
            hi = fullHi;
        }
        if (me < 2 * extra) {  // restore the folded neighbour
            const ChannelInfo &c = chan(me + 1);
            CHK_RET(SendWrite(DataInfo(c, {{whole}, {DataSlice(c.remoteCclMem.addr, base, p.sliceSize, p.count)}},
                                       dataType_),
                              th));
        }
    }
    return LocalCopy(th, whole, DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, p.sliceSize, p.count));
}

// What the steps above amount to: the fold of the odd ranks and the halving rounds replayed on what every rank holds
// of every slice; the doubling rounds and the way back to the folded ranks hand every finished slice to everybody.
bool InsTempAllReduceRHD::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n < 2) return false;
    if (p.count == 0) return true;
    u32 extra = 0;
    std::vector<u32> block;
    RhdBlock(n, extra, block);
    const u32 p2 = static_cast<u32>(block.size());
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, p2, esz);
    std::vector<SliceValues> slice(p2, SliceValues(n));
    for (u32 i = 0; i < extra; ++i) {
        for (SliceValues &v : slice) v.Reduce(2 * i, 2 * i + 1);
    }
    for (SliceValues &v : slice) v.EndRound();
    u32 steps = 0;
    while ((1u << steps) < p2) ++steps;
    std::vector<u32> lo(p2, 0), hi(p2, p2);   // slice range every block rank still owns
    for (u32 s = 0; s < steps; ++s) {
        for (u32 b = 0; b < p2; ++b) {
            const u32 mid = (lo[b] + hi[b]) / 2;
            const bool upper = (b >> s) & 1;
            const u32 partner = block[b ^ (1u << s)];
            for (u32 k = upper ? lo[b] : mid; k < (upper ? mid : hi[b]); ++k) slice[k].Reduce(partner, block[b]);
            if (upper) {
                lo[b] = mid;
            } else {
                hi[b] = mid;
            }
        }
        for (SliceValues &v : slice) v.EndRound();
    }
    std::vector<u32> owner(p2, 0);
    for (u32 b = 0; b < p2; ++b) {
        if (hi[b] != lo[b] + 1) return false;
        owner[lo[b]] = block[b];
    }
    for (u32 k = 0; k < p2; ++k) {
        if (sl[k].size == 0) continue;
        ClosedFold f;
        slice[k].Emit(owner[k], p.buffInfo.inBuffBaseOff + sl[k].offset, f);
        if (f.src.size() != n) return false;
        f.bytes = sl[k].size;
        for (u32 r = 0; r < n; ++r) f.dst.push_back({r, p.buffInfo.outBuffBaseOff + sl[k].offset});
        out.push_back(std::move(f));
    }
    return true;
}

}  // namespace ops_hccl
