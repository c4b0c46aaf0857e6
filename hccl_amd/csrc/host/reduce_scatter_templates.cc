// ReduceScatter algorithm templates, restated from the reference
// (src/ops/reduce_scatter/template/aicpu/):
//   InsTempReduceScatterMesh1D   ins_temp_reduce_scatter_mesh_1D.cc:65-227
//   InsTempReduceScatterNHR      ins_temp_reduce_scatter_nhr.cc:77-425
//   InsTempReduceScatterAicpuReduceNHR   ins_temp_reduce_scatter_aicpu_reduce_nhr.cc:52-300
//   InsTempReduceScatterOrderPreservedLevel1   ins_temp_reduce_scatter_order_preserved_level1.cc:52-330
//   InsTempReduceScatterOrderPreservedGroup    ins_temp_reduce_scatter_order_preserved_group.cc:63-413
// and src/ops/reduce_scatter_v/template/aicpu/:
//   InsTempReduceScatterVMesh1D  ins_temp_reduce_scatter_v_mesh_1D.cc:50-179
#include "data_move_templates.h"

namespace ops_hccl {

namespace {
bool NeedsCpuReduce(HcclDataType dt, HcclReduceOp op)
{
    return dt == HCCL_DATA_TYPE_INT64 || dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64 ||
           op == HCCL_REDUCE_PROD;
}
}  // namespace

// Every rank writes its slice k into slot <own rank> of rank k's scratch; rank k then copies its own
// slice to the output and folds the other slots in, ranks ascending.
HcclResult InsTempReduceScatterMesh1D::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                 TemplateResource &res)
{
    if (p.sliceSize == 0 && p.tailSize == 0) return HCCL_SUCCESS;
    threadNum_ = static_cast<u32>(GetThreadNum());
    CHK_PRT_RET(res.threads.size() < threadNum_, HCCL_ERROR("[RS mesh] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const u32 n = templateRankSize_;
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + threadNum_);
    auto sliceOf = [&](u32 algRank) { return (algRank == n - 1 && p.tailSize > 0) ? p.tailSize : p.sliceSize; };

    CHK_RET(PreSync(threads));
    u32 que = 1;
    for (u32 i = 1; i < n; ++i) {
        const u32 next = (me + i) % n;
        const u64 size = sliceOf(next);
        const u64 slotStride = size;  // slots are laid out with the slice size of this chunk
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][next])[0];
        std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
        for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
            txSrc.emplace_back(p.buffInfo.inputPtr,
                               p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + next * p.inputSliceStride, size,
                               size / esz);
            txDst.emplace_back(link.remoteCclMem.addr,
                               p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + me * slotStride, size,
                               size / esz);
            rxSrc.emplace_back(link.remoteCclMem.addr,
                               p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + me * p.inputSliceStride, size,
                               size / esz);
            rxDst.emplace_back(p.buffInfo.hcclBuff.addr,
                               p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + next * slotStride, size,
                               size / esz);
        }
        SendRecvInfo info{{link, link}, {{txSrc, txDst}, {rxSrc, rxDst}}, dataType_};
        CHK_RET(SendRecvBatchWrite(info, threads[que]));
        que++;
    }
    CHK_RET(PostSync(threads));
    const bool cpu = NeedsCpuReduce(dataType_, reduceOp_);
    if (cpu) {
        CHK_RET(HcommBatchModeEnd(param.algTag.c_str()));
        CHK_RET(HcommBatchModeStart(param.algTag.c_str()));
        for (ThreadHandle t : threads) CHK_RET(HcommThreadJoin(t, CUSTOM_TIMEOUT));
    }

    // PostCopy: own slice input -> output, then fold the scratch slots of the other ranks into it
    const u64 size = sliceOf(me);
    const u64 count = size / esz;
    for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
        DataSlice dst(p.buffInfo.outputPtr,
                      p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride + me * p.outputSliceStride, size, count);
        if (p.buffInfo.inBuffType != p.buffInfo.outBuffType || p.buffInfo.inBuffBaseOff != p.buffInfo.outBuffBaseOff) {
            DataSlice src(p.buffInfo.inputPtr,
                          p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + me * p.inputSliceStride, size, count);
            CHK_RET(LocalCopy(threads[0], src, dst));
        }
        for (u32 k = 0; k < n; ++k) {
            if (k == me) continue;
            DataSlice src(p.buffInfo.hcclBuff.addr, p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + k * size,
                          size, count);
            CHK_RET(LocalReduce(threads[0], src, dst, dataType_, reduceOp_));
        }
    }
    return HCCL_SUCCESS;
}

// What the steps above amount to, for the layout the sole executor passes (one repeat, equal slices, the output not
// sliced): rank r's output is its own shard r with the other ranks' shards r reduced onto it, ranks ascending.
bool InsTempReduceScatterMesh1D::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    const u32 n = templateRankSize_;
    if (n < 2 || p.repeatNum != 1 || p.tailSize != p.sliceSize || p.outputSliceStride != 0) return false;
    if (p.buffInfo.inBuffType == p.buffInfo.outBuffType) return false;   // the in-scratch variant: record it
    if (p.sliceSize == 0) return true;
    for (u32 r = 0; r < n; ++r) {
        ClosedFold f;
        f.bytes = p.sliceSize;
        const u64 inOff = p.buffInfo.inBuffBaseOff + r * p.inputSliceStride;
        f.src.push_back({r, inOff});
        for (u32 k = 0; k < n; ++k) {
            if (k != r) f.src.push_back({k, inOff});
        }
        f.dst.push_back({r, p.buffInfo.outBuffBaseOff});
        out.push_back(std::move(f));
    }
    return true;
}

// One round per shard: every rank puts its copy of shard k into slot <own rank> of its scratch, the NHR
// all-gather steps spread the slots until every rank holds all N copies, and rank k alone folds them: own
// input first, then the slots of the other ranks ascending.  N all-gathers move N times the data a
// reduce-scatter needs; the reference accepts that for PROD and 64-bit types, which its CPU has to reduce.
HcclResult InsTempReduceScatterAicpuReduceNHR::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                         TemplateResource &res)
{
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[RS AicpuReduceNHR] no thread"), HCCL_E_INTERNAL);
    if (p.sliceSize == 0) return HCCL_SUCCESS;
    dataType_ = param.DataDes.dataType;
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 size = p.sliceSize;
    const u64 count = p.count;
    const u64 rpts = p.repeatNum > 1 ? p.repeatNum : 1;
    auto slot = [&](void *buf, u64 rpt, u32 k) {  // :250-262: scratch repeats are N slots apart
        return DataSlice(buf, p.buffInfo.hcclBuffBaseOff + rpt * size * n + k * size, size, count);
    };
    std::vector<NHRStepInfo> steps;
    if (n > 1) GetNHRAllGatherSteps(n, me, steps);  // GetStepInfo :268-300

    for (u32 shard = 0; shard < n; ++shard) {
        for (u64 rpt = 0; rpt < rpts; ++rpt) {  // LocalDataCopy :82-113
            const u64 inOff = p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + shard * p.inputSliceStride;
            const u64 scOff = p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + me * size;
            if (p.buffInfo.inBuffType != p.buffInfo.hcclBuffType || inOff != scOff) {
                CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, inOff, size, count), DataSlice(ccl, scOff, size, count)));
            }
            if (shard != me) continue;  // LocalCopyToOutput :115-138
            const u64 outOff = p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride;
            if (p.buffInfo.inBuffType != p.buffInfo.outBuffType || inOff != outOff) {
                CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, inOff, size, count),
                                  DataSlice(p.buffInfo.outputPtr, outOff, size, count)));
            }
        }
        for (const NHRStepInfo &st : steps) {  // RunAllGather :180-240
            const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
            const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
            std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
            for (u64 rpt = 0; rpt < rpts; ++rpt) {
                for (u32 i = 0; i < st.nSlices; ++i) {
                    txSrc.push_back(slot(ccl, rpt, st.txSliceIdxs[i]));
                    txDst.push_back(slot(send.remoteCclMem.addr, rpt, st.txSliceIdxs[i]));
                    rxSrc.push_back(slot(recv.remoteCclMem.addr, rpt, st.rxSliceIdxs[i]));
                    rxDst.push_back(slot(ccl, rpt, st.rxSliceIdxs[i]));
                }
            }
            SendRecvInfo info{{send, recv}, {{txSrc, txDst}, {rxSrc, rxDst}}};
            // over PCIe links the receiver fetches (:62-63, :239-247)
            CHK_RET(IsPcieProtocol(res.channels) ? SendRecvRead(info, th) : SendRecvWrite(info, th));
        }
        CHK_RET(HcommBatchModeEnd(param.algTag.c_str()));  // :66-70: the CPU fold needs the data to have landed
        CHK_RET(HcommBatchModeStart(param.algTag.c_str()));
        for (ThreadHandle t : res.threads) CHK_RET(HcommThreadJoin(t, CUSTOM_TIMEOUT));
        if (shard != me) continue;
        for (u64 rpt = 0; rpt < rpts; ++rpt) {  // PostLocalReduce :140-178
            DataSlice dst(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride, size, count);
            for (u32 k = 0; k < n; ++k) {
                if (k == me) continue;
                DataSlice src(ccl, p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + k * size, size, count);
                CHK_RET(LocalReduce(th, src, dst, dataType_, reduceOp_));
            }
        }
    }
    return HCCL_SUCCESS;
}

// What the rounds above amount to: the all-gather of round k puts every rank's shard k into rank k's scratch, and
// rank k folds them onto its own in ascending rank order.  (The N rounds of N log N forwarded copies are what makes
// the recorded schedule grow with the cube of the rank count.)
bool InsTempReduceScatterAicpuReduceNHR::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    const u32 n = templateRankSize_;
    if (n == 0 || p.repeatNum > 1) return false;
    if (p.sliceSize == 0) return true;
    for (u32 k = 0; k < n; ++k) {
        ClosedFold f;
        f.bytes = p.sliceSize;
        const u64 inOff = p.buffInfo.inBuffBaseOff + k * p.inputSliceStride;
        f.src.push_back({k, inOff});
        for (u32 q = 0; q < n; ++q) {
            if (q != k) f.src.push_back({q, inOff});
        }
        f.dst.push_back({k, p.buffInfo.outBuffBaseOff});
        out.push_back(std::move(f));
    }
    return true;
}

// Shards are copied into scratch slots (slot k = shard k), the NHR reduce-scatter steps fold them across
// ranks, and the own slot is copied out.  The slices a rank sends in step 0 go straight from its input
// (ins_temp_reduce_scatter_nhr.cc:98-101, :329-332), so they are not pre-copied -- in write mode.  Over PCIe links
// the receiver fetches (read mode, :91-92, :353-363): every shard is pre-copied, because a peer can only read
// what lies in the scratch buffer.
HcclResult InsTempReduceScatterNHR::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                              TemplateResource &res)
{
    if (p.sliceSize == 0 && p.tailSize == 0) return HCCL_SUCCESS;
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[RS NHR] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    auto sizeOf = [&](u32 idx) { return (idx == n - 1 && p.tailSize > 0) ? p.tailSize : p.sliceSize; };

    const bool dmaRead = IsPcieProtocol(res.channels);
    std::vector<NHRStepInfo> steps;
    if (n > 1) GetNHRReduceScatterSteps(n, me, steps);
    std::vector<bool> sentInStep0(n, false);
    if (!steps.empty() && !dmaRead) {
        for (u32 idx : steps[0].txSliceIdxs) sentInStep0[idx] = true;
    }
    for (u32 k = 0; k < n; ++k) {
        if (sentInStep0[k]) continue;
        const u64 size = sizeOf(k);
        CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff + k * p.inputSliceStride, size),
                          DataSlice(ccl, p.buffInfo.hcclBuffBaseOff + k * p.sliceSize, size)));
    }
    for (u32 s = 0; s < steps.size(); ++s) {
        const NHRStepInfo &st = steps[s];
        const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
        const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
        std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
        for (u32 i = 0; i < st.nSlices; ++i) {
            const u32 tx = st.txSliceIdxs[i];
            const u32 rx = st.rxSliceIdxs[i];
            const u64 txOff = p.buffInfo.hcclBuffBaseOff + p.sliceSize * tx;
            const u64 rxOff = p.buffInfo.hcclBuffBaseOff + p.sliceSize * rx;
            if (s == 0 && !dmaRead) {
                txSrc.emplace_back(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff + p.inputSliceStride * tx, sizeOf(tx),
                                   sizeOf(tx) / esz);
            } else {
                txSrc.emplace_back(ccl, txOff, sizeOf(tx), sizeOf(tx) / esz);
            }
            txDst.emplace_back(send.remoteCclMem.addr, txOff, sizeOf(tx), sizeOf(tx) / esz);
            rxSrc.emplace_back(recv.remoteCclMem.addr, rxOff, sizeOf(rx), sizeOf(rx) / esz);
            rxDst.emplace_back(ccl, rxOff, sizeOf(rx), sizeOf(rx) / esz);
        }
        SendRecvReduceInfo info{{send, recv}, {{txSrc, txDst}, {rxSrc, rxDst}}, dataType_, reduceOp_};
        CHK_RET(dmaRead ? SendRecvReadReduce(info, th) : SendRecvBatchWriteReduce(info, th));
    }
    const u64 size = sizeOf(me);
    return LocalCopy(th, DataSlice(ccl, p.buffInfo.hcclBuffBaseOff + p.sliceSize * me, size),
                     DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff + me * p.outputSliceStride, size));
}

// What the steps above amount to: the rounds replayed on what every rank holds of every shard; rank r's output is
// what it ends up holding of shard r.
bool InsTempReduceScatterNHR::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    const u32 n = templateRankSize_;
    if (n < 2 || p.buffInfo.inBuffType == p.buffInfo.outBuffType) return false;
    if (p.sliceSize == 0 && p.tailSize == 0) return true;
    std::vector<SliceValues> shard(n, SliceValues(n));
    std::vector<std::vector<NHRStepInfo>> steps(n);
    for (u32 r = 0; r < n; ++r) GetNHRReduceScatterSteps(n, r, steps[r]);
    for (size_t s = 0; s < steps[0].size(); ++s) {
        for (u32 r = 0; r < n; ++r) {
            const NHRStepInfo &st = steps[r][s];
            for (u32 i = 0; i < st.nSlices; ++i) shard[st.txSliceIdxs[i]].Reduce(st.toRank, r);
        }
        for (SliceValues &v : shard) v.EndRound();
    }
    for (u32 r = 0; r < n; ++r) {
        const u64 size = (r == n - 1 && p.tailSize > 0) ? p.tailSize : p.sliceSize;
        if (size == 0) continue;
        ClosedFold f;
        shard[r].Emit(r, p.buffInfo.inBuffBaseOff + r * p.inputSliceStride, f);
        if (f.src.size() != n) return false;   // rank r must hold all of shard r
        f.bytes = size;
        f.dst.push_back({r, p.buffInfo.outBuffBaseOff + r * p.outputSliceStride});
        out.push_back(std::move(f));
    }
    return true;
}

// Ragged mesh ReduceScatter: rank k owns allRankSliceSize[k] bytes at allRankDispls[k] of every input.
// Every rank writes its part for rank k into slot <own rank> of rank k's scratch (slots are
// outputSliceStride apart); rank k copies its own part to the output and folds the other slots in,
// ranks ascending.  The main thread takes the first peer itself, so N - 1 threads are used.
HcclResult InsTempReduceScatterVMesh1D::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                  TemplateResource &res)
{
    threadNum_ = static_cast<u32>(GetThreadNum());
    CHK_PRT_RET(res.threads.size() < threadNum_, HCCL_ERROR("[RSV mesh] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.vDataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u32 n = templateRankSize_;
    CHK_PRT_RET(p.allRankSliceSize.size() != n || p.allRankDispls.size() != n,
                HCCL_ERROR("[RSV mesh] slice tables do not match the rank size"), HCCL_E_INTERNAL);
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + threadNum_);

    CHK_RET(PreSync(threads));
    for (u32 que = 0; que < threadNum_ && n > 1; ++que) {
        const u32 next = (me + 1 + que) % n;
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][next])[0];
        const u64 size = p.allRankSliceSize[next];
        std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
        for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
            txSrc.emplace_back(p.buffInfo.inputPtr,
                               p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + p.allRankDispls[next], size,
                               size / esz);
            txDst.emplace_back(link.remoteCclMem.addr,
                               p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + me * p.outputSliceStride, size,
                               size / esz);
        }
        SendRecvInfo info{{link, link}, {{txSrc, txDst}, {rxSrc, rxDst}}, dataType_};
        CHK_RET(SendRecvWrite(info, threads[que]));
    }
    CHK_RET(PostSync(threads));

    const u64 size = p.allRankSliceSize[me];
    const u64 count = size / esz;
    for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
        DataSlice dst(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride, size, count);
        DataSlice own(p.buffInfo.inputPtr,
                      p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + p.allRankDispls[me], size, count);
        CHK_RET(LocalCopy(threads[0], own, dst));
        // the CPU reduce loop runs on the host: flush what was queued so far (mesh_1D.cc:103-108)
        if (dataType_ == HCCL_DATA_TYPE_INT64 || reduceOp_ == HCCL_REDUCE_PROD) {
            CHK_RET(HcommBatchModeEnd(param.algTag.c_str()));
            CHK_RET(HcommBatchModeStart(param.algTag.c_str()));
            for (ThreadHandle t : threads) CHK_RET(HcommThreadJoin(t, CUSTOM_TIMEOUT));
        }
        for (u32 k = 0; k < n; ++k) {
            if (k == me) continue;
            DataSlice src(p.buffInfo.hcclBuff.addr,
                          p.buffInfo.hcclBuffBaseOff + rpt * p.outputRepeatStride + k * p.outputSliceStride, size, count);
            CHK_RET(LocalReduce(threads[0], src, dst, dataType_, reduceOp_));
        }
    }
    return HCCL_SUCCESS;
}

// What the steps above amount to for one repeat: rank r's output is its own part r with the other ranks' parts r
// reduced onto it, ranks ascending; a rank whose part is empty in this loop gets nothing.
bool InsTempReduceScatterVMesh1D::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    (void)esz;
    const u32 n = templateRankSize_;
    if (n < 2 || p.repeatNum != 1 || p.allRankSliceSize.size() != n || p.allRankDispls.size() != n) return false;
    if (p.buffInfo.inBuffType == p.buffInfo.outBuffType) return false;
    for (u32 r = 0; r < n; ++r) {
        if (p.allRankSliceSize[r] == 0) continue;
        ClosedFold f;
        f.bytes = p.allRankSliceSize[r];
        const u64 inOff = p.buffInfo.inBuffBaseOff + p.allRankDispls[r];
        f.src.push_back({r, inOff});
        for (u32 k = 0; k < n; ++k) {
            if (k != r) f.src.push_back({k, inOff});
        }
        f.dst.push_back({r, p.buffInfo.outBuffBaseOff});
        out.push_back(std::move(f));
    }
    return true;
}

// Strictly deterministic ReduceScatter: every rank sends shard k of its input to rank k (an all-to-all into
// scratch slots), and rank k folds the N blocks in a tree that is the same on every rank: while more than one
// block remains, with M the largest power of two below the number of blocks, block v >= M is folded into block
// v % M, then M blocks remain.  Blocks are numbered by the rank they came from, so the
// association does not depend on which rank owns the shard.
std::vector<u32> InsTempReduceScatterOrderPreservedLevel1::SendOrder(u32 me) const
{
    std::vector<u32> order;
    for (u32 i = 1; i < templateRankSize_; ++i) order.push_back((me + i) % templateRankSize_);
    return order;
}

std::vector<u32> InsTempReduceScatterOrderPreservedGroup::SendOrder(u32 me) const
{
    std::vector<u32> order;
    const u32 n = templateRankSize_;
    for (u32 distance = 1; distance <= n / 2; ++distance) {
        const u32 right = (me + distance) % n;
        const u32 left = (me + n - distance) % n;
        order.push_back(right);
        if (left != right) order.push_back(left);
    }
    return order;
}

HcclResult InsTempReduceScatterOrderPreservedLevel1::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                               TemplateResource &res)
{
    if (p.sliceSize == 0 && p.tailSize == 0) return HCCL_SUCCESS;
    const u32 n = templateRankSize_;
    threadNum_ = static_cast<u32>(res.threads.size());
    CHK_PRT_RET(threadNum_ == 0, HCCL_ERROR("[RS order preserved] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    reduceOp_ = param.reduceType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const MemBlockInfo &mb = memBlockInfo_;
    CHK_PRT_RET(mb.size.size() != n || mb.userInputOffsets.size() != n || mb.outputOffsets.size() != n,
                HCCL_ERROR("[RS order preserved] block table does not match the rank size"), HCCL_E_INTERNAL);
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    void *in = p.buffInfo.inputPtr;
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 size = mb.size[me];

    if (size != 0) {   // own shard into its slot
        CHK_RET(LocalCopy(res.threads[0], DataSlice(in, mb.userInputOffsets[me], size),
                          DataSlice(ccl, mb.outputOffsets[CalcOutputIndex(me, me)], size)));
    }
    CHK_RET(PreSync(res.threads));
    u32 que = 1;
    for (const u32 next : SendOrder(me)) {   // all-to-all: shard `next` goes to rank `next`, into the slot of this rank
        const auto ch = res.channels.find(subCommRanks_[0][next]);
        CHK_PRT_RET(ch == res.channels.end() || ch->second.empty(), HCCL_ERROR("[RS order preserved] channel not found"),
                    HCCL_E_INTERNAL);
        const ChannelInfo &link = ch->second[0];
        DataSlice txSrc(in, mb.userInputOffsets[next], mb.size[next]);
        DataSlice txDst(link.remoteCclMem.addr, mb.outputOffsets[CalcOutputIndex(next, me)], mb.size[next]);
        SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{}, {}}}, dataType_};
        CHK_RET(SendRecvWrite(info, res.threads[threadNum_ > 1 ? que : 0]));
        if (++que >= threadNum_) que = 1;
    }
    CHK_RET(PostSync(res.threads));
    if (dataType_ == HCCL_DATA_TYPE_FP64 || reduceOp_ == HCCL_REDUCE_PROD) {
        CHK_RET(HcommBatchModeEnd(param.algTag.c_str()));
        CHK_RET(HcommBatchModeStart(param.algTag.c_str()));
        for (ThreadHandle t : res.threads) CHK_RET(HcommThreadJoin(t, CUSTOM_TIMEOUT));
    }

    // the tree: block v of this rank sits in slot (v + me) % n
    u32 remaining = n;
    while (remaining > 1 && size != 0) {
        u32 m = 1;
        while (m * 2 < remaining) m *= 2;   // largest power of two below `remaining`
        for (u32 v = m; v < remaining; ++v) {
            DataSlice src(ccl, mb.outputOffsets[CalcOutputIndex(v, me)], size, size / esz);
            DataSlice dst(ccl, mb.outputOffsets[CalcOutputIndex(v % m, me)], size, size / esz);
            CHK_RET(LocalReduce(res.threads[0], src, dst, dataType_, reduceOp_));
        }
        remaining = m;
    }
    if (size != 0) {
        CHK_RET(LocalCopy(res.threads[0], DataSlice(ccl, mb.outputOffsets[CalcOutputIndex(0, me)], size),
                          DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size)));
    }
    return HCCL_SUCCESS;
}

// What the steps above amount to (whatever order the shards were sent in): every rank's output is the one tree over
// the ranks' copies of its shard, blocks numbered by the rank they came from.
bool InsTempReduceScatterOrderPreservedLevel1::ClosedForm(const TemplateDataParams &p, u64 esz,
                                                          std::vector<ClosedFold> &out) const
{
    (void)esz;
    const u32 n = templateRankSize_;
    const MemBlockInfo &mb = memBlockInfo_;
    if (n < 2 || mb.size.size() != n || mb.userInputOffsets.size() != n) return false;
    if (p.buffInfo.inBuffType == p.buffInfo.outBuffType) return false;
    SliceValues blocks(n);
    u32 remaining = n;
    while (remaining > 1) {
        u32 m = 1;
        while (m * 2 < remaining) m *= 2;
        for (u32 v = m; v < remaining; ++v) blocks.Reduce(v % m, v);
        blocks.EndRound();
        remaining = m;
    }
    for (u32 r = 0; r < n; ++r) {
        if (mb.size[r] == 0) continue;
        ClosedFold f;
        blocks.Emit(0, mb.userInputOffsets[r], f);
        f.bytes = mb.size[r];
        f.dst.push_back({r, p.buffInfo.outBuffBaseOff});
        out.push_back(std::move(f));
    }
    return true;
}

}  // namespace ops_hccl
