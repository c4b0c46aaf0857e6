// AllGather and AllGatherV algorithm templates, restated from the reference:
//   InsTempAllGatherMesh1D    src/ops/all_gather/template/aicpu/ins_temp_all_gather_mesh_1D.cc:61-306
//   InsTempAllGatherNHR       src/ops/all_gather/template/aicpu/ins_temp_all_gather_nhr.cc:100-440
//   InsTempAllGatherVMesh1D   src/ops/all_gather_v/template/aicpu/ins_temp_all_gather_v_mesh_1D.cc:59-242
#include "data_move_templates.h"

namespace ops_hccl {

// Own block: input -> output slot and -> own scratch slot; every peer's scratch slot is then read
// straight into the output.
HcclResult InsTempAllGatherMesh1D::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    if (p.sliceSize == 0 && p.tailSize == 0) return HCCL_SUCCESS;
    threadNum_ = static_cast<u32>(GetThreadNum());
    CHK_PRT_RET(res.threads.size() < threadNum_, HCCL_ERROR("[AG mesh] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + threadNum_);
    auto sizeOf = [&](u32 idx) { return (p.tailSize != 0 && idx == n - 1) ? p.tailSize : p.sliceSize; };

    for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {  // LocalDataCopy
        const u64 inOff = p.inputSliceStride * me + p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride;
        const u64 outOff = p.outputSliceStride * me + p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride;
        const u64 cclOff = p.buffInfo.hcclBuffBaseOff + rpt * p.sliceSize * n + p.sliceSize * me;
        DataSlice src(p.buffInfo.inputPtr, inOff, sizeOf(me), sizeOf(me) / esz);
        if (!(p.buffInfo.inputPtr == p.buffInfo.outputPtr && inOff == outOff)) {
            CHK_RET(LocalCopy(threads[0], src, DataSlice(p.buffInfo.outputPtr, outOff, sizeOf(me), sizeOf(me) / esz)));
        }
        CHK_RET(LocalCopy(threads[0], src, DataSlice(p.buffInfo.hcclBuff.addr, cclOff, sizeOf(me), sizeOf(me) / esz)));
    }
    if (n == 1) return HCCL_SUCCESS;

    CHK_RET(PreSync(threads));
    for (u32 t = 0; t + 1 < n; ++t) {
        const u32 peer = (me + 1 + t) % n;
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][peer])[0];
        std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
        for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
            const u64 outBase = p.buffInfo.outBuffBaseOff + rpt * p.outputRepeatStride;
            const u64 scratchBase = p.buffInfo.hcclBuffBaseOff + rpt * p.sliceSize * n;
            const u64 size = sizeOf(peer);
            txSrc.emplace_back(p.buffInfo.outputPtr, p.outputSliceStride * me + outBase, size, size / esz);
            txDst.emplace_back(link.remoteCclMem.addr, scratchBase + p.sliceSize * me, size, size / esz);
            rxSrc.emplace_back(link.remoteCclMem.addr, scratchBase + p.sliceSize * peer, size, size / esz);
            rxDst.emplace_back(p.buffInfo.outputPtr, p.outputSliceStride * peer + outBase, size, size / esz);
        }
        SendRecvInfo info{{link, link}, {{txSrc, txDst}, {rxSrc, rxDst}}};
        CHK_RET(SendRecvRead(info, threads[t]));
    }
    return PostSync(threads);
}

// Own block -> own scratch slot; NHR all-gather steps spread the slots; all slots -> output.
HcclResult InsTempAllGatherNHR::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    if (p.sliceSize == 0 && p.tailSize == 0) return HCCL_SUCCESS;
    CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[AG NHR] no thread"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    const ThreadHandle th = res.threads[0];
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 base = p.buffInfo.hcclBuffBaseOff;
    auto sizeOf = [&](u32 idx) { return (p.tailSize != 0 && idx == n - 1) ? p.tailSize : p.sliceSize; };

    CHK_RET(LocalCopy(th, DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff + p.inputSliceStride * me, sizeOf(me)),
                      DataSlice(ccl, base + p.sliceSize * me, sizeOf(me))));
    if (n > 1) {
        std::vector<NHRStepInfo> steps;
        GetNHRAllGatherSteps(n, me, steps);
        for (const NHRStepInfo &st : steps) {
            const ChannelInfo &recv = res.channels.at(subCommRanks_[0][st.fromRank]).at(0);
            const ChannelInfo &send = res.channels.at(subCommRanks_[0][st.toRank]).at(0);
            std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
            for (u32 i = 0; i < st.nSlices; ++i) {
                const u32 tx = st.txSliceIdxs[i];
                const u32 rx = st.rxSliceIdxs[i];
                txSrc.emplace_back(ccl, base + p.sliceSize * tx, sizeOf(tx), sizeOf(tx) / esz);
                txDst.emplace_back(send.remoteCclMem.addr, base + p.sliceSize * tx, sizeOf(tx), sizeOf(tx) / esz);
                rxSrc.emplace_back(recv.remoteCclMem.addr, base + p.sliceSize * rx, sizeOf(rx), sizeOf(rx) / esz);
                rxDst.emplace_back(ccl, base + p.sliceSize * rx, sizeOf(rx), sizeOf(rx) / esz);
            }
            SendRecvInfo info{{send, recv}, {{txSrc, txDst}, {rxSrc, rxDst}}};
            // over PCIe links the receiver fetches (ins_temp_all_gather_nhr.cc:119, :320-328)
            CHK_RET(IsPcieProtocol(res.channels) ? SendRecvRead(info, th) : SendRecvBatchWrite(info, th));
        }
    }
    for (u32 k = 0; k < n; ++k) {  // PostLocalCopy
        CHK_RET(LocalCopy(th, DataSlice(ccl, base + p.sliceSize * k, sizeOf(k)),
                          DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff + p.outputSliceStride * k,
                                    sizeOf(k))));
    }
    return HCCL_SUCCESS;
}

// Own block: input -> output at displs[own]; written from there into the own slot of every peer's
// scratch; each rank then copies the peers' slots to their displacements in the output.
HcclResult InsTempAllGatherVMesh1D::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    if (p.sliceSize == 0) return HCCL_SUCCESS;
    threadNum_ = static_cast<u32>(GetThreadNum());
    CHK_PRT_RET(res.threads.size() < threadNum_, HCCL_ERROR("[AGV mesh] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.vDataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u32 n = templateRankSize_;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + threadNum_);
    const u64 outBase = p.buffInfo.outBuffBaseOff;
    const u64 myOutOff = p.allRankDispls[me] * esz + outBase;

    if (p.buffInfo.inputPtr != p.buffInfo.outputPtr) {  // LocalDataCopy
        CHK_RET(LocalCopy(threads[0],
                          DataSlice(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, p.allRankSliceSize[me], p.count),
                          DataSlice(p.buffInfo.outputPtr, myOutOff, p.allRankSliceSize[me], p.count)));
    }
    if (n == 1) return HCCL_SUCCESS;

    CHK_RET(PreSync(threads));
    for (u32 t = 0; t + 1 < n; ++t) {
        const u32 peer = (me + 1 + t) % n;
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][peer])[0];
        const u64 scratchBase = p.buffInfo.hcclBuffBaseOff;
        DataSlice txSrc(p.buffInfo.outputPtr, myOutOff, p.allRankSliceSize[me], p.count);
        DataSlice txDst(link.remoteCclMem.addr, scratchBase + p.sliceSize * me, p.allRankSliceSize[me], p.count);
        DataSlice rxSrc(link.remoteCclMem.addr, p.allRankDispls[peer] * esz + outBase, p.allRankSliceSize[peer],
                        p.count);
        DataSlice rxDst(p.buffInfo.outputPtr, scratchBase + p.sliceSize * peer, p.allRankSliceSize[peer], p.count);
        SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}};
        CHK_RET(SendRecvWrite(info, threads[t]));
    }
    CHK_RET(PostSync(threads));

    for (u32 k = 0; k < n; ++k) {  // PostLocalCopy
        if (k == me) continue;
        const u64 outOff = p.allRankDispls[k] * esz + p.allRankProcessedDataCount[k] * esz;
        CHK_RET(LocalCopy(threads[0],
                          DataSlice(p.buffInfo.hcclBuff.addr, p.buffInfo.hcclBuffBaseOff + p.sliceSize * k,
                                    p.allRankSliceSize[k], p.count),
                          DataSlice(p.buffInfo.outputPtr, outOff, p.allRankSliceSize[k], p.count)));
    }
    return HCCL_SUCCESS;
}

}  // namespace ops_hccl
