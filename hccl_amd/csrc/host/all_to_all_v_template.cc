// AlltoAllV mesh template, restated from the reference
// (src/ops/all_to_all_v/template/aicpu/ins_temp_all_to_all_v_mesh_1D.cc:75-440), one channel per peer.
// Write mode: the block for rank j is packed into a slot of rank j's scratch buffer, rank j unpacks it to
// rdispls[i] of its output.  Read mode (PCIe links, :137-139, :194-206, :291-294, :343-359): the block for rank j is
// packed into a slot of the sender's OWN scratch buffer and rank j fetches it straight into its output.  The own
// block is copied directly in both.  Peers are visited in rounds of at most 16, left and right neighbours at
// growing distance, and each pair of ranks agrees on its slots through the distance between them.
#include <algorithm>

#include "data_move_templates.h"

namespace ops_hccl {

void InsTempAlltoAllVMesh1D::CalcCommRankSetForOneLoop(u32 roundIdx, u32 remainRankSize,
                                                       std::vector<u32> &commRanks) const
{
    commRanks.clear();
    const u32 conc = Concurrent();
    const u32 pairNumPerRound = (conc + 1) / 2;
    const u32 pairSize = (remainRankSize < conc) ? (remainRankSize + 1) / 2 : pairNumPerRound;
    for (u32 i = roundIdx * pairNumPerRound + 1; i < roundIdx * pairNumPerRound + pairSize + 1; ++i) {
        const u32 left = (myRank_ + templateRankSize_ - i % templateRankSize_) % templateRankSize_;
        const u32 right = (myRank_ + i) % templateRankSize_;
        commRanks.push_back(left);
        if (left == right) break;
        commRanks.push_back(right);
    }
}

void InsTempAlltoAllVMesh1D::CalcCclBuffIdx(u32 remoteRank, u32 &myRankCclBuffIdx, u32 &remoteCclBuffIdx) const
{
    const u32 pairNum = (Concurrent() + 1) / 2;
    const u32 gapRight = (templateRankSize_ + remoteRank - myRank_) % templateRankSize_;
    const u32 gapLeft = (templateRankSize_ + myRank_ - remoteRank) % templateRankSize_;
    if (gapLeft < gapRight) {
        myRankCclBuffIdx = pairNum - 1 - ((gapLeft - 1) % pairNum);
        remoteCclBuffIdx = pairNum + ((gapLeft - 1) % pairNum);
    } else if (gapLeft > gapRight) {
        myRankCclBuffIdx = pairNum + ((gapRight - 1) % pairNum);
        remoteCclBuffIdx = pairNum - 1 - ((gapRight - 1) % pairNum);
    } else {
        myRankCclBuffIdx = 0;
        remoteCclBuffIdx = 0;
    }
}

HcclResult InsTempAlltoAllVMesh1D::KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res)
{
    threadNum_ = static_cast<u32>(res.threads.size());
    CHK_PRT_RET(threadNum_ < GetThreadNum(), HCCL_ERROR("[A2AV mesh] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.all2AllVDataDes.sendType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + GetThreadNum());
    const u32 conc = Concurrent();
    const u32 commLoops = conc ? (templateRankSize_ - 1 + conc - 1) / conc : 0;
    u32 remain = templateRankSize_ - 1;

    const bool dmaRead = IsPcieProtocol(res.channels);
    // PreCopy (:412-423): the block for `remote` into the slot of the own scratch buffer that `remote` reads
    auto preCopy = [&](u32 remote) -> HcclResult {
        if (p.sendCounts[remote] == 0) return HCCL_SUCCESS;
        u32 mySlot = 0;
        u32 remoteSlot = 0;
        CalcCclBuffIdx(remote, mySlot, remoteSlot);
        const u64 sendSize = p.sendCounts[remote] * esz;
        return LocalCopy(threads[mySlot + 1],
                         DataSlice(p.buffInfo.inputPtr, p.sdispls[remote] * esz, sendSize, p.sendCounts[remote]),
                         DataSlice(p.buffInfo.hcclBuff.addr, mySlot * p.inputSliceStride + p.buffInfo.hcclBuffBaseOff,
                                   sendSize, p.sendCounts[remote]));
    };

    CHK_RET(PreSync(threads));
    if (commLoops == 0 && p.sendCounts[me] > 0) {  // a single rank still moves its own block
        CHK_RET(LocalCopy(threads[0],
                          DataSlice(p.buffInfo.inputPtr, p.sdispls[me] * esz, p.sendCounts[me] * esz, p.sendCounts[me]),
                          DataSlice(p.buffInfo.outputPtr, p.rdispls[me] * esz, p.recvCounts[me] * esz,
                                    p.recvCounts[me])));
    }
    std::vector<u32> commRanks;
    for (u32 round = 0; round < commLoops && remain > 0; ++round) {
        CalcCommRankSetForOneLoop(round, remain, commRanks);
        if (dmaRead && round == 0) {
            // the first round packs all its blocks before anything else, then joins the threads so that the own
            // block's copy does not run beside them (:194-203)
            for (u32 remote : commRanks) CHK_RET(preCopy(remote));
            if (threads.size() > 1) {
                CHK_RET(PostSync(threads));
                CHK_RET(PreSync(threads));
            }
        }
        if (round == 0 && p.sendCounts[me] > 0) {  // LocalCopyForMyRank
            CHK_RET(LocalCopy(threads[0],
                              DataSlice(p.buffInfo.inputPtr, p.sdispls[me] * esz, p.sendCounts[me] * esz,
                                        p.sendCounts[me]),
                              DataSlice(p.buffInfo.outputPtr, p.rdispls[me] * esz, p.recvCounts[me] * esz,
                                        p.recvCounts[me])));
        }
        for (u32 remote : commRanks) {
            auto it = res.channels.find(remote);
            CHK_PRT_RET(it == res.channels.end(), HCCL_ERROR("[A2AV mesh] remoteRank[%u] has no channel", remote),
                        HCCL_E_PARA);
            const ChannelInfo &link = it->second[0];
            u32 mySlot = 0;
            u32 remoteSlot = 0;
            CalcCclBuffIdx(remote, mySlot, remoteSlot);
            const ThreadHandle th = threads[mySlot + 1];
            if (dmaRead && round != 0) CHK_RET(preCopy(remote));   // :291-294
            const u64 sendSize = p.sendCounts[remote] * esz;
            const u64 recvSize = p.recvCounts[remote] * esz;
            DataSlice txSrc(p.buffInfo.inputPtr, p.sdispls[remote] * esz, sendSize, p.sendCounts[remote]);
            DataSlice txDst(link.remoteCclMem.addr, remoteSlot * p.inputSliceStride + p.buffInfo.hcclBuffBaseOff,
                            sendSize, p.sendCounts[remote]);
            DataSlice rxSrc(link.remoteCclMem.addr, remoteSlot * p.inputSliceStride + p.buffInfo.hcclBuffBaseOff,
                            recvSize, p.recvCounts[remote]);
            DataSlice rxDst(p.buffInfo.outputPtr, p.rdispls[remote] * esz, recvSize, p.recvCounts[remote]);
            if (dmaRead) {   // RunSendRecv, read branch (:343-359): the peer's slot straight into the output
                if (sendSize > 0 && recvSize > 0) {
                    SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_};
                    CHK_RET(SendRecvRead(info, th));
                } else if (sendSize > 0) {
                    CHK_RET(SendRead(DataInfo(link, {{txSrc}, {txDst}}, dataType_), th));
                } else if (recvSize > 0) {
                    CHK_RET(RecvRead(DataInfo(link, {{rxSrc}, {rxDst}}, dataType_), th));
                }
                continue;
            }
            if (sendSize > 0 && recvSize > 0) {
                SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_};
                CHK_RET(SendRecvWrite(info, th));
            } else {
                if (sendSize > 0) CHK_RET(SendWrite(DataInfo(link, {{txSrc}, {txDst}}, dataType_), th));
                if (recvSize > 0) CHK_RET(RecvWrite(DataInfo(link, {{rxSrc}, {rxDst}}, dataType_), th));
            }
            if (recvSize > 0) {  // PostCopy: own scratch slot -> output
                CHK_RET(LocalCopy(th,
                                  DataSlice(p.buffInfo.hcclBuff.addr,
                                            mySlot * p.inputSliceStride + p.buffInfo.hcclBuffBaseOff, recvSize,
                                            p.recvCounts[remote]),
                                  rxDst));
            }
        }
        remain -= static_cast<u32>(commRanks.size());
    }
    return PostSync(threads);
}

}  // namespace ops_hccl
