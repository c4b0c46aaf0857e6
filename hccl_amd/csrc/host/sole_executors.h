// The "sole" executors: one chunk loop per op between the op entry and a template.  They are class templates
// over (topology match, algorithm template), so that REGISTER_EXEC_V2 can pair them with a template that is
// defined outside this library.
//
// Reference: src/ops/<op>/executor/ins_v2_<op>_sole_executor.cc (cited per class below).
#pragma once
#include <algorithm>

#include "data_move_templates.h"
#include "executor.h"

namespace ops_hccl {

namespace detail {

inline void FillBuffInfo(const OpParam &param, const AlgResourceCtxSerializable &resCtx, TemplateDataParams &t,
                  TemplateResource &res)
{
    res.channels = resCtx.channels;
    res.threads = resCtx.threads;
    t.buffInfo.inputPtr = param.inputPtr;
    t.buffInfo.outputPtr = param.outputPtr;
    t.buffInfo.inputSize = param.inputSize;
    t.buffInfo.outputSize = param.outputSize;
    t.buffInfo.hcclBuff = resCtx.cclMem;
    t.buffInfo.inBuffType = BufferType::INPUT;
    t.buffInfo.outBuffType = BufferType::OUTPUT;
    t.buffInfo.hcclBuffType = BufferType::HCCL_BUFFER;
    t.enableRemoteMemAccess = (param.opMode == OpMode::OFFLOAD);
    t.repeatNum = 1;
    t.inputRepeatStride = 0;
    t.outputRepeatStride = 0;
}

}  // namespace detail

// ---------------------------------------------------------------------------------------------------
// AllReduce (src/ops/all_reduce/executor/ins_v2_all_reduce_sole_executor.cc:92-185)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate> class InsV2AllReduceSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "AllReduce sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.DataDes.dataType;
        dataCount_ = param.DataDes.count;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        return Loops(alg, t, [&]() { return alg.KernelRun(param, t, res); });
    }
    bool ClosedForm(const OpParam &param, u32 rankSize, u64 cclBytes, std::vector<ClosedFold> &out) override
    {
        dataType_ = param.DataDes.dataType;
        dataCount_ = param.DataDes.count;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        TemplateDataParams t;
        t.buffInfo.hcclBuff.size = cclBytes;
        t.buffInfo.inBuffType = BufferType::INPUT;
        t.buffInfo.outBuffType = BufferType::OUTPUT;
        t.buffInfo.hcclBuffType = BufferType::HCCL_BUFFER;
        t.repeatNum = 1;
        InsAlgTemplate alg(param, 0, AlgTopoMatch::Match(rankSize));
        bool all = true;
        const HcclResult res = Loops(alg, t, [&]() {
            all = all && alg.ClosedForm(t, dataTypeSize_, out);
            return HCCL_SUCCESS;
        });
        return res == HCCL_SUCCESS && all;
    }

private:
    // The chunk loop (:120-185): `body` runs once per chunk with `t` describing it.
    template <typename F> HcclResult Loops(InsAlgTemplate &alg, TemplateDataParams &t, F &&body)
    {
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, maxTmpMemSize_) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[AllReduce executor] maxDataCountPerLoop is 0"), HCCL_E_INTERNAL);
        const u64 loops = dataCount_ / maxCount + (dataCount_ % maxCount != 0);
        u64 done = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            const u64 cur = (loop == loops - 1) ? dataCount_ - done : maxCount;
            t.count = cur;
            t.buffInfo.inBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.sliceSize = cur * dataTypeSize_;
            t.tailSize = t.sliceSize;
            t.inputSliceStride = 0;
            t.outputSliceStride = 0;
            CHK_RET(body());
            done += cur;
        }
        return HCCL_SUCCESS;
    }
};

// ---------------------------------------------------------------------------------------------------
// ReduceScatter (src/ops/reduce_scatter/executor/ins_v2_reduce_scatter_sole_executor.cc:123-170)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate> class InsV2ReduceScatterSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "ReduceScatter sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.DataDes.dataType;
        dataCount_ = param.DataDes.count;  // recvCount
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataSize_ = dataCount_ * dataTypeSize_;
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        return Loops(alg, t, [&]() { return alg.KernelRun(param, t, res); });
    }
    bool ClosedForm(const OpParam &param, u32 rankSize, u64 cclBytes, std::vector<ClosedFold> &out) override
    {
        dataType_ = param.DataDes.dataType;
        dataCount_ = param.DataDes.count;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataSize_ = dataCount_ * dataTypeSize_;
        TemplateDataParams t;
        t.buffInfo.hcclBuff.size = cclBytes;
        t.buffInfo.inBuffType = BufferType::INPUT;
        t.buffInfo.outBuffType = BufferType::OUTPUT;
        t.buffInfo.hcclBuffType = BufferType::HCCL_BUFFER;
        t.repeatNum = 1;
        InsAlgTemplate alg(param, 0, AlgTopoMatch::Match(rankSize));
        bool all = true;
        const HcclResult res = Loops(alg, t, [&]() {
            all = all && alg.ClosedForm(t, dataTypeSize_, out);
            return HCCL_SUCCESS;
        });
        return res == HCCL_SUCCESS && all;
    }

private:
    // The chunk loop (:123-170): `body` runs once per chunk with `t` describing it.
    template <typename F> HcclResult Loops(InsAlgTemplate &alg, TemplateDataParams &t, F &&body)
    {
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size - 1 * 1024 * 1024;  // one MiB is kept back (:126-128)
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, maxTmpMemSize_) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[ReduceScatter executor] maxDataCountPerLoop is 0"), HCCL_E_INTERNAL);
        const u64 loops = dataCount_ / maxCount + (dataCount_ % maxCount != 0);
        u64 done = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            const u64 cur = (loop == loops - 1) ? dataCount_ - done : maxCount;
            t.count = cur;
            t.buffInfo.inBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.sliceSize = cur * dataTypeSize_;
            t.tailSize = t.sliceSize;
            t.inputSliceStride = dataSize_;  // shard k of the input starts k * (recvCount * size) in
            t.outputSliceStride = 0;
            CHK_RET(body());
            done += cur;
        }
        return HCCL_SUCCESS;
    }
};

// ---------------------------------------------------------------------------------------------------
// AllGather (src/ops/all_gather/executor/ins_v2_all_gather_sole_executor.cc:128-176)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate> class InsV2AllGatherSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "AllGather sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.DataDes.dataType;
        dataCount_ = param.DataDes.count;  // sendCount
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataSize_ = dataCount_ * dataTypeSize_;
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, UB_MAX_DATA_SIZE) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[AllGather executor] maxCountPerLoop is 0"), HCCL_E_INTERNAL);
        const u64 loops = dataCount_ / maxCount + (dataCount_ % maxCount != 0);
        u64 done = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            const u64 cur = (loop == loops - 1) ? dataCount_ - done : maxCount;
            t.buffInfo.inBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.count = cur;
            t.sliceSize = cur * dataTypeSize_;
            t.tailSize = t.sliceSize;
            t.inputSliceStride = 0;
            t.outputSliceStride = dataSize_;  // rank k's block starts k * (sendCount * size) into the output
            CHK_RET(alg.KernelRun(param, t, res));
            done += cur;
        }
        return HCCL_SUCCESS;
    }
};

// ---------------------------------------------------------------------------------------------------
// AllGatherV (src/ops/all_gather_v/executor/ins_v2_all_gather_v_sole_executor.cc:105-192)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate> class InsV2AllGatherVSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "AllGatherV sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.vDataDes.dataType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataSize_ = param.DataDes.count * dataTypeSize_;
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        const std::vector<u64> &counts = param.vDataDes.counts;
        t.allRankDispls = param.vDataDes.displs;
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, UB_MAX_DATA_SIZE) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[AllGatherV executor] maxCountPerLoop is 0"), HCCL_E_INTERNAL);
        u64 maxSend = 0;
        for (u32 j = 0; j < rankSize_; ++j) maxSend = std::max(maxSend, counts[j]);
        if (maxSend == 0) return HCCL_SUCCESS;
        const u64 loops = 1 + ((maxSend - 1) / maxCount);
        std::vector<u64> processed(rankSize_, 0);
        t.sliceSize = 0;
        t.tailSize = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            t.allRankSliceSize.clear();
            for (u32 i = 0; i < rankSize_; ++i) {
                const u64 left = processed[i] < counts[i] ? std::min(maxCount, counts[i] - processed[i]) : 0;
                t.allRankSliceSize.push_back(left * dataTypeSize_);
                if (loop == 0) t.sliceSize = std::max(t.sliceSize, t.allRankSliceSize[i]);
            }
            t.buffInfo.inBuffBaseOff = processed[myRank_] * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = processed[myRank_] * dataTypeSize_;
            t.allRankProcessedDataCount = processed;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.inputSliceStride = dataSize_;
            t.outputSliceStride = maxCount * dataTypeSize_;
            CHK_RET(alg.KernelRun(param, t, res));
            for (u32 i = 0; i < rankSize_; ++i) processed[i] += t.allRankSliceSize[i] / dataTypeSize_;
            t.tailSize += maxCount;
        }
        return HCCL_SUCCESS;
    }
};

// ---------------------------------------------------------------------------------------------------
// ReduceScatterV (src/ops/reduce_scatter_v/executor/ins_v2_reduce_scatter_v_sole_executor.cc:75-170)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate>
class InsV2ReduceScatterVSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "ReduceScatterV sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.vDataDes.dataType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        return Loops(param, alg, t, [&]() { return alg.KernelRun(param, t, res); });
    }
    bool ClosedForm(const OpParam &param, u32 rankSize, u64 cclBytes, std::vector<ClosedFold> &out) override
    {
        rankSize_ = rankSize;
        dataType_ = param.vDataDes.dataType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        TemplateDataParams t;
        t.buffInfo.hcclBuff.size = cclBytes;
        t.buffInfo.inBuffType = BufferType::INPUT;
        t.buffInfo.outBuffType = BufferType::OUTPUT;
        t.buffInfo.hcclBuffType = BufferType::HCCL_BUFFER;
        InsAlgTemplate alg(param, 0, AlgTopoMatch::Match(rankSize));
        bool all = true;
        const HcclResult res = Loops(param, alg, t, [&]() {
            all = all && alg.ClosedForm(t, dataTypeSize_, out);
            return HCCL_SUCCESS;
        });
        return res == HCCL_SUCCESS && all;
    }

private:
    // The chunk loop (sole_executor.cc:133-166): `body` runs once per chunk with `t` describing it.
    template <typename F> HcclResult Loops(const OpParam &param, InsAlgTemplate &alg, TemplateDataParams &t, F &&body)
    {
        t.repeatNum = 1;
        t.inputRepeatStride = 0;
        t.outputRepeatStride = 0;
        const std::vector<u64> &counts = param.vDataDes.counts;
        CHK_PRT_RET(counts.size() != rankSize_ || param.vDataDes.displs.size() != rankSize_,
                    HCCL_ERROR("[ReduceScatterV executor] count tables do not match the rank size"), HCCL_E_PARA);
        t.allRankDispls = param.vDataDes.displs;
        for (u64 &d : t.allRankDispls) d *= dataTypeSize_;
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, UB_MAX_DATA_SIZE) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[ReduceScatterV executor] maxDataCountPerLoop is 0"), HCCL_E_INTERNAL);
        u64 maxRecv = 0;
        for (u32 i = 0; i < rankSize_; ++i) maxRecv = std::max(maxRecv, counts[i]);
        if (maxRecv == 0) return HCCL_SUCCESS;   // the op entry returns before it gets here
        const u64 loops = 1 + ((maxRecv - 1) / maxCount);
        u64 processed = 0;
        t.allRankSliceSize.assign(rankSize_, 0);
        for (u64 loop = 0; loop < loops; ++loop) {
            u64 largest = 0;
            for (u32 i = 0; i < rankSize_; ++i) {
                const u64 left = processed < counts[i] ? std::min(maxCount, counts[i] - processed) : 0;
                t.allRankSliceSize[i] = left * dataTypeSize_;
                largest = std::max(largest, left);
            }
            // every rank's part advances by the same element offset
            t.buffInfo.inBuffBaseOff = processed * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = processed * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.outputSliceStride = maxCount * dataTypeSize_;
            CHK_RET(body());
            processed += largest;
        }
        return HCCL_SUCCESS;
    }
};

// ---------------------------------------------------------------------------------------------------
// AlltoAll / AlltoAllV / AlltoAllVC (src/ops/all_to_all_v/executor/ins_v2_all_to_all_v_sole_executor.cc:183-368)
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate> class InsV2AlltoAllVSoleExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "AlltoAllV sole executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.all2AllVDataDes.sendType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        const std::vector<u64> &sendCounts = param.all2AllVDataDes.sendCounts;
        const std::vector<u64> &recvCounts = param.all2AllVDataDes.recvCounts;
        const std::vector<u64> &sdispls = param.all2AllVDataDes.sdispls;
        const std::vector<u64> &rdispls = param.all2AllVDataDes.rdispls;
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, UB_MAX_DATA_SIZE) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[AlltoAllV executor] maxDataCountPerLoop is 0"), HCCL_E_INTERNAL);
        u64 maxBlock = 0;
        for (u32 i = 0; i < rankSize_; ++i) maxBlock = std::max(maxBlock, std::max(sendCounts[i], recvCounts[i]));
        const u64 loops = maxBlock / maxCount + (maxBlock % maxCount != 0);
        t.inputSliceStride = maxCount * dataTypeSize_;   // size of one scratch slot
        t.outputSliceStride = maxBlock * dataTypeSize_;
        u64 done = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            const u64 cur = (loop == loops - 1) ? maxBlock - done : maxCount;
            t.count = cur;
            t.dataType = dataType_;
            t.buffInfo.inBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            t.processedDataCount = done;
            t.sliceSize = cur * dataTypeSize_;
            t.tailSize = t.sliceSize;
            t.sendCounts.assign(rankSize_, 0);
            t.recvCounts.assign(rankSize_, 0);
            t.sdispls.assign(rankSize_, 0);
            t.rdispls.assign(rankSize_, 0);
            for (u32 i = 0; i < rankSize_; ++i) {  // every block contributes its sub-range of this loop
                if (sendCounts[i] > done) {
                    t.sendCounts[i] = std::min(cur, sendCounts[i] - done);
                    t.sdispls[i] = sdispls[i] + done;
                } else {
                    t.sdispls[i] = sdispls[i] + sendCounts[i];
                }
                if (recvCounts[i] > done) {
                    t.recvCounts[i] = std::min(cur, recvCounts[i] - done);
                    t.rdispls[i] = rdispls[i] + done;
                } else {
                    t.rdispls[i] = rdispls[i] + recvCounts[i];
                }
            }
            CHK_RET(alg.KernelRun(param, t, res));
            done += cur;
        }
        return HCCL_SUCCESS;
    }
};

// Names as the reference registers them (e.g. ins_v2_reduce_scatter_sole_executor.cc:256-265); the two
// documentation-derived AllReduce templates are added under their own names.

// ---------------------------------------------------------------------------------------------------
// Order-preserved ReduceScatter
// (src/ops/reduce_scatter/executor/ins_v2_reduce_scatter_order_preserved_executor.cc:77-186): the chunk loop of
// the sole executor with the whole scratch buffer, the 256 MiB transport bound and a table of where each
// rank's block sits in this loop.
// ---------------------------------------------------------------------------------------------------
template <typename AlgTopoMatch, typename InsAlgTemplate>
class InsV2ReduceScatterOrderPreservedExecutor : public InsCollAlgBase {
public:
    std::string Describe() const override { return "ReduceScatter order-preserved executor"; }
    u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) override
    {
        InsAlgTemplate t(param, rank, AlgTopoMatch::Match(rankSize));
        return t.GetThreadNum();
    }
    HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) override
    {
        myRank_ = resCtx.topoInfo.userRank;
        rankSize_ = resCtx.topoInfo.userRankSize;
        dataType_ = param.DataDes.dataType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataCount_ = param.DataDes.count;
        dataSize_ = dataCount_ * dataTypeSize_;
        TemplateResource res;
        TemplateDataParams t;
        detail::FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
        return Loops(alg, t, [&]() { return alg.KernelRun(param, t, res); });
    }
    bool ClosedForm(const OpParam &param, u32 rankSize, u64 cclBytes, std::vector<ClosedFold> &out) override
    {
        rankSize_ = rankSize;
        dataType_ = param.DataDes.dataType;
        dataTypeSize_ = DATATYPE_SIZE_TABLE[dataType_];
        dataCount_ = param.DataDes.count;
        dataSize_ = dataCount_ * dataTypeSize_;
        TemplateDataParams t;
        t.buffInfo.hcclBuff.size = cclBytes;
        t.buffInfo.inBuffType = BufferType::INPUT;
        t.buffInfo.outBuffType = BufferType::OUTPUT;
        t.buffInfo.hcclBuffType = BufferType::HCCL_BUFFER;
        t.repeatNum = 1;
        InsAlgTemplate alg(param, 0, AlgTopoMatch::Match(rankSize));
        bool all = true;
        const HcclResult res = Loops(alg, t, [&]() {
            all = all && alg.ClosedForm(t, dataTypeSize_, out);
            return HCCL_SUCCESS;
        });
        return res == HCCL_SUCCESS && all;
    }

private:
    // The chunk loop: `body` runs once per chunk with `t` and the template's block table describing it.
    template <typename F> HcclResult Loops(InsAlgTemplate &alg, TemplateDataParams &t, F &&body)
    {
        const u64 mult = alg.CalcScratchMultiple(t.buffInfo.inBuffType, t.buffInfo.outBuffType);
        maxTmpMemSize_ = t.buffInfo.hcclBuff.size;
        const u64 maxCount = MaxDataSizePerLoop(maxTmpMemSize_, mult, UB_MAX_DATA_SIZE) / dataTypeSize_;
        CHK_PRT_RET(maxCount == 0, HCCL_ERROR("[ReduceScatter order-preserved executor] maxDataCountPerLoop is 0"),
                    HCCL_E_INTERNAL);
        const u64 loops = dataCount_ / maxCount + (dataCount_ % maxCount != 0);
        u64 done = 0;
        for (u64 loop = 0; loop < loops; ++loop) {
            const u64 cur = (loop == loops - 1) ? dataCount_ - done : maxCount;
            const u64 blockSize = cur * dataTypeSize_;
            t.count = cur;
            t.buffInfo.inBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.outBuffBaseOff = done * dataTypeSize_;
            t.buffInfo.hcclBuffBaseOff = 0;
            MemBlockInfo blocks;
            for (u32 k = 0; k < rankSize_; ++k) {
                blocks.size.push_back(blockSize);
                blocks.userInputOffsets.push_back(done * dataTypeSize_ + k * dataSize_);
                blocks.inputOffsets.push_back(k * blockSize);
                blocks.outputOffsets.push_back(k * blockSize);
            }
            t.sliceSize = blockSize;
            t.tailSize = blockSize;
            t.inputSliceStride = dataSize_;
            t.outputSliceStride = 0;
            alg.SetMemBlockInfo(blocks);
            CHK_RET(body());
            done += cur;
        }
        return HCCL_SUCCESS;
    }
};

}  // namespace ops_hccl
