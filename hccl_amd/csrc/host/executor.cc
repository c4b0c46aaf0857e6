#include "executor.h"

#include <algorithm>

#include "all_reduce_templates.h"
#include "data_move_templates.h"

namespace ops_hccl {

CollAlgExecRegistryV2 &CollAlgExecRegistryV2::Instance()
{
    static CollAlgExecRegistryV2 inst;
    return inst;
}

HcclResult CollAlgExecRegistryV2::Register(HcclCMDType type, const std::string &tag, const CollExecCreatorV2 &creator)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (execCreators_[type].count(tag)) return HCCL_E_INTERNAL;
    execCreators_[type].emplace(tag, creator);
    return HCCL_SUCCESS;
}

std::unique_ptr<InsCollAlgBase> CollAlgExecRegistryV2::GetAlgExec(HcclCMDType type, const std::string &tag)
{
    std::lock_guard<std::mutex> lock(mu_);
    auto t = execCreators_.find(type);
    if (t == execCreators_.end()) return nullptr;
    auto e = t->second.find(tag);
    if (e == t->second.end()) return nullptr;
    return std::unique_ptr<InsCollAlgBase>(e->second());
}

std::vector<std::string> CollAlgExecRegistryV2::Names(HcclCMDType type)
{
    std::lock_guard<std::mutex> lock(mu_);
    std::vector<std::string> out;
    for (auto &kv : execCreators_[type]) out.push_back(kv.first);
    return out;
}

u64 MaxDataSizePerLoop(u64 scratchSize, u64 scratchMultiple, u64 transportBound)
{
    if (scratchMultiple == 0) return transportBound;
    const u64 scratchBound = scratchSize / scratchMultiple / HCCL_MIN_SLICE_ALIGN * HCCL_MIN_SLICE_ALIGN;
    return std::min(transportBound, scratchBound);
}

namespace {

void FillBuffInfo(const OpParam &param, const AlgResourceCtxSerializable &resCtx, TemplateDataParams &t,
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

}  // namespace

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
        FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
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
            CHK_RET(alg.KernelRun(param, t, res));
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
        FillBuffInfo(param, resCtx, t, res);
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
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
            CHK_RET(alg.KernelRun(param, t, res));
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
        FillBuffInfo(param, resCtx, t, res);
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
        FillBuffInfo(param, resCtx, t, res);
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
        FillBuffInfo(param, resCtx, t, res);
        t.repeatNum = 1;
        t.inputRepeatStride = 0;
        t.outputRepeatStride = 0;
        const std::vector<u64> &counts = param.vDataDes.counts;
        t.allRankDispls = param.vDataDes.displs;
        for (u64 &d : t.allRankDispls) d *= dataTypeSize_;
        InsAlgTemplate alg(param, myRank_, resCtx.subCommRanks);
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
            CHK_RET(alg.KernelRun(param, t, res));
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
        FillBuffInfo(param, resCtx, t, res);
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
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceMesh1DOneShot, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceMesh1DOneShot);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceMesh1DTwoShot, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceMesh1DTwoShot);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceNHR, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceNHR);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceAicpuReduceNHR, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceAicpuReduceNHR);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceRing, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceRing);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceRHD, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 InsTempAllReduceRHD);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, InsReduceScatterMesh1D, InsV2ReduceScatterSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, InsReduceScatterNHR, InsV2ReduceScatterSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterNHR);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLGATHER, InsAllGatherMesh1D, InsV2AllGatherSoleExecutor, TopoMatch1D,
                 InsTempAllGatherMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLGATHER, InsAllGatherNHR, InsV2AllGatherSoleExecutor, TopoMatch1D,
                 InsTempAllGatherNHR);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, InsAllReduceMesh1DTwoShotMeshChunk, InsV2AllReduceSoleExecutor,
                 TopoMatch1D, InsTempAllReduceMesh1DTwoShotMeshChunk);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, InsReduceScatterMesh1DMeshChunk, InsV2ReduceScatterSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterMesh1DMeshChunk);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V, InsReduceScatterVMesh1D, InsV2ReduceScatterVSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLGATHER_V, InsAllGatherVMesh1D, InsV2AllGatherVSoleExecutor, TopoMatch1D,
                 InsTempAllGatherVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALLV, InsAlltoAllVMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALL, InsAlltoAllMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALLVC, InsAlltoAllVCMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);

}  // namespace ops_hccl
