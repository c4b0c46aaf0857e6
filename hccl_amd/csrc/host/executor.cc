#include "executor.h"

#include <algorithm>

#include "all_reduce_templates.h"
#include "data_move_templates.h"
#include "sole_executors.h"

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
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, InsReduceScatterAicpuReduceNHR, InsV2ReduceScatterSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterAicpuReduceNHR);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, InsReduceScatterMesh1DMeshChunk, InsV2ReduceScatterSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterMesh1DMeshChunk);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, ReduceScatterOrderPreserved, InsV2ReduceScatterOrderPreservedExecutor,
                 TopoMatch1D, InsTempReduceScatterOrderPreservedLevel1);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, ReduceScatterOrderPreservedGroup, InsV2ReduceScatterOrderPreservedExecutor,
                 TopoMatch1D, InsTempReduceScatterOrderPreservedGroup);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V, InsReduceScatterVMesh1D, InsV2ReduceScatterVSoleExecutor,
                 TopoMatch1D, InsTempReduceScatterVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLGATHER_V, InsAllGatherVMesh1D, InsV2AllGatherVSoleExecutor, TopoMatch1D,
                 InsTempAllGatherVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALLV, InsAlltoAllVMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALL, InsAlltoAllMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALL, InsAlltoAllMesh1DSingleChannel, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLTOALLVC, InsAlltoAllVCMesh1D, InsV2AlltoAllVSoleExecutor, TopoMatch1D,
                 InsTempAlltoAllVMesh1D);

}  // namespace ops_hccl
