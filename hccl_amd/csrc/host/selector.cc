#include "selector.h"

#include "alg_env_config.h"

namespace ops_hccl {

SelectorRegistry *SelectorRegistry::Global()
{
    static SelectorRegistry *inst = new SelectorRegistry;
    return inst;
}

HcclResult SelectorRegistry::RegisterByOpType(HcclCMDType opType, u32 priority, AutoSelectorBase *selector)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (opTypeImpls_[opType].count(priority)) return HCCL_E_INTERNAL;
    opTypeImpls_[opType][priority] = selector;
    return HCCL_SUCCESS;
}

std::map<u32, AutoSelectorBase *> SelectorRegistry::GetSelectorsByOpType(HcclCMDType opType)
{
    std::lock_guard<std::mutex> lock(mu_);
    return opTypeImpls_[opType];
}

HcclResult ExecuteSelector::Run(OpParam &opParam, TopoInfoWithNetLayerDetails *topoInfo,
                                std::string &selectAlgName) const
{
    for (auto &kv : SelectorRegistry::Global()->GetSelectorsByOpType(opParam.opType)) {
        if (kv.second->Select(opParam, topoInfo, selectAlgName) == SelectorStatus::MATCH) return HCCL_SUCCESS;
    }
    HCCL_ERROR("[Algo][Selector] No selector is matched.");
    return HCCL_E_NOT_SUPPORT;
}

namespace {

bool IsSpecial(HcclDataType dt, HcclReduceOp op)
{
    return dt == HCCL_DATA_TYPE_INT64 || dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64 ||
           op == HCCL_REDUCE_PROD;
}

// ---- AllReduce (src/ops/all_reduce/selector/all_reduce_auto_selector.cc:351-529) -----------------------
constexpr u64 AR_AICPU_1D_SMALL_DATA_SIZE = 8ull * 1024 * 1024;
constexpr u64 AR_AICPU_1D_MAX_DATA_SIZE = 32ull * 1024 * 1024;
constexpr u64 AR_AICPU_1D_64DATATYPE_DATA_SIZE = 8ull * 1024 * 1024;
constexpr u64 RS_AICPU_1D_MAX_DATA_SIZE = 16ull * 1024 * 1024;   // reduce_scatter_auto_selector.cc:20
constexpr double DEFAULT_RANK_SIZE = 8.0;                        // op_common/selector/auto_selector_base.h:27

class AllReduceAutoSelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topo, const OpParam &p,
                                   std::string &name) const override
    {
        const u64 dataSize = p.DataDes.count * DATATYPE_SIZE_TABLE[p.DataDes.dataType];
        const bool special = IsSpecial(p.DataDes.dataType, p.reduceType);
        const double n = topo->userRankSize ? static_cast<double>(topo->userRankSize) : 1.0;
        if (topo->topoLevelNums > 1) {
            // several levels: the flat log-step algorithm; the reference's hierarchical mesh+NHR
            // combinations (:396-409) need real link tiers and are not built
            name = special ? "InsAllReduceAicpuReduceNHR" : "InsAllReduceNHR";
            return SelectorStatus::MATCH;
        }
        if (topo->level0Topo == Level0Shape::MESH_1D) {
            if (special) {
                name = dataSize <= AR_AICPU_1D_64DATATYPE_DATA_SIZE ? "InsAllReduceMesh1DOneShot"
                                                                    : "InsAllReduceMesh1DTwoShot";
            } else if (dataSize <= AR_AICPU_1D_SMALL_DATA_SIZE) {
                name = "InsAllReduceMesh1DOneShot";
            } else if (static_cast<double>(dataSize) * (DEFAULT_RANK_SIZE / n / n) > AR_AICPU_1D_MAX_DATA_SIZE) {
                // large messages reduce in place, chunk by chunk (:485-487; the Z-axis detour variant of
                // two-level machines is not modelled)
                name = "InsAllReduceMesh1DTwoShotMeshChunk";
            } else {
                name = "InsAllReduceMesh1DTwoShot";
            }
            return SelectorStatus::MATCH;
        }
        if (topo->level0Topo == Level0Shape::CLOS) {
            name = special ? "InsAllReduceAicpuReduceNHR" : "InsAllReduceNHR";
            return SelectorStatus::MATCH;
        }
        return SelectorStatus::NOT_MATCH;  // MESH_1D_CLOS machines: not modelled
    }
};

// ---- ReduceScatter (src/ops/reduce_scatter/selector/reduce_scatter_auto_selector.cc:328-446) ---------------
class ReduceScatterAutoSelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topo, const OpParam &p,
                                   std::string &name) const override
    {
        if (IsNeedStrictModeForOrderPreserved(p.DataDes.dataType, p.reduceType, topo->userRankSize)) {
            // strict determinism (:337-347): an all-to-all of the shards, then a fixed tree over the ranks;
            // above 32 ranks the all-to-all runs on a capped number of threads
            name = topo->userRankSize > MAX_RANK_NUM_FOR_ORDER_PRESERVED ? "ReduceScatterOrderPreservedGroup"
                                                                         : "ReduceScatterOrderPreserved";
            return SelectorStatus::MATCH;
        }
        if (topo->topoLevelNums > 1 || topo->level0Topo == Level0Shape::CLOS) {
            // PROD and 64-bit types gather and fold locally (:350, :430)
            name = IsSpecial(p.DataDes.dataType, p.reduceType) ? "InsReduceScatterAicpuReduceNHR" : "InsReduceScatterNHR";
            return SelectorStatus::MATCH;
        }
        if (topo->level0Topo == Level0Shape::MESH_1D) {
            // 64-bit types and PROD stay with the slot-per-rank template; otherwise a shard of more than
            // 16 MiB * (N/8)^2 is reduced in place, chunk by chunk (:383-408)
            const u64 dataSize = p.DataDes.count * DATATYPE_SIZE_TABLE[p.DataDes.dataType];
            const double n = topo->userRankSize ? static_cast<double>(topo->userRankSize) : 1.0;
            const double ratio = topo->userRankSize ? (DEFAULT_RANK_SIZE / n) * (DEFAULT_RANK_SIZE / n) : 1.0;
            if (!IsSpecial(p.DataDes.dataType, p.reduceType) && static_cast<double>(dataSize) * ratio > RS_AICPU_1D_MAX_DATA_SIZE) {
                name = "InsReduceScatterMesh1DMeshChunk";
            } else {
                name = "InsReduceScatterMesh1D";
            }
            return SelectorStatus::MATCH;
        }
        return SelectorStatus::NOT_MATCH;
    }
};

// ---- AllGather (src/ops/all_gather/selector/all_gather_auto_selector.cc:258-340) ---------------------------
class AllGatherAutoSelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topo, const OpParam &p,
                                   std::string &name) const override
    {
        (void)p;
        if (topo->topoLevelNums > 1 || topo->level0Topo == Level0Shape::CLOS) {
            name = "InsAllGatherNHR";
            return SelectorStatus::MATCH;
        }
        if (topo->level0Topo == Level0Shape::MESH_1D) {
            name = "InsAllGatherMesh1D";
            return SelectorStatus::MATCH;
        }
        return SelectorStatus::NOT_MATCH;
    }
};

// ---- AllGatherV: always the mesh template (src/ops/all_gather_v/selector/all_gather_v_auto_selector.cc:63-77)
class AllGatherVAutoSelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *, const OpParam &, std::string &name) const override
    {
        name = "InsAllGatherVMesh1D";
        return SelectorStatus::MATCH;
    }
};

// ---- ReduceScatterV (src/ops/reduce_scatter_v/selector/reduce_scatter_v_auto_selector.cc:204-220): the mesh
//      template for one to three topology levels; uint64 and fp64 have no AICPU algorithm
class ReduceScatterVAutoSelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topo, const OpParam &p,
                                   std::string &name) const override
    {
        const HcclDataType dt = p.vDataDes.dataType;
        if (dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64) return SelectorStatus::NOT_MATCH;
        if (topo->topoLevelNums < 1 || topo->topoLevelNums > 3) return SelectorStatus::NOT_MATCH;
        name = "InsReduceScatterVMesh1D";
        return SelectorStatus::MATCH;
    }
};

// ---- AlltoAll family (src/ops/all_to_all_v/selector/alltoallv_auto_selector.cc:94-128,
//      alltoall_auto_selector.cc:111-154, alltoallvc_auto_selector.cc:53-62) -------------------------------
constexpr u64 ALLTOALL_ENABLE_MULTI_CHANNEL_DATA_SIZE_LIMIT = 150ull * 1024 * 1024;
template <int KIND> class AlltoAllFamilySelector : public AutoSelectorBase {
protected:
    SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topo, const OpParam &p, std::string &name) const override
    {
        if (topo->level0Topo != Level0Shape::MESH_1D && topo->level0Topo != Level0Shape::CLOS) {
            return SelectorStatus::NOT_MATCH;
        }
        name = KIND == 0 ? "InsAlltoAllMesh1D" : KIND == 1 ? "InsAlltoAllVMesh1D" : "InsAlltoAllVCMesh1D";
        if (KIND == 0 && !p.all2AllVDataDes.sendCounts.empty()) {
            // up to 150 MiB per rank one link per pair is used (alltoall_auto_selector.cc:127-135); the
            // steps the template records are the same, only the number of links it would spread them over differs
            const u64 bytes = p.all2AllVDataDes.sendCounts[0] * DATATYPE_SIZE_TABLE[p.all2AllVDataDes.sendType];
            if (bytes * topo->userRankSize <= ALLTOALL_ENABLE_MULTI_CHANNEL_DATA_SIZE_LIMIT) {
                name = "InsAlltoAllMesh1DSingleChannel";
            }
        }
        return SelectorStatus::MATCH;
    }
};
using AlltoAllAutoSelector = AlltoAllFamilySelector<0>;
using AlltoAllVAutoSelector = AlltoAllFamilySelector<1>;
using AlltoAllVCAutoSelector = AlltoAllFamilySelector<2>;

}  // namespace

REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLREDUCE, SELECTOR_PRIORITY_BUILTIN, AllReduceAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_REDUCE_SCATTER, SELECTOR_PRIORITY_BUILTIN, ReduceScatterAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V, SELECTOR_PRIORITY_BUILTIN, ReduceScatterVAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLGATHER, SELECTOR_PRIORITY_BUILTIN, AllGatherAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLGATHER_V, SELECTOR_PRIORITY_BUILTIN, AllGatherVAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLTOALL, SELECTOR_PRIORITY_BUILTIN, AlltoAllAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLTOALLV, SELECTOR_PRIORITY_BUILTIN, AlltoAllVAutoSelector);
REGISTER_SELECTOR_BY_OPTYPE(HcclCMDType::HCCL_CMD_ALLTOALLVC, SELECTOR_PRIORITY_BUILTIN, AlltoAllVCAutoSelector);

}  // namespace ops_hccl
