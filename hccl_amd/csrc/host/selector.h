// Algorithm selection: registry, priority walk and the AICPU branch of the built-in selectors.
//
// Reference: SelectorRegistry / REGISTER_SELECTOR_BY_OPTYPE (src/ops/op_common/selector/selector_registry.h:21-54),
// ExecuteSelector::Run (src/ops/op_common/selector/execute_selector.cc:21-55), AutoSelectorBase::Select
// (src/ops/op_common/selector/auto_selector_base.cc:17-68).  The reference tries engines in the order
// host DPU -> CCU -> AIV -> AICPU; only the AICPU branch has a counterpart here, so Select goes there.
#pragma once
#include <map>
#include <mutex>
#include <string>

#include "alg_param.h"

namespace ops_hccl {

enum class SelectorStatus { MATCH, NOT_MATCH };

constexpr double DEFAULT_RANK_SIZE = 8.0;  // auto_selector_base.h:27

// What the selectors read of the topology (TopoInfoWithNetLayerDetails in the reference).
struct TopoInfoWithNetLayerDetails {
    u32 userRank = 0;
    u32 userRankSize = 0;
    u32 topoLevelNums = 1;
    Level0Shape level0Topo = Level0Shape::MESH_1D;
    u32 localNetInsSizeOfLayer0 = 0;  // devices per server; 1 = a topology of single-device servers
    bool Level1Nhr = false;
};

class AutoSelectorBase {
public:
    virtual ~AutoSelectorBase() = default;
    SelectorStatus Select(OpParam &opParam, TopoInfoWithNetLayerDetails *topoInfo, std::string &selectAlgName) const
    {
        const SelectorStatus ret = SelectAicpuAlgo(topoInfo, opParam, selectAlgName);
        if (ret == SelectorStatus::MATCH) opParam.engine = CommEngine::COMM_ENGINE_AICPU_TS;
        return ret;
    }

protected:
    virtual SelectorStatus SelectAicpuAlgo(const TopoInfoWithNetLayerDetails *topoInfo, const OpParam &opParam,
                                           std::string &selectAlgName) const = 0;
};

class SelectorRegistry {
public:
    static SelectorRegistry *Global();
    HcclResult RegisterByOpType(HcclCMDType opType, u32 priority, AutoSelectorBase *selector);
    std::map<u32, AutoSelectorBase *> GetSelectorsByOpType(HcclCMDType opType);

private:
    std::map<HcclCMDType, std::map<u32, AutoSelectorBase *>> opTypeImpls_;
    std::mutex mu_;
};

#define REGISTER_SELECTOR_BY_OPTYPE_HELPER(ctr, optype, priority, selector) \
    static HcclResult g_selector_##selector##_##ctr =                       \
        SelectorRegistry::Global()->RegisterByOpType(optype, priority, new selector())
#define REGISTER_SELECTOR_BY_OPTYPE_HELPER_1(ctr, optype, priority, selector) \
    REGISTER_SELECTOR_BY_OPTYPE_HELPER(ctr, optype, priority, selector)
#define REGISTER_SELECTOR_BY_OPTYPE(optype, priority, selector) \
    REGISTER_SELECTOR_BY_OPTYPE_HELPER_1(__COUNTER__, optype, priority, selector)

class ExecuteSelector {
public:
    // Walks the selectors of the op type in priority order; the first MATCH wins, none -> HCCL_E_NOT_SUPPORT.
    HcclResult Run(OpParam &opParam, TopoInfoWithNetLayerDetails *topoInfo, std::string &selectAlgName) const;
};

}  // namespace ops_hccl
