// Executors: the chunk loops between an op entry and its template, and their registry.
//
// Reference: InsCollAlgBase (src/ops/op_common/executor/executor_v2_base.h:29-92), CollAlgExecRegistryV2 and
// REGISTER_EXEC_V2 (src/ops/op_common/executor/registry/coll_alg_v2_exec_registry.h:33-72), and the five
// "sole" executors (src/ops/<op>/executor/ins_v2_<op>_sole_executor.cc).  An executor cuts the operand into
// pieces that fit the scratch buffer -- maxDataSizePerLoop = min(transport bound, floor(scratch / scratch
// multiple / 128) * 128) -- and runs the template once per piece.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>

#include "alg_param.h"
#include "template_base.h"

namespace ops_hccl {

// One flat level holding ranks 0..N-1 (src/ops/op_common/topo/topo_match_1d.cc:23-63).
class TopoMatch1D {
public:
    static std::vector<std::vector<u32>> Match(u32 rankSize)
    {
        std::vector<std::vector<u32>> out(1);
        for (u32 r = 0; r < rankSize; ++r) out[0].push_back(r);
        return out;
    }
};

class InsCollAlgBase {
public:
    virtual ~InsCollAlgBase() = default;
    virtual std::string Describe() const = 0;
    // Threads the template of this executor needs on one rank.
    virtual u64 CalcThreadNum(const OpParam &param, u32 rank, u32 rankSize) = 0;
    virtual HcclResult Orchestrate(const OpParam &param, const AlgResourceCtxSerializable &resCtx) = 0;
    // The whole collective among `rankSize` ranks in closed form (see ClosedFold), when the template has one: the
    // same chunk loop as Orchestrate, asking the template for the net effect of each chunk instead of its steps.
    virtual bool ClosedForm(const OpParam &param, u32 rankSize, u64 cclBytes, std::vector<ClosedFold> &out)
    {
        (void)param;
        (void)rankSize;
        (void)cclBytes;
        (void)out;
        return false;
    }

protected:
    u32 myRank_ = INVALID_VALUE_RANKID;
    u32 rankSize_ = 0;
    HcclReduceOp reduceOp_ = HCCL_REDUCE_RESERVED;
    HcclDataType dataType_ = HCCL_DATA_TYPE_RESERVED;
    u64 dataCount_ = 0;
    u64 maxTmpMemSize_ = 0;
    u64 dataSize_ = 0;
    u64 dataTypeSize_ = 0;
};

using CollExecCreatorV2 = std::function<InsCollAlgBase *()>;

class CollAlgExecRegistryV2 {
public:
    static CollAlgExecRegistryV2 &Instance();
    HcclResult Register(HcclCMDType type, const std::string &tag, const CollExecCreatorV2 &creator);
    std::unique_ptr<InsCollAlgBase> GetAlgExec(HcclCMDType type, const std::string &tag);
    std::vector<std::string> Names(HcclCMDType type);

private:
    std::map<HcclCMDType, std::map<std::string, CollExecCreatorV2>> execCreators_;
    std::mutex mu_;
};

#define REGISTER_EXEC_V2_HELPER(ctr, type, name, Executor, AlgTopoMatch, InsAlgTemplate)       \
    static HcclResult g_exec_##name##_##ctr = CollAlgExecRegistryV2::Instance().Register(       \
        type, std::string(#name), []() -> InsCollAlgBase * { return new Executor<AlgTopoMatch, InsAlgTemplate>(); })
#define REGISTER_EXEC_V2_HELPER_1(ctr, type, name, Executor, AlgTopoMatch, InsAlgTemplate) \
    REGISTER_EXEC_V2_HELPER(ctr, type, name, Executor, AlgTopoMatch, InsAlgTemplate)
#define REGISTER_EXEC_V2(type, name, Executor, AlgTopoMatch, InsAlgTemplate) \
    REGISTER_EXEC_V2_HELPER_1(__COUNTER__, type, name, Executor, AlgTopoMatch, InsAlgTemplate)

// floor(scratch / multiple / 128) * 128, capped by the transport bound; 0 multiple = transport bound.
u64 MaxDataSizePerLoop(u64 scratchSize, u64 scratchMultiple, u64 transportBound);

}  // namespace ops_hccl
