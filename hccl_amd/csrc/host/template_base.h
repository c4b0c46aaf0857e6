// Base class of the algorithm templates (reference: src/ops/op_common/template/common_alg_template_base.h:19-56,
// alg_v2_template_base.h:18-76, alg_v2_template_base.cc:15-26).  A template turns one executor chunk into
// copy / reduce / send / receive steps by calling the verbs of alg_data_trans_wrapper.h.
//
// Left out on purpose: CalcRes / GetRes / FastLaunch / DPUKernelRun -- resource plumbing for real links,
// CCU fast launch and DPU offload, none of which exists for virtual ranks in one GPU.
#pragma once
#include <string>
#include <vector>

#include "alg_data_trans_wrapper.h"
#include "alg_param.h"

namespace ops_hccl {

class InsAlgTemplateBase {
public:
    InsAlgTemplateBase(const OpParam &param, u32 rankId, const std::vector<std::vector<u32>> &subCommRanks)
        : opMode_(param.opMode), myRank_(rankId), subCommRanks_(subCommRanks), reduceOp_(param.reduceType)
    {
        templateRankSize_ = subCommRanks.empty() ? 0 : static_cast<u32>(subCommRanks[0].size());
    }
    virtual ~InsAlgTemplateBase() = default;

    virtual std::string Describe() const = 0;
    // Threads (task queues) of this rank the template spreads its steps over.
    virtual u64 GetThreadNum() const = 0;
    // How many chunk-sized slots of the scratch buffer one KernelRun needs.
    virtual u64 CalcScratchMultiple(BufferType inBuffType, BufferType outBuffType) = 0;
    virtual HcclResult KernelRun(const OpParam &param, const TemplateDataParams &tempAlgParams,
                                 TemplateResource &templateResource) = 0;

    // The net effect of one KernelRun among all ranks, appended to `out`, for templates whose recorded steps grow
    // with the cube of the rank count: the world then plans from this instead of recording and tracing them.  Only
    // the offsets, strides and counts of `tempAlgParams` are used.  The default: no closed form (record the steps).
    virtual bool ClosedForm(const TemplateDataParams &tempAlgParams, u64 dataTypeSize, std::vector<ClosedFold> &out) const
    {
        (void)tempAlgParams;
        (void)dataTypeSize;
        (void)out;
        return false;
    }

    virtual void GetNotifyIdxMainToSub(std::vector<u32> &notifyIdxMainToSub)
    {
        // every sub thread is woken on its own notify 0
        notifyIdxMainToSub.assign(GetThreadNum() > 0 ? GetThreadNum() - 1 : 0, 0);
    }
    virtual void GetNotifyIdxSubToMain(std::vector<u32> &notifyIdxSubToMain)
    {
        // the main thread has one notify per sub thread
        notifyIdxSubToMain.clear();
        for (u32 i = 0; i + 1 < GetThreadNum(); ++i) notifyIdxSubToMain.push_back(i);
    }

protected:
    // True when a link of this rank is PCIe: the templates that have a read mode then let the receiver fetch
    // (alg_v2_template_base.cc:91-101).
    static bool IsPcieProtocol(const std::map<u32, std::vector<ChannelInfo>> &channels)
    {
        for (const auto &kv : channels) {
            if (!kv.second.empty() && kv.second[0].protocol == CommProtocol::COMM_PROTOCOL_PCIE) return true;
        }
        return false;
    }

    HcclResult PreSync(const std::vector<ThreadHandle> &threads)
    {
        if (threads.size() <= 1) return HCCL_SUCCESS;
        std::vector<ThreadHandle> subs(threads.begin() + 1, threads.end());
        std::vector<u32> idx(subs.size(), 0);
        return PreSyncInterThreads(threads[0], subs, idx);
    }
    HcclResult PostSync(const std::vector<ThreadHandle> &threads)
    {
        if (threads.size() <= 1) return HCCL_SUCCESS;
        std::vector<ThreadHandle> subs(threads.begin() + 1, threads.end());
        std::vector<u32> idx;
        for (u32 i = 0; i < subs.size(); ++i) idx.push_back(i);
        return PostSyncInterThreads(threads[0], subs, idx);
    }

    OpMode opMode_;
    u32 myRank_ = INVALID_VALUE_RANKID;
    u32 templateRankSize_ = 0;
    std::vector<std::vector<u32>> subCommRanks_;
    u32 threadNum_ = 0;
    HcclReduceOp reduceOp_;
    HcclDataType dataType_ = HCCL_DATA_TYPE_RESERVED;
};

// ceil(count / n) elements per slice, the remainder short or empty
// (SplitData, src/ops/all_reduce/template/aicpu/ins_temp_all_reduce_nhr.cc:137-163).
std::vector<SliceInfo> SplitDataByRank(u64 count, u32 sliceNum, u64 dataTypeSize);

// Step tables of the NHR (nonuniform hierarchical ring) algorithm
// (ins_temp_all_reduce_nhr.cc:325-404).
void GetNHRReduceScatterSteps(u32 rankSize, u32 myRankIdx, std::vector<NHRStepInfo> &steps);
void GetNHRAllGatherSteps(u32 rankSize, u32 myRankIdx, std::vector<NHRStepInfo> &steps);

// What every rank holds of ONE slice while a schedule reduces and copies whole slices from rank to rank: which ranks'
// data went into it, and in which tree.  For the templates whose result is a tree (log-step schedules) and that
// state it in closed form: they replay their step tables on these values, N^2 small steps instead of N^2 log N
// recorded, ordered and traced ones.  The steps of one round read the values from before the round.
class SliceValues {
public:
    explicit SliceValues(u32 ranks);            // every rank holds its own data
    void Reduce(u32 dstRank, u32 srcRank);      // dst = src (+) dst, when the round ends
    void Copy(u32 dstRank, u32 srcRank);        // dst = src, when the round ends
    void EndRound();
    bool Same(u32 a, u32 b) const { return held_[a] == held_[b]; }
    // What rank `r` holds, as the sources (every rank's piece at `inOffset`) and the tree of a closed fold.
    void Emit(u32 r, u64 inOffset, ClosedFold &f) const;

private:
    struct Node {
        int src = -1;   // inner node: the two operands of its step
        int dst = -1;
        u32 rank = 0;   // leaf: whose data
    };
    u32 EmitNode(int node, u64 inOffset, ClosedFold &f) const;
    std::vector<Node> nodes_;
    std::vector<int> held_;
    std::vector<std::pair<u32, int>> staged_;
};

}  // namespace ops_hccl
