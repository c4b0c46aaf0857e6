// ReduceScatter, ReduceScatterV, AllGather, AllGatherV and AlltoAllV templates: see the .cc files for what each restates.
#pragma once
#include "all_reduce_templates.h"

namespace ops_hccl {

// scratch multiples: reduce_scatter mesh_1D.cc:59-63 (N), nhr.cc:369-377 (N); all_gather mesh/NHR (N);
// all_gather_v mesh_1D.cc:48-57 (N in single-op mode); all_to_all_v mesh_1D.cc:66-73 (min(16, N-1)).
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempReduceScatterMesh1D, "ReduceScatter mesh 1D",
                      (templateRankSize_ > 1 ? templateRankSize_ : 1), templateRankSize_);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempReduceScatterNHR, "ReduceScatter NHR", 1, templateRankSize_);
// reduce_scatter aicpu_reduce_nhr.cc:46-50, :242-249: one thread, N scratch slots
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempReduceScatterAicpuReduceNHR, "ReduceScatter NHR gather + local reduce", 1, templateRankSize_);
// reduce_scatter_v mesh_1D.cc:26-48: N-1 threads (the main thread sends too), N scratch slots
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempReduceScatterVMesh1D, "ReduceScatterV mesh 1D",
                      (templateRankSize_ > 1 ? templateRankSize_ - 1 : 1), templateRankSize_);
// mesh-chunk templates (mesh_chunk_templates.cc): reduce_scatter meshchunk.cc:25-52 (N-1 threads, N-1 scratch
// multiple); all_reduce two_shot_mesh_chunk.cc:17-38 (N threads, scratch multiple 2)
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempReduceScatterMesh1DMeshChunk, "ReduceScatter mesh 1D, chunked",
                      (templateRankSize_ > 1 ? templateRankSize_ - 1 : 1), (templateRankSize_ > 0 ? templateRankSize_ - 1 : 0));
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceMesh1DTwoShotMeshChunk, "AllReduce mesh 1D two-shot, chunked",
                      (templateRankSize_ > 1 ? templateRankSize_ : 1), 2);
// Where each rank's block sits in the scratch buffer during one loop of the order-preserved ReduceScatter
// (ins_v2_reduce_scatter_order_preserved_executor.h:37-42).
struct MemBlockInfo {
    std::vector<u64> size;
    std::vector<u64> userInputOffsets;
    std::vector<u64> inputOffsets;
    std::vector<u64> outputOffsets;
};

// order_preserved_level1.cc:35-50, :128-131: N threads, N scratch slots
class InsTempReduceScatterOrderPreservedLevel1 : public InsAlgTemplateBase {
public:
    using InsAlgTemplateBase::InsAlgTemplateBase;
    std::string Describe() const override { return "ReduceScatter, order preserved"; }
    u64 GetThreadNum() const override { return templateRankSize_ > 1 ? templateRankSize_ : 1; }
    u64 CalcScratchMultiple(BufferType, BufferType) override { return templateRankSize_; }
    HcclResult KernelRun(const OpParam &param, const TemplateDataParams &tempAlgParams,
                         TemplateResource &templateResource) override;
    void SetMemBlockInfo(const MemBlockInfo &info) { memBlockInfo_ = info; }
    bool ClosedForm(const TemplateDataParams &tempAlgParams, u64 dataTypeSize, std::vector<ClosedFold> &out) const override;

protected:
    // the peers in the order their shards are sent: ranks me+1, me+2, ... (:200-240)
    virtual std::vector<u32> SendOrder(u32 me) const;
    // slot of the block that rank `peer` sent to rank `localRank` (:153-158)
    u32 CalcOutputIndex(u32 peer, u32 localRank) const { return (peer + localRank) % templateRankSize_; }
    MemBlockInfo memBlockInfo_;
};

// The variant for more than 32 ranks (order_preserved_group.cc:35-61, :132-141, :236-262): at most
// ORDER_PRESERVED_MAX_THREADS threads, and the shards go out by growing distance, right neighbour then left.
// Slots and the tree are the ones of the level-1 template, so the results are the same bits.
constexpr u32 ORDER_PRESERVED_MAX_THREADS = 32;  // src/common/order_preserved_common.h:24-33
class InsTempReduceScatterOrderPreservedGroup : public InsTempReduceScatterOrderPreservedLevel1 {
public:
    using InsTempReduceScatterOrderPreservedLevel1::InsTempReduceScatterOrderPreservedLevel1;
    std::string Describe() const override { return "ReduceScatter, order preserved, grouped all-to-all"; }
    u64 GetThreadNum() const override
    {
        const u32 n = templateRankSize_ > 1 ? templateRankSize_ : 1;
        return n < ORDER_PRESERVED_MAX_THREADS ? n : ORDER_PRESERVED_MAX_THREADS;
    }

protected:
    std::vector<u32> SendOrder(u32 me) const override;
};

HCCL_DECLARE_TEMPLATE(InsTempAllGatherMesh1D, "AllGather mesh 1D",
                      (templateRankSize_ > 1 ? templateRankSize_ - 1 : 1), templateRankSize_);
HCCL_DECLARE_TEMPLATE(InsTempAllGatherNHR, "AllGather NHR", 1, templateRankSize_);
HCCL_DECLARE_TEMPLATE(InsTempAllGatherVMesh1D, "AllGatherV mesh 1D",
                      (templateRankSize_ > 1 ? templateRankSize_ - 1 : 1), templateRankSize_);

constexpr u32 ALLTOALLV_DIRECT_FULLMESH_CONCURRENT_SIZE = 16;

class InsTempAlltoAllVMesh1D : public InsAlgTemplateBase {
public:
    using InsAlgTemplateBase::InsAlgTemplateBase;
    std::string Describe() const override { return "AlltoAllV mesh 1D"; }
    u64 GetThreadNum() const override { return Concurrent() + 1; }
    u64 CalcScratchMultiple(BufferType, BufferType) override { return Concurrent(); }
    HcclResult KernelRun(const OpParam &param, const TemplateDataParams &tempAlgParams,
                         TemplateResource &templateResource) override;
    // peers of one round: left and right neighbours at growing distance (mesh_1D.cc:75-93)
    void CalcCommRankSetForOneLoop(u32 roundIdx, u32 remainRankSize, std::vector<u32> &commRanks) const;
    // which scratch slot each side of a pair uses (mesh_1D.cc:101-126)
    void CalcCclBuffIdx(u32 remoteRank, u32 &myRankCclBuffIdx, u32 &remoteCclBuffIdx) const;

private:
    u32 Concurrent() const
    {
        const u32 peers = templateRankSize_ > 0 ? templateRankSize_ - 1 : 0;
        return peers < ALLTOALLV_DIRECT_FULLMESH_CONCURRENT_SIZE ? peers : ALLTOALLV_DIRECT_FULLMESH_CONCURRENT_SIZE;
    }
};

}  // namespace ops_hccl
