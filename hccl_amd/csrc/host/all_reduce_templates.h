// AllReduce templates: see all_reduce_templates.cc for what each restates.
#pragma once
#include "hcomm_primitives.h"
#include "template_base.h"

namespace ops_hccl {

#define HCCL_DECLARE_TEMPLATE(CLASS, NAME, THREADS, SCRATCH)                                              \
    class CLASS : public InsAlgTemplateBase {                                                             \
    public:                                                                                               \
        using InsAlgTemplateBase::InsAlgTemplateBase;                                                     \
        std::string Describe() const override { return NAME; }                                            \
        u64 GetThreadNum() const override { return THREADS; }                                             \
        u64 CalcScratchMultiple(BufferType, BufferType) override { return SCRATCH; }                      \
        HcclResult KernelRun(const OpParam &param, const TemplateDataParams &tempAlgParams,               \
                             TemplateResource &templateResource) override;                                \
    }

// The same for a template that also states its result in closed form.
#define HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(CLASS, NAME, THREADS, SCRATCH)                             \
    class CLASS : public InsAlgTemplateBase {                                                             \
    public:                                                                                               \
        using InsAlgTemplateBase::InsAlgTemplateBase;                                                     \
        std::string Describe() const override { return NAME; }                                            \
        u64 GetThreadNum() const override { return THREADS; }                                             \
        u64 CalcScratchMultiple(BufferType, BufferType) override { return SCRATCH; }                      \
        HcclResult KernelRun(const OpParam &param, const TemplateDataParams &tempAlgParams,               \
                             TemplateResource &templateResource) override;                                \
        bool ClosedForm(const TemplateDataParams &tempAlgParams, u64 dataTypeSize,                        \
                        std::vector<ClosedFold> &out) const override;                                     \
    }

// scratch multiples: one_shot.cc:42-48 (N), two_shot.cc:20-27 (2), nhr.cc:20-26 (1), aicpu_reduce_nhr.cc:22-28 (N)
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceMesh1DOneShot, "AllReduce mesh 1D one-shot",
                      (templateRankSize_ > 1 ? templateRankSize_ : 1), templateRankSize_);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceMesh1DTwoShot, "AllReduce mesh 1D two-shot",
                      (templateRankSize_ > 1 ? templateRankSize_ : 1), 2);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceNHR, "AllReduce NHR", 1, 1);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceAicpuReduceNHR, "AllReduce NHR gather + local reduce", 1,
                                       templateRankSize_);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceRing, "AllReduce ring", 1, 1);
HCCL_DECLARE_TEMPLATE_WITH_CLOSED_FORM(InsTempAllReduceRHD, "AllReduce recursive halving-doubling", 1, 1);

// Block of ranks that runs halving-doubling when n is not a power of two: the even rank of each of the
// first `extra` pairs, then every rank from 2 * extra on (RHD.md:17).
void RhdBlock(u32 n, u32 &extra, std::vector<u32> &block);

}  // namespace ops_hccl
