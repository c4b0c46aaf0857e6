// A plug-in: AllReduce templates written against the template-facing API (host/*.h) from outside the library and
// registered through REGISTER_EXEC_V2, the way a maintainer adds an algorithm to the reference
// (src/ops/op_common/executor/registry/coll_alg_v2_exec_registry.h:71-72).  They exist to exercise the one-sided
// reduce verbs of the wrapper (src/ops/op_common/template/wrapper/alg_data_trans_wrapper.h:33-76), which none of the
// built-in templates call: one rank (the root, rank 0) collects every rank's data with the verb under test, then
// hands the result out.  Every variant computes  x_{n-1} (+) (... (x_1 (+) x_0))  on every rank.
//
//   make -C hccl_amd/csrc      (builds hccl_amd/lib/libhccl_one_sided_templates.so)
//   load it after libhccl_amd.so (dlopen / ctypes.CDLL with RTLD_GLOBAL), then select by name:
//   hcclxCommSetAlgorithm(comm, HCCLX_CMD_ALLREDUCE, "ExampleAllReduceReadReduce")
#include "host/data_move_templates.h"
#include "host/sole_executors.h"

using namespace ops_hccl;

namespace {

enum class Verb { READ_REDUCE, BATCH_READ_REDUCE, WRITE_REDUCE, BATCH_WRITE_REDUCE, READ_THEN_AICPU_REDUCE };

// Scratch slots of a rank (each p.sliceSize bytes): slot 0 the value being collected (the root) or the rank's own
// data (the others, for the root to read); slot 1 where the root's result lands; slot 2 + k what the root fetched
// from rank k (READ_THEN_AICPU_REDUCE only).
template <Verb V>
class RootCollects : public InsAlgTemplateBase {
public:
    using InsAlgTemplateBase::InsAlgTemplateBase;
    std::string Describe() const override { return "AllReduce: the root collects with a one-sided reduce verb"; }
    u64 GetThreadNum() const override { return 1; }
    u64 CalcScratchMultiple(BufferType, BufferType) override { return templateRankSize_ + 2; }

    HcclResult KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res) override
    {
        CHK_PRT_RET(res.threads.empty(), HCCL_ERROR("[RootCollects] no thread"), HCCL_E_INTERNAL);
        if (p.count == 0) return HCCL_SUCCESS;
        const HcclDataType dt = param.DataDes.dataType;
        const u32 n = templateRankSize_;
        const u64 size = p.sliceSize;
        const u64 count = p.count;
        const u64 base = p.buffInfo.hcclBuffBaseOff;
        const ThreadHandle th = res.threads[0];
        void *ccl = p.buffInfo.hcclBuff.addr;
        auto slot = [&](void *buf, u64 k) { return DataSlice(buf, base + k * size, size, count); };
        const DataSlice usrIn(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, size, count);
        const DataSlice usrOut(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size, count);

        CHK_RET(LocalCopy(th, usrIn, slot(ccl, 0)));
        if (n == 1) return LocalCopy(th, slot(ccl, 0), usrOut);

        if (myRank_ == 0) {
            for (u32 k = 1; k < n; ++k) {   // ranks ascending: slot 0 = x_k (+) slot 0
                const ChannelInfo &link = res.channels.at(subCommRanks_[0][k])[0];
                const DataReduceInfo fetch(link, {{slot(link.remoteCclMem.addr, 0)}, {slot(ccl, 0)}}, dt, reduceOp_);
                switch (V) {
                    case Verb::READ_REDUCE:
                        CHK_RET(RecvReadReduce(fetch, th));
                        break;
                    case Verb::BATCH_READ_REDUCE:
                        CHK_RET(RecvBatchReadReduce(fetch, th));
                        break;
                    case Verb::WRITE_REDUCE:
                    case Verb::BATCH_WRITE_REDUCE:
                        CHK_RET(RecvWriteReduce(fetch, th));   // the peer does the work; slices unused on this side
                        break;
                    case Verb::READ_THEN_AICPU_REDUCE:
                        CHK_RET(RecvRead(DataInfo(link, {{slot(link.remoteCclMem.addr, 0)}, {slot(ccl, 2 + k)}}), th));
                        CHK_RET(AicpuReduce(th, slot(ccl, 2 + k), slot(ccl, 0), dt, reduceOp_));
                        break;
                }
            }
            for (u32 k = 1; k < n; ++k) {   // hand the result out
                const ChannelInfo &link = res.channels.at(subCommRanks_[0][k])[0];
                CHK_RET(SendWrite(DataInfo(link, {{slot(ccl, 0)}, {slot(link.remoteCclMem.addr, 1)}}), th));
            }
            return LocalCopy(th, slot(ccl, 0), usrOut);
        }

        const ChannelInfo &root = res.channels.at(subCommRanks_[0][0])[0];
        const DataReduceInfo give(root, {{slot(ccl, 0)}, {slot(root.remoteCclMem.addr, 0)}}, dt, reduceOp_);
        switch (V) {
            case Verb::READ_REDUCE:
            case Verb::BATCH_READ_REDUCE:
                CHK_RET(SendReadReduce(give, th));             // the root does the work
                break;
            case Verb::WRITE_REDUCE:
                CHK_RET(SendWriteReduce(give, th));
                break;
            case Verb::BATCH_WRITE_REDUCE:
                CHK_RET(SendBatchWriteReduce(give, th));
                break;
            case Verb::READ_THEN_AICPU_REDUCE:
                CHK_RET(SendRead(DataInfo(root, {{slot(ccl, 0)}, {slot(root.remoteCclMem.addr, 2 + myRank_)}}), th));
                break;
        }
        CHK_RET(RecvWrite(DataInfo(root, {{slot(root.remoteCclMem.addr, 0)}, {slot(ccl, 1)}}), th));
        return LocalCopy(th, slot(ccl, 1), usrOut);
    }
};

// Two ranks fetch each other's data with the two-sided batch read-reduce: out_r = x_other (+) x_r.
class PairReadsEachOther : public InsAlgTemplateBase {
public:
    using InsAlgTemplateBase::InsAlgTemplateBase;
    std::string Describe() const override { return "AllReduce of two ranks: each read-reduces the other's data"; }
    u64 GetThreadNum() const override { return 1; }
    u64 CalcScratchMultiple(BufferType, BufferType) override { return 1; }

    HcclResult KernelRun(const OpParam &param, const TemplateDataParams &p, TemplateResource &res) override
    {
        CHK_PRT_RET(templateRankSize_ != 2, HCCL_ERROR("[PairReadsEachOther] needs exactly two ranks"), HCCL_E_NOT_SUPPORT);
        if (p.count == 0) return HCCL_SUCCESS;
        const ThreadHandle th = res.threads[0];
        const DataSlice own(p.buffInfo.hcclBuff.addr, p.buffInfo.hcclBuffBaseOff, p.sliceSize, p.count);
        const DataSlice usrIn(p.buffInfo.inputPtr, p.buffInfo.inBuffBaseOff, p.sliceSize, p.count);
        const DataSlice usrOut(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, p.sliceSize, p.count);
        CHK_RET(LocalCopy(th, usrIn, own));
        CHK_RET(LocalCopy(th, usrIn, usrOut));
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][1 - myRank_])[0];
        const DataSlice theirs(link.remoteCclMem.addr, p.buffInfo.hcclBuffBaseOff, p.sliceSize, p.count);
        SendRecvReduceInfo info{{link, link}, {{{own}, {theirs}}, {{theirs}, {usrOut}}}, param.DataDes.dataType, reduceOp_};
        return SendRecvBatchReadReduce(info, th);
    }
};

using ReadReduce = RootCollects<Verb::READ_REDUCE>;
using BatchReadReduce = RootCollects<Verb::BATCH_READ_REDUCE>;
using WriteReduce = RootCollects<Verb::WRITE_REDUCE>;
using BatchWriteReduce = RootCollects<Verb::BATCH_WRITE_REDUCE>;
using ReadThenAicpuReduce = RootCollects<Verb::READ_THEN_AICPU_REDUCE>;

}  // namespace

REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReduceReadReduce, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 ReadReduce);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReduceBatchReadReduce, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 BatchReadReduce);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReduceWriteReduce, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 WriteReduce);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReduceBatchWriteReduce, InsV2AllReduceSoleExecutor, TopoMatch1D,
                 BatchWriteReduce);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReduceReadThenAicpuReduce, InsV2AllReduceSoleExecutor,
                 TopoMatch1D, ReadThenAicpuReduce);
REGISTER_EXEC_V2(HcclCMDType::HCCL_CMD_ALLREDUCE, ExampleAllReducePairReadsEachOther, InsV2AllReduceSoleExecutor,
                 TopoMatch1D, PairReadsEachOther);
