#include "alg_data_trans_wrapper.h"

#include <cstdlib>

#include "hcomm_primitives.h"

namespace ops_hccl {

namespace {
constexpr u32 kTimeout = CUSTOM_TIMEOUT;

HcclResult R(int32_t rc) { return static_cast<HcclResult>(rc); }

// Every wait of a verb takes the process-wide time-out when the backend exports the *WithDefaultTimeout form and
// falls back to the explicit one otherwise (wrapper.cc:22-31 over hcomm_primitives_dl.cc:155-173).  This backend
// exports both; HCCL_VRANK_NO_DEFAULT_TIMEOUT=1 takes the fallback, so that both routes stay exercised.
bool UseDefaultTimeout()
{
    static const bool on = [] {
        const char *v = std::getenv("HCCL_VRANK_NO_DEFAULT_TIMEOUT");
        return !(v != nullptr && v[0] == '1');
    }();
    return on;
}

HcclResult WaitChannel(const ThreadHandle &thread, const ChannelInfo &ch, u32 idx)
{
    if (UseDefaultTimeout()) return R(HcommChannelNotifyWaitOnThreadWithDefaultTimeout(thread, ch.handle, idx));
    return R(HcommChannelNotifyWaitOnThread(thread, ch.handle, idx, kTimeout));
}

HcclResult WaitThread(const ThreadHandle &thread, u32 idx)
{
    if (UseDefaultTimeout()) return R(HcommThreadNotifyWaitOnThreadWithDefaultTimeout(thread, idx));
    return R(HcommThreadNotifyWaitOnThread(thread, idx, kTimeout));
}

// LocalReduce routes 64-bit types and PROD to the CPU loop AicpuReduce, everything else to the inline
// reduce of the transport (wrapper.cc:837-841).  Both are the same fold kernel here, so the two routes
// only differ in the checks they make.
bool NeedsAicpuReduce(HcclDataType dt, HcclReduceOp op)
{
    return dt == HCCL_DATA_TYPE_INT64 || dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64 ||
           op == HCCL_REDUCE_PROD;
}

bool AicpuReduceSupports(HcclDataType dt)
{
    switch (dt) {  // wrapper.cc:1176-1207
        case HCCL_DATA_TYPE_INT8:
        case HCCL_DATA_TYPE_INT32:
        case HCCL_DATA_TYPE_FP16:
        case HCCL_DATA_TYPE_FP32:
        case HCCL_DATA_TYPE_INT64:
        case HCCL_DATA_TYPE_UINT64:
        case HCCL_DATA_TYPE_FP64:
            return true;
        default:
            return false;
    }
}

HcclResult CheckReduceSlices(const DataSlice &src, const DataSlice &dst, HcclDataType dt)
{
    CHK_PRT_RET(src.count_ * DATATYPE_SIZE_TABLE[dt] != src.size_,
                HCCL_ERROR("reduce: src slice count does not match its size"), HCCL_E_INTERNAL);
    CHK_PRT_RET(dst.count_ * DATATYPE_SIZE_TABLE[dt] != dst.size_,
                HCCL_ERROR("reduce: dst slice count does not match its size"), HCCL_E_INTERNAL);
    return HCCL_SUCCESS;
}
}  // namespace

HcclResult LocalCopy(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice)
{
    if (srcSlice.size_ == 0) return HCCL_SUCCESS;  // zero-size copy is a no-op success (wrapper.cc:817-819)
    CHK_PRT_RET(srcSlice.size_ != dstSlice.size_, HCCL_ERROR("LocalCopy: slice sizes differ"), HCCL_E_INTERNAL);
    return R(HcommLocalCopyOnThread(thread, GetSliceAddr(dstSlice), GetSliceAddr(srcSlice), srcSlice.size_));
}

HcclResult LocalReduce(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice,
                       HcclDataType dataType, HcclReduceOp reduceOp)
{
    if (NeedsAicpuReduce(dataType, reduceOp)) return AicpuReduce(thread, srcSlice, dstSlice, dataType, reduceOp);
    if (srcSlice.size_ == 0) return HCCL_SUCCESS;
    CHK_PRT_RET(srcSlice.size_ != dstSlice.size_, HCCL_ERROR("LocalReduce: slice sizes differ"), HCCL_E_INTERNAL);
    return R(HcommLocalReduceOnThread(thread, GetSliceAddr(dstSlice), GetSliceAddr(srcSlice), srcSlice.count_,
                                      dataType, reduceOp));
}

// The CPU reduce of the reference (wrapper.cc:1165-1210): equal byte sizes, seven element types, anything else is
// HCCL_E_INTERNAL.  The reference runs the loop on the host at once and ignores `thread`; here the step is recorded
// on `thread` like every other reduce and becomes part of the launch.
HcclResult AicpuReduce(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice,
                       HcclDataType dataType, HcclReduceOp reduceOp)
{
    CHK_PRT_RET(srcSlice.size_ != dstSlice.size_, HCCL_ERROR("AicpuReduce: slice sizes differ"), HCCL_E_INTERNAL);
    CHK_PRT_RET(!AicpuReduceSupports(dataType), HCCL_ERROR("AicpuReduce: DataType[%d] not support", dataType),
                HCCL_E_INTERNAL);
    const u64 count = srcSlice.size_ / DATATYPE_SIZE_TABLE[dataType];
    return R(HcommLocalReduceOnThread(thread, GetSliceAddr(dstSlice), GetSliceAddr(srcSlice), count, dataType,
                                      reduceOp));
}

bool IsContinuousSlice(const DataSlice &nxtSlice, const DataSlice &currSlice)
{
    return nxtSlice.addr_ == currSlice.addr_ && nxtSlice.offset_ == currSlice.offset_ + currSlice.size_;
}

HcclResult LocalCopySlices(const ThreadHandle &thread, const std::vector<DataSlice> &srcSlices,
                           const std::vector<DataSlice> &dstSlices)
{
    CHK_PRT_RET(srcSlices.size() != dstSlices.size(), HCCL_ERROR("LocalCopySlices: slice counts differ"),
                HCCL_E_INTERNAL);
    // Address-contiguous neighbours are merged into one copy (wrapper.cc:864-924).
    bool open = false;
    DataSlice runSrc, runDst;
    for (size_t i = 0; i < srcSlices.size(); ++i) {
        if (srcSlices[i].size_ == 0) continue;
        CHK_PRT_RET(srcSlices[i].size_ != dstSlices[i].size_, HCCL_ERROR("LocalCopySlices: slice sizes differ"),
                    HCCL_E_INTERNAL);
        if (open && IsContinuousSlice(srcSlices[i], runSrc) && IsContinuousSlice(dstSlices[i], runDst)) {
            runSrc.size_ += srcSlices[i].size_;
            runDst.size_ += dstSlices[i].size_;
            continue;
        }
        if (open) CHK_RET(LocalCopy(thread, runSrc, runDst));
        runSrc = DataSlice(srcSlices[i].addr_, srcSlices[i].offset_, srcSlices[i].size_);
        runDst = DataSlice(dstSlices[i].addr_, dstSlices[i].offset_, dstSlices[i].size_);
        open = true;
    }
    if (open) CHK_RET(LocalCopy(thread, runSrc, runDst));
    return HCCL_SUCCESS;
}

// ---- write family: the receiver says "my buffer is free" (ACK), the sender writes and says "data is there"

HcclResult SendWrite(const DataInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < sendInfo.slices_.srcSlices_.size(); ++i) {
        const DataSlice &s = sendInfo.slices_.srcSlices_[i];
        const DataSlice &d = sendInfo.slices_.dstSlices_[i];
        if (s.size_ == 0) continue;
        CHK_RET(HcommWriteOnThread(thread, ch.handle, GetSliceAddr(d), GetSliceAddr(s), s.size_));
    }
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult RecvWrite(const DataInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_ACK));
    return WaitChannel(thread, ch, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult SendRecvWrite(const SendRecvInfo &info, const ThreadHandle &thread)
{
    const auto &src = info.sendRecvSlices_.txSlicesList_.srcSlices_;
    const auto &dst = info.sendRecvSlices_.txSlicesList_.dstSlices_;
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, tx, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < src.size(); ++i) {
        if (src[i].size_ == 0) continue;
        CHK_RET(HcommWriteOnThread(thread, tx.handle, GetSliceAddr(dst[i]), GetSliceAddr(src[i]), src[i].size_));
    }
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, rx, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult SendRecvWriteReduce(const SendRecvReduceInfo &info, const ThreadHandle &thread)
{
    const auto &src = info.sendRecvSlices_.txSlicesList_.srcSlices_;
    const auto &dst = info.sendRecvSlices_.txSlicesList_.dstSlices_;
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, tx, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < src.size(); ++i) {
        if (src[i].size_ == 0) continue;
        CHK_RET(CheckReduceSlices(src[i], dst[i], info.dataType_));
        CHK_RET(HcommWriteReduceOnThread(thread, tx.handle, GetSliceAddr(dst[i]), GetSliceAddr(src[i]), src[i].count_,
                                         info.dataType_, info.reduceType_));
    }
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, rx, NOTIFY_IDX_DATA_SIGNAL);
}

// One side of SendRecvWriteReduce each: the sender waits for the receiver's ACK, write-reduces its slices into the
// receiver's buffer and signals; the receiver only shakes hands (wrapper.cc:389-435, :468-477).
HcclResult SendWriteReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < sendInfo.slices_.srcSlices_.size(); ++i) {
        const DataSlice &s = sendInfo.slices_.srcSlices_[i];
        const DataSlice &d = sendInfo.slices_.dstSlices_[i];
        if (s.size_ == 0) continue;
        CHK_RET(CheckReduceSlices(s, d, sendInfo.dataType_));
        CHK_RET(HcommWriteReduceOnThread(thread, ch.handle, GetSliceAddr(d), GetSliceAddr(s), s.count_, sendInfo.dataType_,
                                         sendInfo.reduceType_));
    }
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult RecvWriteReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_ACK));
    return WaitChannel(thread, ch, NOTIFY_IDX_DATA_SIGNAL);
}

// ---- read family: the owner says "my data is ready" (ACK), the reader reads and says "I am done"

// One side of SendRecvReadReduce each: the owner of the data announces it and waits until it has been read; the
// reader read-reduces the owner's slices into its own buffer (wrapper.cc:638-695).
HcclResult SendReadReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_ACK));
    return WaitChannel(thread, ch, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult RecvReadReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < recvInfo.slices_.srcSlices_.size(); ++i) {
        const DataSlice &s = recvInfo.slices_.srcSlices_[i];
        const DataSlice &d = recvInfo.slices_.dstSlices_[i];
        if (s.size_ == 0) continue;
        CHK_RET(CheckReduceSlices(s, d, recvInfo.dataType_));
        CHK_RET(HcommReadReduceOnThread(thread, ch.handle, GetSliceAddr(d), GetSliceAddr(s), s.count_, recvInfo.dataType_,
                                        recvInfo.reduceType_));
    }
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult SendRead(const DataInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_ACK));
    return WaitChannel(thread, ch, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult RecvRead(const DataInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < recvInfo.slices_.srcSlices_.size(); ++i) {
        const DataSlice &s = recvInfo.slices_.srcSlices_[i];
        const DataSlice &d = recvInfo.slices_.dstSlices_[i];
        if (s.size_ == 0) continue;
        CHK_RET(HcommReadOnThread(thread, ch.handle, GetSliceAddr(d), GetSliceAddr(s), s.size_));
    }
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult SendRecvRead(const SendRecvInfo &info, const ThreadHandle &thread)
{
    const auto &src = info.sendRecvSlices_.rxSlicesList_.srcSlices_;
    const auto &dst = info.sendRecvSlices_.rxSlicesList_.dstSlices_;
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, rx, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < src.size(); ++i) {
        if (src[i].size_ == 0) continue;
        CHK_RET(HcommReadOnThread(thread, rx.handle, GetSliceAddr(dst[i]), GetSliceAddr(src[i]), src[i].size_));
    }
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, tx, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult SendRecvReadReduce(const SendRecvReduceInfo &info, const ThreadHandle &thread)
{
    const auto &src = info.sendRecvSlices_.rxSlicesList_.srcSlices_;
    const auto &dst = info.sendRecvSlices_.rxSlicesList_.dstSlices_;
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, rx, NOTIFY_IDX_ACK));
    for (size_t i = 0; i < src.size(); ++i) {
        if (src[i].size_ == 0) continue;
        CHK_RET(CheckReduceSlices(src[i], dst[i], info.dataType_));
        CHK_RET(HcommReadReduceOnThread(thread, rx.handle, GetSliceAddr(dst[i]), GetSliceAddr(src[i]), src[i].count_,
                                        info.dataType_, info.reduceType_));
    }
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, tx, NOTIFY_IDX_DATA_SIGNAL);
}

// ---- batch verbs: every slice of the call in one descriptor array (wrapper.cc:99-125), between the handshakes of
//      the per-slice verbs (DoSendBatchTx :151-168, DoSendRecvBatchTx :127-149, DoRecvBatchRx :171-187)

namespace {

HcclResult RunBatch(const ThreadHandle &thread, const ChannelInfo &ch, const std::vector<DataSlice> &src,
                    const std::vector<DataSlice> &dst, HcclHcommTransferType type, bool reduce, HcclDataType dataType,
                    HcclReduceOp reduceOp)
{
    std::vector<HcclHcommBatchTransferDesc> descs;
    for (size_t i = 0; i < src.size(); ++i) {
        if (src[i].size_ == 0) continue;   // :110-113
        HcclHcommBatchTransferDesc d = {};
        d.transType = type;
        if (reduce) {
            CHK_RET(CheckReduceSlices(src[i], dst[i], dataType));
            d.transferInfo.reduce.count = src[i].count_;
            d.transferInfo.reduce.dst = GetSliceAddr(dst[i]);
            d.transferInfo.reduce.src = GetSliceAddr(src[i]);
            d.transferInfo.reduce.dataType = dataType;
            d.transferInfo.reduce.reduceOp = reduceOp;
        } else {
            d.transferInfo.write.len = src[i].size_;
            d.transferInfo.write.dst = GetSliceAddr(dst[i]);
            d.transferInfo.write.src = GetSliceAddr(src[i]);
        }
        descs.push_back(d);
    }
    if (descs.empty()) return HCCL_SUCCESS;
    return R(HcommBatchTransferOnThread(thread, ch.handle, descs.data(), static_cast<uint32_t>(descs.size())));
}

}  // namespace

HcclResult SendBatchWrite(const DataInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, ch, sendInfo.slices_.srcSlices_, sendInfo.slices_.dstSlices_, HCCL_HCOMM_TRANSFER_TYPE_WRITE,
                     false, HCCL_DATA_TYPE_INT8, HCCL_REDUCE_SUM));
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult SendRecvBatchWrite(const SendRecvInfo &info, const ThreadHandle &thread)
{
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, tx, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, tx, info.sendRecvSlices_.txSlicesList_.srcSlices_, info.sendRecvSlices_.txSlicesList_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_WRITE, false, HCCL_DATA_TYPE_INT8, HCCL_REDUCE_SUM));
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, rx, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult SendRecvBatchWriteReduce(const SendRecvReduceInfo &info, const ThreadHandle &thread)
{
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, tx, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, tx, info.sendRecvSlices_.txSlicesList_.srcSlices_, info.sendRecvSlices_.txSlicesList_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE, true, info.dataType_, info.reduceType_));
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, rx, NOTIFY_IDX_DATA_SIGNAL);
}

HcclResult RecvBatchRead(const DataInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, ch, recvInfo.slices_.srcSlices_, recvInfo.slices_.dstSlices_, HCCL_HCOMM_TRANSFER_TYPE_READ,
                     false, HCCL_DATA_TYPE_INT8, HCCL_REDUCE_SUM));
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult SendRecvBatchRead(const SendRecvInfo &info, const ThreadHandle &thread)
{
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, rx, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, rx, info.sendRecvSlices_.rxSlicesList_.srcSlices_, info.sendRecvSlices_.rxSlicesList_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_READ, false, HCCL_DATA_TYPE_INT8, HCCL_REDUCE_SUM));
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, tx, NOTIFY_IDX_DATA_SIGNAL);
}

// The one-sided reduce verbs and the two-sided read-reduce in their batch form (wrapper.cc:437-466, :697-726,
// :784-813): the same handshakes around one descriptor array.
HcclResult SendBatchWriteReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = sendInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, ch, sendInfo.slices_.srcSlices_, sendInfo.slices_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE, true, sendInfo.dataType_, sendInfo.reduceType_));
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult RecvBatchReadReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread)
{
    const ChannelInfo &ch = recvInfo.channel_;
    CHK_RET(WaitChannel(thread, ch, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, ch, recvInfo.slices_.srcSlices_, recvInfo.slices_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_READ_REDUCE, true, recvInfo.dataType_, recvInfo.reduceType_));
    return R(HcommChannelNotifyRecordOnThread(thread, ch.handle, NOTIFY_IDX_DATA_SIGNAL));
}

HcclResult SendRecvBatchReadReduce(const SendRecvReduceInfo &info, const ThreadHandle &thread)
{
    const ChannelInfo &tx = info.sendRecvChannels_.txChannel_;
    const ChannelInfo &rx = info.sendRecvChannels_.rxChannel_;
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, tx.handle, NOTIFY_IDX_ACK));
    CHK_RET(WaitChannel(thread, rx, NOTIFY_IDX_ACK));
    CHK_RET(RunBatch(thread, rx, info.sendRecvSlices_.rxSlicesList_.srcSlices_, info.sendRecvSlices_.rxSlicesList_.dstSlices_,
                     HCCL_HCOMM_TRANSFER_TYPE_READ_REDUCE, true, info.dataType_, info.reduceType_));
    CHK_RET(HcommChannelNotifyRecordOnThread(thread, rx.handle, NOTIFY_IDX_DATA_SIGNAL));
    return WaitChannel(thread, tx, NOTIFY_IDX_DATA_SIGNAL);
}

// Whether HcommBatchTransferOnThread is there (wrapper.cc:244-247; in the reference the answer comes from dlsym):
// this backend always has it.
bool IsHcommBatchTransferOnThreadSupported() { return true; }

// ---- main thread <-> sub threads

HcclResult PreSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                               const std::vector<u32> &notifyIdxMainToSub)
{
    CHK_PRT_RET(subThreads.empty() || notifyIdxMainToSub.empty(), HCCL_ERROR("PreSyncInterThreads: empty"),
                HCCL_E_INTERNAL);
    CHK_PRT_RET(subThreads.size() != notifyIdxMainToSub.size(), HCCL_ERROR("PreSyncInterThreads: size mismatch"),
                HCCL_E_INTERNAL);
    for (size_t i = 0; i < subThreads.size(); ++i) {
        CHK_RET(HcommThreadNotifyRecordOnThread(mainThread, subThreads[i], notifyIdxMainToSub[i]));
    }
    for (size_t i = 0; i < subThreads.size(); ++i) {
        CHK_RET(WaitThread(subThreads[i], notifyIdxMainToSub[i]));
    }
    return HCCL_SUCCESS;
}

HcclResult PostSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                                const std::vector<u32> &notifyIdxSubToMain)
{
    CHK_PRT_RET(subThreads.empty() || notifyIdxSubToMain.empty(), HCCL_ERROR("PostSyncInterThreads: empty"),
                HCCL_E_INTERNAL);
    CHK_PRT_RET(subThreads.size() != notifyIdxSubToMain.size(), HCCL_ERROR("PostSyncInterThreads: size mismatch"),
                HCCL_E_INTERNAL);
    for (size_t i = 0; i < subThreads.size(); ++i) {
        CHK_RET(WaitThread(mainThread, notifyIdxSubToMain[i]));
    }
    for (size_t i = 0; i < subThreads.size(); ++i) {
        CHK_RET(HcommThreadNotifyRecordOnThread(subThreads[i], mainThread, notifyIdxSubToMain[i]));
    }
    return HCCL_SUCCESS;
}

}  // namespace ops_hccl
