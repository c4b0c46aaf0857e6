// The data-movement verbs the templates call (reference: src/ops/op_common/template/wrapper/
// alg_data_trans_wrapper.{h,cc}).  Each verb checks its slices and expands to the primitive calls and the
// ACK / DATA_SIGNAL handshakes of the reference, in the reference's order; the *Batch* names take the
// reference's per-slice fall-back path (wrapper.cc:127-226), which is what its system tests run.
#pragma once
#include "alg_param.h"

namespace ops_hccl {

HcclResult LocalCopy(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice);
HcclResult LocalReduce(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice,
                       HcclDataType dataType, HcclReduceOp reduceOp);
HcclResult LocalCopySlices(const ThreadHandle &thread, const std::vector<DataSlice> &srcSlices,
                           const std::vector<DataSlice> &dstSlices);
bool IsContinuousSlice(const DataSlice &nxtSlice, const DataSlice &currSlice);

HcclResult SendWrite(const DataInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvWrite(const DataInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvWrite(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRead(const DataInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvRead(const DataInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvRead(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRecvWriteReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRecvReadReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);

inline HcclResult SendBatchWrite(const DataInfo &i, const ThreadHandle &t) { return SendWrite(i, t); }
inline HcclResult SendRecvBatchWrite(const SendRecvInfo &i, const ThreadHandle &t) { return SendRecvWrite(i, t); }
inline HcclResult RecvBatchRead(const DataInfo &i, const ThreadHandle &t) { return RecvRead(i, t); }
inline HcclResult SendRecvBatchRead(const SendRecvInfo &i, const ThreadHandle &t) { return SendRecvRead(i, t); }
inline HcclResult SendRecvBatchWriteReduce(const SendRecvReduceInfo &i, const ThreadHandle &t)
{
    return SendRecvWriteReduce(i, t);
}

HcclResult PreSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                               const std::vector<u32> &notifyIdxMainToSub);
HcclResult PostSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                                const std::vector<u32> &notifyIdxSubToMain);

}  // namespace ops_hccl
