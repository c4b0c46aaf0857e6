// The data-movement verbs the templates call (reference: src/ops/op_common/template/wrapper/
// alg_data_trans_wrapper.{h,cc}).  Each verb checks its slices and expands to the primitive calls and the
// ACK / DATA_SIGNAL handshakes of the reference, in the reference's order.  The *Batch* verbs hand all slices of a
// call to HcommBatchTransferOnThread in one descriptor array, between the same handshakes (wrapper.cc:99-226).
#pragma once
#include "alg_param.h"

namespace ops_hccl {

HcclResult LocalCopy(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice);
HcclResult LocalReduce(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice,
                       HcclDataType dataType, HcclReduceOp reduceOp);
HcclResult LocalCopySlices(const ThreadHandle &thread, const std::vector<DataSlice> &srcSlices,
                           const std::vector<DataSlice> &dstSlices);
bool IsContinuousSlice(const DataSlice &nxtSlice, const DataSlice &currSlice);
HcclResult AicpuReduce(const ThreadHandle &thread, const DataSlice &srcSlice, const DataSlice &dstSlice,
                       HcclDataType dataType, HcclReduceOp reduceOp);

HcclResult SendWrite(const DataInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvWrite(const DataInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvWrite(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRead(const DataInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvRead(const DataInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvRead(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRecvWriteReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRecvReadReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);
// one side of a reduce each (the other side only shakes hands)
HcclResult SendWriteReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvWriteReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendReadReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvReadReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread);

HcclResult SendBatchWrite(const DataInfo &sendInfo, const ThreadHandle &thread);
HcclResult SendRecvBatchWrite(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult RecvBatchRead(const DataInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvBatchRead(const SendRecvInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendRecvBatchWriteReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);
HcclResult SendBatchWriteReduce(const DataReduceInfo &sendInfo, const ThreadHandle &thread);
HcclResult RecvBatchReadReduce(const DataReduceInfo &recvInfo, const ThreadHandle &thread);
HcclResult SendRecvBatchReadReduce(const SendRecvReduceInfo &sendRecvInfo, const ThreadHandle &thread);
bool IsHcommBatchTransferOnThreadSupported();

HcclResult PreSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                               const std::vector<u32> &notifyIdxMainToSub);
HcclResult PostSyncInterThreads(const ThreadHandle &mainThread, const std::vector<ThreadHandle> &subThreads,
                                const std::vector<u32> &notifyIdxSubToMain);

}  // namespace ops_hccl
