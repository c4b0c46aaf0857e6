/*
 * hcomm_primitives.h -- the data-plane primitive ABI the algorithm templates call.
 *
 * In the reference these symbols come from libhcomm.so, loaded with dlopen/dlsym
 * (src/common/hcomm_dlsym/hcomm_dlsym.cc:62-82); their signatures are visible in the system-test stubs
 * (test/st/algorithm/utils/src/hccl_proxy/hccl_stub.cc, line given per function).  Here they are the
 * entry of the virtual-rank backend: every call is recorded on its thread; when all ranks of the
 * communicator have issued their collective, the recorded steps are ordered by their notify
 * dependencies and launched as HIP kernels over buffers that all live in one GPU's HBM.
 * Return value: 0 = success, otherwise an HcclResult.
 */
#ifndef HCCL_AMD_HCOMM_PRIMITIVES_H_
#define HCCL_AMD_HCOMM_PRIMITIVES_H_

#include <stdint.h>
#include "hccl_types.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t ThreadHandle;   /* sim_common.h:40 */
typedef uint64_t ChannelHandle;  /* sim_common.h:41 */
typedef HcclDataType HcommDataType;
typedef HcclReduceOp HcommReduceOp;

/* dst[0..len) = src[0..len), both local to the calling rank.            hccl_stub.cc:467 */
int32_t HcommLocalCopyOnThread(ThreadHandle thread, void *dst, const void *src, uint64_t len);
/* dst[i] = src[i] (+) dst[i] for count elements.                        hccl_stub.cc:633 */
int32_t HcommLocalReduceOnThread(ThreadHandle thread, void *dst, const void *src, uint64_t count,
                                 HcommDataType dataType, HcommReduceOp reduceOp);
/* Write local src into the peer's dst / read the peer's src into local dst.   hccl_stub.cc:495, :534 */
int32_t HcommWriteOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src, uint64_t len);
int32_t HcommReadOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src, uint64_t len);
/* The same with dst = src (+) dst at the destination.                   hccl_stub.cc:664, :705 */
int32_t HcommWriteReduceOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                 uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp);
int32_t HcommReadReduceOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp);
/* Inter-rank handshake over a channel.                                  hccl_stub.cc:573, :601 */
int32_t HcommChannelNotifyRecordOnThread(ThreadHandle thread, ChannelHandle channel, uint32_t remoteNotifyIdx);
int32_t HcommChannelNotifyWaitOnThread(ThreadHandle thread, ChannelHandle channel, uint32_t localNotifyIdx,
                                       uint32_t timeout);
/* Main thread <-> sub thread fan-out / fan-in inside one rank.          hccl_stub.cc:449, :397 */
int32_t HcommThreadNotifyRecordOnThread(ThreadHandle thread, ThreadHandle dstThread, uint32_t dstNotifyIdx);
int32_t HcommThreadNotifyWaitOnThread(ThreadHandle thread, uint32_t notifyIdx, uint32_t timeout);
/* The process-wide time-outs and the waits that use them.  Every wait of the reference's wrapper goes through the
 * *WithDefaultTimeout form first and only falls back to the form with an explicit time-out when libhcomm does not
 * export it (src/common/hcomm_dlsym/hcomm_primitives_dl.h:95-102, hcomm_primitives_dl.cc:131-173;
 * src/ops/op_common/template/wrapper/alg_data_trans_wrapper.cc:22-31).  Recorded waits have no clock: the values
 * are kept and returned as success. */
int32_t HcommSetNotifyWaitTimeOut(uint32_t timeOut);
int32_t HcommThreadResAcquireTimeOut(uint32_t timeOut);
int32_t HcommThreadNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, uint32_t notifyIdx);
int32_t HcommChannelNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, ChannelHandle channel,
                                                         uint32_t localNotifyIdx);
/* A write followed by the record of remoteNotifyIdx on the same channel, and a fence that orders the transfers
 * issued on a channel so far before the later ones (hcomm_primitives_dl.h:103-105).  Steps of one thread are
 * recorded in program order, so the fence only checks its handles. */
int32_t HcommWriteWithNotifyNbiOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                        uint64_t len, uint32_t remoteNotifyIdx);
int32_t HcommChannelFenceOnThread(ThreadHandle thread, ChannelHandle channel);
/* Several transfers and handshakes on one channel in one call: what every *Batch* verb of the wrapper issues first
 * (src/ops/op_common/template/wrapper/alg_data_trans_wrapper.cc:99-125) and falls back from, slice by slice, when
 * libhcomm does not export it.  The reference resolves the symbol by this name
 * (src/common/hcomm_dlsym/hcomm_primitives_dl.cc:115-116); the descriptor is its ABI-compatible mirror
 * (src/common/hcomm_dlsym/hcomm_primitives_dl.h:26-79).  Descriptors are carried out in array order: WRITE / READ
 * copy `len` bytes, the *_REDUCE kinds do dst = src (+) dst on `count` elements, NOTIFY_RECORD / NOTIFY_WAIT are the
 * channel handshakes, and the *_WITH_NOTIFY kinds record the notify after their transfer. */
typedef enum {
    HCCL_HCOMM_TRANSFER_TYPE_INVALID = -1,
    HCCL_HCOMM_TRANSFER_TYPE_WRITE = 0,
    HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE = 1,
    HCCL_HCOMM_TRANSFER_TYPE_WRITE_WITH_NOTIFY = 2,
    HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE_WITH_NOTIFY = 3,
    HCCL_HCOMM_TRANSFER_TYPE_READ = 4,
    HCCL_HCOMM_TRANSFER_TYPE_READ_REDUCE = 5,
    HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_RECORD = 6,
    HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_WAIT = 7,
    HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_WAIT_WITH_DEFAULT_TIMEOUT = 8
} HcclHcommTransferType;

typedef struct {
    HcclHcommTransferType transType;
    uint8_t reserved[4];
    union {
        uint8_t raws[56];
        struct { uint64_t len; void *dst; void *src; } write;
        struct { uint64_t len; void *dst; void *src; } read;
        struct { uint64_t count; void *dst; void *src; HcommReduceOp reduceOp; HcommDataType dataType; } reduce;
        struct { uint32_t notifyIdx; } notifyRecord;
        struct { uint64_t len; void *dst; void *src; uint32_t notifyIdx; } writeWithNotify;
        struct { uint64_t count; void *dst; void *src; HcommReduceOp reduceOp; HcommDataType dataType;
                 uint32_t notifyIdx; } writeReduceWithNotify;
    } transferInfo;
} HcclHcommBatchTransferDesc;

int32_t HcommBatchTransferOnThread(ThreadHandle thread, ChannelHandle channel,
                                   const HcclHcommBatchTransferDesc *transferDescs, uint32_t transferDescNum);

/* Flush / join before CPU-side work.  Stream order already gives that here.   hccl_stub.cc:799, :805, :937 */
int32_t HcommBatchModeStart(const char *batchTag);
int32_t HcommBatchModeEnd(const char *batchTag);
int32_t HcommThreadJoin(ThreadHandle thread, uint32_t timeout);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCOMM_PRIMITIVES_H_ */
