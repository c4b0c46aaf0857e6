/*
 * hccl.h -- the collective entry points of HCCL that this library implements, with the reference's
 * signatures kept as they are (reference include/hccl.h; line of each prototype given below).
 *
 * All ranks of a communicator are virtual ranks inside one GPU: their send and receive buffers are device
 * pointers in the same HBM.  A call queues the rank's part of the collective; the collective is launched
 * on the GPU when the last rank of the communicator has made its call (see hccl_comm.h).  Count and
 * displacement arrays are host arrays of uint64_t, in elements, and only need to outlive the call.
 *
 * Return value: HCCL_SUCCESS or the first failing check, as in the reference:
 *   HCCL_E_PTR          a required pointer (comm, stream, buffers, count arrays) is null
 *   HCCL_E_PARA         count above 0x7FFFFFFFF, sendBuf == recvBuf for AlltoAllV, ranks disagreeing
 *   HCCL_E_NOT_SUPPORT  data type / reduce op not supported for the op
 * Early success: count == 0, all recvCounts == 0; a one-rank communicator does one local copy.
 */
#ifndef HCCL_AMD_HCCL_H_
#define HCCL_AMD_HCCL_H_

#include "hccl_types.h"
#include "hccl_comm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* reference include/hccl.h:35-36.  dataType: int8 int16 int32 int64 uint64 fp16 fp32 fp64 bf16; op: sum prod max min
 * (prod not for int16 / bf16). */
extern HcclResult HcclAllReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:66-67.  sendBuf holds rankSize * recvCount elements. */
extern HcclResult HcclReduceScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType,
    HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:85-86.  Ragged ReduceScatter: rank r receives the reduction of every rank's
 * sendBuf[sendDispls[r] .. +sendCounts[r]); recvCount == sendCounts[own rank].  sendCounts / sendDispls are
 * host uint64_t[rankSize] in elements, the same on every rank. */
extern HcclResult HcclReduceScatterV(void *sendBuf, const void *sendCounts, const void *sendDispls,
    void *recvBuf, uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:116-117.  recvBuf holds rankSize * sendCount elements. */
extern HcclResult HcclAllGather(void *sendBuf, void *recvBuf, uint64_t sendCount, HcclDataType dataType,
    HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:134-135.  recvBuf[recvDispls[i] .. +recvCounts[i]) = rank i's sendBuf. */
extern HcclResult HcclAllGatherV(void *sendBuf, uint64_t sendCount, void *recvBuf,
    const void *recvCounts, const void *recvDispls, HcclDataType dataType, HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:180-181.  sendCountMatrix: rankSize x rankSize, row i = what rank i sends. */
extern HcclResult HcclAlltoAllVC(const void *sendBuf, const void *sendCountMatrix, HcclDataType sendType,
                                 const void *recvBuf, HcclDataType recvType, HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:202-204. */
extern HcclResult HcclAlltoAllV(const void *sendBuf, const void *sendCounts, const void *sdispls, HcclDataType sendType,
                         const void *recvBuf, const void *recvCounts, const void *rdispls, HcclDataType recvType,
                         HcclComm comm, aclrtStream stream);

/* reference include/hccl.h:221-223. */
extern HcclResult HcclAlltoAll(const void *sendBuf, uint64_t sendCount, HcclDataType sendType,
                               const void *recvBuf, uint64_t recvCount, HcclDataType recvType,
                               HcclComm comm, aclrtStream stream);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_H_ */
