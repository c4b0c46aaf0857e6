/*
 * hccl_types.h -- scalar types, enums and handles of the HCCL public API, as this library defines them.
 *
 * The reference takes these from HCOMM's <hccl/hccl_types.h> (included at include/hccl.h:14), which is not
 * part of the reference tree.  What the reference tree itself pins, and what this header keeps:
 *   - the order of HcclDataType, through DATATYPE_SIZE_TABLE (src/ops/op_common/inc/alg_param.h:43-45)
 *     and the name table (src/common/hccl_common.h:49-68);
 *   - the HcclReduceOp names sum/prod/max/min (src/common/hccl_common.h:108-114);
 *   - the HcclResult names used on the data path (src/ops/op_common/op_common.cc:2030, :2049, :2103;
 *     src/ops/all_to_all_v/all_to_all_v_op.cc:487-489).
 * The numeric values below follow the published CANN header; a maintainer linking against the real
 * HCOMM header drops this file and keeps everything else.
 */
#ifndef HCCL_AMD_HCCL_TYPES_H_
#define HCCL_AMD_HCCL_TYPES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    HCCL_SUCCESS = 0,
    HCCL_E_PARA = 1,
    HCCL_E_PTR = 2,
    HCCL_E_MEMORY = 3,
    HCCL_E_INTERNAL = 4,
    HCCL_E_NOT_SUPPORT = 5,
    HCCL_E_NOT_FOUND = 6,
    HCCL_E_UNAVAIL = 7,
    HCCL_E_SYSCALL = 8,
    HCCL_E_TIMEOUT = 9,
    HCCL_E_OPEN_FILE_FAILURE = 10,
    HCCL_E_TCP_CONNECT = 11,
    HCCL_E_ROCE_CONNECT = 12,
    HCCL_E_TCP_TRANSFER = 13,
    HCCL_E_ROCE_TRANSFER = 14,
    HCCL_E_RUNTIME = 15,
    HCCL_E_DRV = 16,
    HCCL_E_PROFILING = 17,
    HCCL_E_CCE = 18,
    HCCL_E_NETWORK = 19,
    HCCL_E_AGAIN = 20,
    HCCL_E_REMOTE = 21,
    HCCL_E_SUSPENDING = 22,
    HCCL_E_RESERVED
} HcclResult;

/* Order pinned by DATATYPE_SIZE_TABLE: sizes 1,2,4,2,4,8,8,1,2,4,8,2,16,2,1,1,1,1. */
typedef enum {
    HCCL_DATA_TYPE_INT8 = 0,
    HCCL_DATA_TYPE_INT16 = 1,
    HCCL_DATA_TYPE_INT32 = 2,
    HCCL_DATA_TYPE_FP16 = 3,
    HCCL_DATA_TYPE_FP32 = 4,
    HCCL_DATA_TYPE_INT64 = 5,
    HCCL_DATA_TYPE_UINT64 = 6,
    HCCL_DATA_TYPE_UINT8 = 7,
    HCCL_DATA_TYPE_UINT16 = 8,
    HCCL_DATA_TYPE_UINT32 = 9,
    HCCL_DATA_TYPE_FP64 = 10,
    HCCL_DATA_TYPE_BFP16 = 11,
    HCCL_DATA_TYPE_INT128 = 12,
    HCCL_DATA_TYPE_BF16_SAT = 13,
    HCCL_DATA_TYPE_HIF8 = 14,
    HCCL_DATA_TYPE_FP8E4M3 = 15,
    HCCL_DATA_TYPE_FP8E5M2 = 16,
    HCCL_DATA_TYPE_FP8E8M0 = 17,
    HCCL_DATA_TYPE_RESERVED = 18
} HcclDataType;

typedef enum {
    HCCL_REDUCE_SUM = 0,
    HCCL_REDUCE_PROD = 1,
    HCCL_REDUCE_MAX = 2,
    HCCL_REDUCE_MIN = 3,
    HCCL_REDUCE_RESERVED = 4
} HcclReduceOp;

/* Opaque communicator handle: one per (virtual) rank. */
typedef void *HcclComm;

/* The reference's stream type comes from <acl/acl.h>; on this platform it is a hipStream_t. */
typedef void *aclrtStream;

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_TYPES_H_ */
