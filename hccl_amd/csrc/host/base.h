// Scalar types, enums, constants and error macros of the host runtime.
//
// Names follow the reference so that its selector / executor / template code reads the same here:
//   HcclCMDType, CommEngine, BufferType, DATATYPE_SIZE_TABLE   src/ops/op_common/inc/alg_param.h:43-45, :102-113
//   SYS_MAX_COUNT                                              src/common/hccl_common.h:42
//   HCCL_MIN_SLICE_ALIGN                                       src/ops/op_common/template/alg_template_base.h:35
//   UB_MAX_DATA_SIZE                                           src/ops/op_common/inc/alg_param.h:37
#pragma once
#include <stdint.h>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "hccl_types.h"

namespace ops_hccl {

using u8 = uint8_t;
using u16 = uint16_t;
using u32 = uint32_t;
using u64 = uint64_t;
using s32 = int32_t;
using s64 = int64_t;

using ThreadHandle = uint64_t;   // test/st/algorithm/utils/inc/sim_common.h:40-41
using ChannelHandle = uint64_t;

constexpr u32 INVALID_VALUE_RANKID = 0xFFFFFFFFu;
constexpr u64 SYS_MAX_COUNT = 0x7FFFFFFFFull;
constexpr u64 HCCL_MIN_SLICE_ALIGN = 128;
constexpr u64 UB_MAX_DATA_SIZE = 256ull * 1024 * 1024;
constexpr u64 AICPU_ALIGN_SIZE = 4096;   // src/ops/op_common/inc/alg_param.h:75
constexpr u64 HCCL_CCL_BUFFER_DEFAULT = 200ull * 1024 * 1024;  // HCCL_BUFFSIZE default, 200 MiB in the ST harness
constexpr u32 NOTIFY_IDX_ACK = 0;
constexpr u32 NOTIFY_IDX_DATA_SIGNAL = 1;
constexpr u32 CUSTOM_TIMEOUT = 1836;
constexpr u32 SELECTOR_PRIORITY_BUILTIN = 18;  // priority of the built-in selectors

constexpr u32 DATATYPE_SIZE_TABLE[HCCL_DATA_TYPE_RESERVED] = {1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1};

enum class HcclCMDType : int {
    HCCL_CMD_INVALID = 0,
    HCCL_CMD_BROADCAST = 1,
    HCCL_CMD_ALLREDUCE = 2,
    HCCL_CMD_REDUCE = 3,
    HCCL_CMD_SEND = 4,
    HCCL_CMD_RECEIVE = 5,
    HCCL_CMD_ALLGATHER = 6,
    HCCL_CMD_REDUCE_SCATTER = 7,
    HCCL_CMD_ALLTOALLV = 8,
    HCCL_CMD_ALLTOALLVC = 9,
    HCCL_CMD_ALLTOALL = 10,
    HCCL_CMD_GATHER = 11,
    HCCL_CMD_SCATTER = 12,
    HCCL_CMD_BATCH_SEND_RECV = 13,
    HCCL_CMD_ALLGATHER_V = 16,
    HCCL_CMD_REDUCE_SCATTER_V = 17,
};

enum class BufferType { INPUT = 0, OUTPUT = 1, HCCL_BUFFER = 2, DEFAULT };

// Only the AICPU engine's branch of the reference is built; its "device" is the virtual-rank backend.
enum class CommEngine { COMM_ENGINE_AICPU_TS = 0, COMM_ENGINE_RESERVED };

enum class OpMode { OFFLOAD = 0, OPBASE = 1 };

enum class Level0Shape { CLOS = 0, MESH_1D = 1, MESH_1D_CLOS = 2 };

inline bool LogEnabled()
{
    static const bool on = (std::getenv("HCCL_DEBUG_LOG") != nullptr);
    return on;
}

#define HCCL_ERROR(fmt, ...)                                                        \
    do {                                                                            \
        if (::ops_hccl::LogEnabled()) std::fprintf(stderr, "[HCCL][ERROR] " fmt "\n", ##__VA_ARGS__); \
    } while (0)
#define HCCL_WARNING(fmt, ...)                                                      \
    do {                                                                            \
        if (::ops_hccl::LogEnabled()) std::fprintf(stderr, "[HCCL][WARN] " fmt "\n", ##__VA_ARGS__);  \
    } while (0)
#define HCCL_INFO(fmt, ...) \
    do {                    \
    } while (0)

// First failing check returns, as the reference's CHK_RET does.
#define CHK_RET(call)                                  \
    do {                                               \
        HcclResult ret_ = static_cast<HcclResult>(call); \
        if (ret_ != HCCL_SUCCESS) return ret_;         \
    } while (0)

#define CHK_PRT_RET(cond, log, ret) \
    do {                            \
        if (cond) {                 \
            log;                    \
            return ret;             \
        }                           \
    } while (0)

#define CHK_PTR_NULL(p)                     \
    do {                                    \
        if ((p) == nullptr) return HCCL_E_PTR; \
    } while (0)

inline u64 RoundUp(const u64 dividend, const u64 divisor)
{
    // src/ops/op_common/template/template_utils.h:449-456
    if (divisor == 0) return dividend;
    return dividend / divisor + ((dividend % divisor != 0) ? 1 : 0);
}

}  // namespace ops_hccl
