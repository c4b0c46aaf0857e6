// Op entry points: parameter checks, OpParam fill, single-rank shortcut, hand-over to the rendezvous.
//
// Check order and error codes follow the reference's op files:
//   HcclAllReduce      src/ops/all_reduce/all_reduce_op.cc:23-56, :106-178
//   HcclReduceScatter  src/ops/reduce_scatter/reduce_scatter_op.cc:23, :180
//   HcclReduceScatterV src/ops/reduce_scatter_v/reduce_scatter_v_op.cc:24-72, :142-167, :169-222
//   HcclAllGather      src/ops/all_gather/all_gather_op.cc:24, :167
//   HcclAllGatherV     src/ops/all_gather_v/all_gather_v_op.cc:22-67, :140-262
//   HcclAlltoAll[V|VC] src/ops/all_to_all_v/all_to_all_v_op.cc:84-142, :385-430, :470-500
//   CheckCount / CheckDataType / CheckReduceOp / SingleRankProc   src/ops/op_common/op_common.cc:2025-2107, :2148-2201
#include <algorithm>
#include <cstring>

#include "hccl.h"
#include "hcclx.h"
#include "schedule.h"
#include "vcomm.h"

using namespace ops_hccl;

namespace {

HcclResult CheckCount(u64 count) { return count > SYS_MAX_COUNT ? HCCL_E_PARA : HCCL_SUCCESS; }

HcclResult CheckDataType(HcclDataType dt, bool needReduce)
{
    if (needReduce) {
        switch (dt) {
            case HCCL_DATA_TYPE_INT8:
            case HCCL_DATA_TYPE_INT16:
            case HCCL_DATA_TYPE_INT32:
            case HCCL_DATA_TYPE_INT64:
            case HCCL_DATA_TYPE_UINT64:
            case HCCL_DATA_TYPE_FP16:
            case HCCL_DATA_TYPE_FP32:
            case HCCL_DATA_TYPE_FP64:
            case HCCL_DATA_TYPE_BFP16:
                return HCCL_SUCCESS;
            default:
                return HCCL_E_NOT_SUPPORT;
        }
    }
    if (dt >= HCCL_DATA_TYPE_RESERVED || dt < HCCL_DATA_TYPE_INT8 || dt == HCCL_DATA_TYPE_INT128) {
        return HCCL_E_NOT_SUPPORT;
    }
    return HCCL_SUCCESS;
}

HcclResult CheckReduceOp(HcclDataType dt, HcclReduceOp op)
{
    if (op < HCCL_REDUCE_SUM || op >= HCCL_REDUCE_RESERVED) return HCCL_E_NOT_SUPPORT;
    if (op == HCCL_REDUCE_PROD) {
        switch (dt) {
            case HCCL_DATA_TYPE_INT8:
            case HCCL_DATA_TYPE_INT32:
            case HCCL_DATA_TYPE_INT64:
            case HCCL_DATA_TYPE_UINT64:
            case HCCL_DATA_TYPE_FP16:
            case HCCL_DATA_TYPE_FP32:
            case HCCL_DATA_TYPE_FP64:
                return HCCL_SUCCESS;
            default:
                return HCCL_E_NOT_SUPPORT;
        }
    }
    return HCCL_SUCCESS;
}

HcclResult CheckBufNullptr(const u64 *counts, u32 rankSize, const void *buf)
{
    for (u32 i = 0; i < rankSize; ++i) {
        if (counts[i] > 0 && buf == nullptr) return HCCL_E_PTR;
    }
    return HCCL_SUCCESS;
}

// One rank: a local copy of `len` bytes unless the op is in place.
HcclResult SingleRankProc(const OpParam &param, u64 len, World *w)
{
    if (param.inputPtr == param.outputPtr || len == 0) return HCCL_SUCCESS;
    if (w->dryRun) return HCCL_SUCCESS;
    hcclx_seg_t s;
    std::memset(&s, 0, sizeof(s));
    s.count = len;
    s.nsrc = 1;
    s.ndst = 1;
    s.src[0] = param.inputPtr;
    s.dst[0] = param.outputPtr;
    return static_cast<HcclResult>(hcclx_fold(&s, 1, HCCL_DATA_TYPE_INT8, 0, HCCLX_FOLD_CHAIN, param.stream));
}

void FillCommon(OpParam &p, RankComm *rc, const char *opName, HcclCMDType type, aclrtStream stream, const void *in,
                const void *out)
{
    p.hcclComm = rc;
    p.tag = std::string(opName) + "_vworld";
    p.stream = stream;
    p.inputPtr = const_cast<void *>(in);
    p.outputPtr = const_cast<void *>(out);
    p.opType = type;
    p.opMode = OpMode::OPBASE;
}

HcclResult AlltoAllCommon(RankComm *rc, OpParam &p, const void *sendBuf, const void *recvBuf, HcclDataType type)
{
    const u32 n = rc->world->rankSize;
    const u64 esz = DATATYPE_SIZE_TABLE[type];
    auto &d = p.all2AllVDataDes;
    d.sendType = type;
    d.recvType = type;
    u64 inElems = 0;
    u64 outElems = 0;
    for (u32 i = 0; i < n; ++i) {
        inElems = std::max(inElems, d.sdispls[i] + d.sendCounts[i]);
        outElems = std::max(outElems, d.rdispls[i] + d.recvCounts[i]);
    }
    p.inputSize = inElems * esz;
    p.outputSize = outElems * esz;
    (void)sendBuf;
    (void)recvBuf;
    if (n == 1) return SingleRankProc(p, d.sendCounts[0] * esz, rc->world);
    return SubmitOp(rc, p);
}

}  // namespace

extern "C" {

// ---- communicators -------------------------------------------------------------------------------
namespace {
// HCCL_BUFFSIZE (MiB) or 200 MiB (test/st/algorithm/utils/inc/sim_common.h:36)
u64 DefaultCclBytes()
{
    u64 ccl = HCCL_CCL_BUFFER_DEFAULT;
    if (const char *mb = std::getenv("HCCL_BUFFSIZE")) {
        const u64 v = std::strtoull(mb, nullptr, 10);
        if (v >= 2) ccl = v * 1024 * 1024;
    }
    return ccl;
}
}  // namespace

HcclResult hcclxCommInitAll(uint32_t nranks, uint64_t cclBytes, int dry, HcclComm *comms)
{
    CHK_PTR_NULL(comms);
    if (cclBytes == 0) cclBytes = DefaultCclBytes();
    if (!dry && hcclx_init() != HCCL_SUCCESS) return HCCL_E_RUNTIME;
    std::vector<HcclComm> v;
    CHK_RET(WorldCreate(nranks, cclBytes, dry != 0, v));
    for (uint32_t i = 0; i < nranks; ++i) comms[i] = v[i];
    return HCCL_SUCCESS;
}

HcclResult HcclCommInitAll(uint32_t ndev, int32_t *devices, HcclComm *comms)
{
    (void)devices;
    return hcclxCommInitAll(ndev, 0, 0, comms);
}

HcclResult HcclCommDestroy(HcclComm comm) { return WorldDestroyRank(comm); }

HcclResult HcclGetRankSize(HcclComm comm, uint32_t *rankSize)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PTR_NULL(rankSize);
    *rankSize = rc->world->rankSize;
    return HCCL_SUCCESS;
}

HcclResult HcclGetRankId(HcclComm comm, uint32_t *rank)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PTR_NULL(rank);
    *rank = rc->rank;
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetExecMode(HcclComm comm, hcclxExecMode mode)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    if (mode != HCCLX_EXEC_FUSED && mode != HCCLX_EXEC_STEP) return HCCL_E_PARA;
    std::lock_guard<std::mutex> lock(rc->world->mu);
    rc->world->mode = (mode == HCCLX_EXEC_STEP) ? ExecMode::STEP : ExecMode::FUSED;
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetBlocking(HcclComm comm, int blocking)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    std::lock_guard<std::mutex> lock(rc->world->mu);
    rc->world->blocking = (blocking != 0);
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetAlgorithm(HcclComm comm, int cmdType, const char *algName)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    SetForcedAlgorithm(rc->world, static_cast<HcclCMDType>(cmdType), algName ? algName : "");
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetTopo(HcclComm comm, uint32_t levels, int level0Shape, uint32_t devicesPerServer)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    if (levels == 0 || level0Shape < 0 || level0Shape > 2) return HCCL_E_PARA;
    SetWorldTopo(rc->world, levels, static_cast<Level0Shape>(level0Shape), devicesPerServer);
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetLinkProtocol(HcclComm comm, int protocol)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    if (protocol < HCCLX_LINK_HCCS || protocol > HCCLX_LINK_PCIE) return HCCL_E_PARA;
    SetWorldLinkProtocol(rc->world, static_cast<CommProtocol>(protocol));
    return HCCL_SUCCESS;
}

HcclResult hcclxCommGetLastOpInfo(HcclComm comm, hcclxLastOpInfo *info)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PTR_NULL(info);
    World *w = rc->world;
    std::lock_guard<std::mutex> lock(w->mu);
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->algName, w->lastAlgName.c_str(), sizeof(info->algName) - 1);
    info->levels = w->lastLevels;
    info->launches = w->lastLaunches;
    info->fusedSegments = w->lastFusedSegments;
    info->fused = w->lastWasFused ? 1 : 0;
    info->planCacheHit = w->lastPlanCacheHit;
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetTrace(HcclComm comm, int on)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    std::lock_guard<std::mutex> lock(rc->world->mu);
    rc->world->traceText = (on != 0);
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetClosedForm(HcclComm comm, int mode)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PRT_RET(mode < 0 || mode > 2, HCCL_ERROR("[hcclxCommSetClosedForm] mode %d is not 0, 1 or 2", mode), HCCL_E_PARA);
    std::lock_guard<std::mutex> lock(rc->world->mu);
    rc->world->closedForm = mode;
    return HCCL_SUCCESS;
}

HcclResult hcclxCommSetCheck(HcclComm comm, int on)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    std::lock_guard<std::mutex> lock(rc->world->mu);
    rc->world->check = (on != 0);
    return HCCL_SUCCESS;
}

HcclResult hcclxCommGetLastCheck(HcclComm comm, hcclxCheckReport *report)
{
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PTR_NULL(report);
    World *w = rc->world;
    std::lock_guard<std::mutex> lock(w->mu);
    const CheckReport &c = w->lastCheck;
    std::memset(report, 0, sizeof(*report));
    report->steps = c.steps;
    report->levels = c.levels;
    report->copies = c.copies;
    report->reduces = c.reduces;
    report->races = c.races;
    report->semanticErrors = c.semanticErrors;
    report->exhaustive = c.exhaustive ? 1 : 0;
    std::strncpy(report->firstProblem, c.firstProblem.c_str(), sizeof(report->firstProblem) - 1);
    return HCCL_SUCCESS;
}

uint64_t hcclxCommGetLastTrace(HcclComm comm, char *buf, uint64_t size)
{
    RankComm *rc = AsRankComm(comm);
    if (rc == nullptr) return 0;
    World *w = rc->world;
    std::lock_guard<std::mutex> lock(w->mu);
    if (buf != nullptr && size > 0) {
        const u64 n = std::min<u64>(size - 1, w->lastTrace.size());
        std::memcpy(buf, w->lastTrace.data(), n);
        buf[n] = 0;
    }
    return w->lastTrace.size();
}

// ---- collectives --------------------------------------------------------------------------------
HcclResult HcclAllReduce(void *sendBuf, void *recvBuf, uint64_t count, HcclDataType dataType, HcclReduceOp op,
                         HcclComm comm, aclrtStream stream)
{
    if (count == 0) return HCCL_SUCCESS;
    CHK_PTR_NULL(stream);
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendBuf);
    CHK_PTR_NULL(recvBuf);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_RET(CheckCount(count));
    CHK_RET(CheckDataType(dataType, true));
    CHK_RET(CheckReduceOp(dataType, op));
    OpParam p;
    FillCommon(p, rc, "AllReduce", HcclCMDType::HCCL_CMD_ALLREDUCE, stream, sendBuf, recvBuf);
    p.inputSize = count * DATATYPE_SIZE_TABLE[dataType];
    p.outputSize = p.inputSize;
    p.reduceType = op;
    p.DataDes.count = count;
    p.DataDes.dataType = dataType;
    if (rc->world->rankSize == 1) return SingleRankProc(p, p.inputSize, rc->world);
    return SubmitOp(rc, p);
}

HcclResult HcclReduceScatter(void *sendBuf, void *recvBuf, uint64_t recvCount, HcclDataType dataType, HcclReduceOp op,
                             HcclComm comm, aclrtStream stream)
{
    if (recvCount == 0) return HCCL_SUCCESS;
    CHK_PTR_NULL(stream);
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendBuf);
    CHK_PTR_NULL(recvBuf);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_RET(CheckCount(recvCount));
    CHK_RET(CheckDataType(dataType, true));
    CHK_RET(CheckReduceOp(dataType, op));
    OpParam p;
    FillCommon(p, rc, "ReduceScatter", HcclCMDType::HCCL_CMD_REDUCE_SCATTER, stream, sendBuf, recvBuf);
    p.outputSize = recvCount * DATATYPE_SIZE_TABLE[dataType];
    p.inputSize = p.outputSize * rc->world->rankSize;
    p.reduceType = op;
    p.DataDes.count = recvCount;
    p.DataDes.dataType = dataType;
    if (rc->world->rankSize == 1) return SingleRankProc(p, p.outputSize, rc->world);
    return SubmitOp(rc, p);
}

HcclResult HcclReduceScatterV(void *sendBuf, const void *sendCounts, const void *sendDispls, void *recvBuf,
                              uint64_t recvCount, HcclDataType dataType, HcclReduceOp op, HcclComm comm,
                              aclrtStream stream)
{
    CHK_PTR_NULL(stream);
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendCounts);
    CHK_PTR_NULL(sendDispls);
    if (recvCount > 0) CHK_PTR_NULL(recvBuf);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    const u32 n = rc->world->rankSize;
    const u64 *counts = static_cast<const u64 *>(sendCounts);
    const u64 *displs = static_cast<const u64 *>(sendDispls);
    if (std::all_of(counts, counts + n, [](u64 c) { return c == 0; })) return HCCL_SUCCESS;
    CHK_RET(CheckCount(recvCount));
    CHK_RET(CheckDataType(dataType, true));
    CHK_RET(CheckReduceOp(dataType, op));
    // The reference trusts these two; here a wrong value would make a kernel read or write out of bounds.
    CHK_PTR_NULL(sendBuf);
    CHK_PRT_RET(counts[rc->rank] != recvCount, HCCL_ERROR("[HcclReduceScatterV] recvCount != sendCounts[rank]"),
                HCCL_E_PARA);
    OpParam p;
    FillCommon(p, rc, "ReduceScatterV", HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V, stream, sendBuf, recvBuf);
    const u64 esz = DATATYPE_SIZE_TABLE[dataType];
    p.reduceType = op;
    p.vDataDes.counts.assign(counts, counts + n);
    p.vDataDes.displs.assign(displs, displs + n);
    p.vDataDes.dataType = dataType;
    p.DataDes.dataType = dataType;
    p.DataDes.count = recvCount;
    u64 inElems = 0;
    for (u32 i = 0; i < n; ++i) inElems = std::max(inElems, displs[i] + counts[i]);
    p.inputSize = inElems * esz;
    p.outputSize = recvCount * esz;
    if (n == 1) return SingleRankProc(p, counts[0] * esz, rc->world);
    return SubmitOp(rc, p);
}

HcclResult HcclAllGather(void *sendBuf, void *recvBuf, uint64_t sendCount, HcclDataType dataType, HcclComm comm,
                         aclrtStream stream)
{
    if (sendCount == 0) return HCCL_SUCCESS;
    CHK_PTR_NULL(stream);
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendBuf);
    CHK_PTR_NULL(recvBuf);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_RET(CheckCount(sendCount));
    CHK_RET(CheckDataType(dataType, false));
    OpParam p;
    FillCommon(p, rc, "AllGather", HcclCMDType::HCCL_CMD_ALLGATHER, stream, sendBuf, recvBuf);
    p.inputSize = sendCount * DATATYPE_SIZE_TABLE[dataType];
    p.outputSize = p.inputSize * rc->world->rankSize;
    p.DataDes.count = sendCount;
    p.DataDes.dataType = dataType;
    if (rc->world->rankSize == 1) return SingleRankProc(p, p.inputSize, rc->world);
    return SubmitOp(rc, p);
}

HcclResult HcclAllGatherV(void *sendBuf, uint64_t sendCount, void *recvBuf, const void *recvCounts,
                          const void *recvDispls, HcclDataType dataType, HcclComm comm, aclrtStream stream)
{
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(recvCounts);
    CHK_PTR_NULL(recvDispls);
    CHK_PTR_NULL(stream);
    if (sendCount > 0) CHK_PTR_NULL(sendBuf);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    const u32 n = rc->world->rankSize;
    const u64 *counts = static_cast<const u64 *>(recvCounts);
    const u64 *displs = static_cast<const u64 *>(recvDispls);
    if (std::all_of(counts, counts + n, [](u64 c) { return c == 0; })) return HCCL_SUCCESS;
    CHK_PTR_NULL(recvBuf);
    CHK_RET(CheckCount(*std::max_element(counts, counts + n)));
    CHK_RET(CheckDataType(dataType, false));
    CHK_PRT_RET(counts[rc->rank] != sendCount, HCCL_ERROR("[HcclAllGatherV] sendCount != recvCounts[rank]"),
                HCCL_E_PARA);
    OpParam p;
    FillCommon(p, rc, "AllGatherV", HcclCMDType::HCCL_CMD_ALLGATHER_V, stream, sendBuf, recvBuf);
    const u64 esz = DATATYPE_SIZE_TABLE[dataType];
    p.vDataDes.counts.assign(counts, counts + n);
    p.vDataDes.displs.assign(displs, displs + n);
    p.vDataDes.dataType = dataType;
    p.DataDes.count = sendCount;
    p.inputSize = sendCount * esz;
    u64 outElems = 0;
    for (u32 i = 0; i < n; ++i) outElems = std::max(outElems, displs[i] + counts[i]);
    p.outputSize = outElems * esz;
    if (n == 1) return SingleRankProc(p, counts[0] * esz, rc->world);
    return SubmitOp(rc, p);
}

HcclResult HcclAlltoAllV(const void *sendBuf, const void *sendCounts, const void *sdispls, HcclDataType sendType,
                         const void *recvBuf, const void *recvCounts, const void *rdispls, HcclDataType recvType,
                         HcclComm comm, aclrtStream stream)
{
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendCounts);
    CHK_PTR_NULL(sdispls);
    CHK_PTR_NULL(recvCounts);
    CHK_PTR_NULL(rdispls);
    CHK_PTR_NULL(stream);
    CHK_PRT_RET(sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf,
                HCCL_ERROR("[HcclAlltoAllV] sendBuf and recvBuf cannot be the same"), HCCL_E_PARA);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    const u32 n = rc->world->rankSize;
    const u64 *sc = static_cast<const u64 *>(sendCounts);
    const u64 *rcv = static_cast<const u64 *>(recvCounts);
    CHK_RET(CheckBufNullptr(sc, n, sendBuf));
    CHK_RET(CheckBufNullptr(rcv, n, recvBuf));
    u64 maxCount = 0;
    for (u32 i = 0; i < n; ++i) maxCount = std::max(maxCount, std::max(sc[i], rcv[i]));
    CHK_RET(CheckCount(maxCount));
    CHK_RET(CheckDataType(recvType, false));
    CHK_PRT_RET(sendType != recvType, HCCL_ERROR("[HcclAlltoAllV] sendType != recvType"), HCCL_E_PARA);
    OpParam p;
    FillCommon(p, rc, "ALLTOALLV", HcclCMDType::HCCL_CMD_ALLTOALLV, stream, sendBuf, recvBuf);
    p.all2AllVDataDes.sendCounts.assign(sc, sc + n);
    p.all2AllVDataDes.recvCounts.assign(rcv, rcv + n);
    p.all2AllVDataDes.sdispls.assign(static_cast<const u64 *>(sdispls), static_cast<const u64 *>(sdispls) + n);
    p.all2AllVDataDes.rdispls.assign(static_cast<const u64 *>(rdispls), static_cast<const u64 *>(rdispls) + n);
    return AlltoAllCommon(rc, p, sendBuf, recvBuf, recvType);
}

HcclResult HcclAlltoAll(const void *sendBuf, uint64_t sendCount, HcclDataType sendType, const void *recvBuf,
                        uint64_t recvCount, HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(stream);
    if (sendCount == 0 && recvCount == 0) return HCCL_SUCCESS;
    CHK_PTR_NULL(sendBuf);
    CHK_PTR_NULL(recvBuf);
    CHK_PRT_RET(sendBuf == recvBuf, HCCL_ERROR("[HcclAlltoAll] sendBuf and recvBuf cannot be the same"), HCCL_E_PARA);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    CHK_PRT_RET(sendCount != recvCount || sendType != recvType,
                HCCL_ERROR("[HcclAlltoAll] send and receive count / type differ"), HCCL_E_PARA);
    CHK_RET(CheckCount(sendCount));
    CHK_RET(CheckDataType(recvType, false));
    const u32 n = rc->world->rankSize;
    OpParam p;
    FillCommon(p, rc, "ALLTOALL", HcclCMDType::HCCL_CMD_ALLTOALL, stream, sendBuf, recvBuf);
    p.all2AllDataDes.sendCount = sendCount;
    p.all2AllDataDes.recvCount = recvCount;
    auto &d = p.all2AllVDataDes;
    d.sendCounts.assign(n, sendCount);
    d.recvCounts.assign(n, recvCount);
    d.sdispls.resize(n);
    d.rdispls.resize(n);
    u64 off = 0;  // ConvertAlltoAllParam, all_to_all_v_op.cc:385-394
    for (u32 i = 0; i < n; ++i) {
        d.sdispls[i] = off;
        d.rdispls[i] = off;
        off += recvCount;
    }
    return AlltoAllCommon(rc, p, sendBuf, recvBuf, recvType);
}

HcclResult HcclAlltoAllVC(const void *sendBuf, const void *sendCountMatrix, HcclDataType sendType, const void *recvBuf,
                          HcclDataType recvType, HcclComm comm, aclrtStream stream)
{
    CHK_PTR_NULL(comm);
    CHK_PTR_NULL(sendCountMatrix);
    CHK_PTR_NULL(stream);
    CHK_PRT_RET(sendBuf != nullptr && recvBuf != nullptr && sendBuf == recvBuf,
                HCCL_ERROR("[HcclAlltoAllVC] sendBuf and recvBuf cannot be the same"), HCCL_E_PARA);
    RankComm *rc = AsRankComm(comm);
    CHK_PTR_NULL(rc);
    const u32 n = rc->world->rankSize;
    const u64 *m = static_cast<const u64 *>(sendCountMatrix);
    CHK_RET(CheckCount(*std::max_element(m, m + static_cast<size_t>(n) * n)));
    CHK_RET(CheckDataType(recvType, false));
    CHK_PRT_RET(sendType != recvType, HCCL_ERROR("[HcclAlltoAllVC] sendType != recvType"), HCCL_E_PARA);
    OpParam p;
    FillCommon(p, rc, "ALLTOALLVC", HcclCMDType::HCCL_CMD_ALLTOALLVC, stream, sendBuf, recvBuf);
    auto &d = p.all2AllVDataDes;
    d.sendCounts.resize(n);
    d.recvCounts.resize(n);
    d.sdispls.resize(n);
    d.rdispls.resize(n);
    u64 off = 0;  // ConvertAlltoAllVCParam, all_to_all_v_op.cc:396-430: my row is what I send ...
    for (u32 i = 0; i < n; ++i) {
        d.sendCounts[i] = m[static_cast<size_t>(rc->rank) * n + i];
        d.sdispls[i] = off;
        off += d.sendCounts[i];
    }
    off = 0;  // ... my column is what I receive
    for (u32 i = 0; i < n; ++i) {
        d.recvCounts[i] = m[static_cast<size_t>(i) * n + rc->rank];
        d.rdispls[i] = off;
        off += d.recvCounts[i];
    }
    CHK_RET(CheckBufNullptr(d.sendCounts.data(), n, sendBuf));
    CHK_RET(CheckBufNullptr(d.recvCounts.data(), n, recvBuf));
    return AlltoAllCommon(rc, p, sendBuf, recvBuf, recvType);
}

}  // extern "C"
