#include "schedule.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <sstream>
#include <unordered_map>

#include "executor.h"
#include "hcclx.h"
#include "schedule_internal.h"
#include "selector.h"

namespace ops_hccl {

void SetForcedAlgorithm(World *w, HcclCMDType type, const std::string &algName)
{
    std::lock_guard<std::mutex> lock(w->mu);
    w->forcedAlg[static_cast<int>(type)] = algName;
}

std::string GetForcedAlgorithm(World *w, HcclCMDType type)
{
    auto it = w->forcedAlg.find(static_cast<int>(type));
    return it == w->forcedAlg.end() ? std::string() : it->second;
}

void SetWorldTopo(World *w, u32 levels, Level0Shape shape, u32 devicesPerServer)
{
    std::lock_guard<std::mutex> lock(w->mu);
    w->topoLevels = levels;
    w->topoShape = shape;
    w->devicesPerServer = devicesPerServer;
}

void SetWorldLinkProtocol(World *w, CommProtocol protocol)
{
    std::lock_guard<std::mutex> lock(w->mu);
    w->linkProtocol = protocol;
}

using namespace sched;

namespace {

bool SameOperands(const OpParam &a, const OpParam &b)
{
    if (a.opType != b.opType) return false;
    switch (a.opType) {
        case HcclCMDType::HCCL_CMD_ALLREDUCE:
        case HcclCMDType::HCCL_CMD_REDUCE_SCATTER:
            return a.DataDes.count == b.DataDes.count && a.DataDes.dataType == b.DataDes.dataType &&
                   a.reduceType == b.reduceType;
        case HcclCMDType::HCCL_CMD_ALLGATHER:
            return a.DataDes.count == b.DataDes.count && a.DataDes.dataType == b.DataDes.dataType;
        case HcclCMDType::HCCL_CMD_ALLGATHER_V:
            return a.vDataDes.dataType == b.vDataDes.dataType && a.vDataDes.counts == b.vDataDes.counts &&
                   a.vDataDes.displs == b.vDataDes.displs;
        case HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V:
            return a.vDataDes.dataType == b.vDataDes.dataType && a.vDataDes.counts == b.vDataDes.counts &&
                   a.vDataDes.displs == b.vDataDes.displs && a.reduceType == b.reduceType;
        default:
            return a.all2AllVDataDes.sendType == b.all2AllVDataDes.sendType;
    }
}

bool IsDataMove(HcclCMDType t)
{
    return t == HcclCMDType::HCCL_CMD_ALLGATHER || t == HcclCMDType::HCCL_CMD_ALLGATHER_V ||
           t == HcclCMDType::HCCL_CMD_ALLTOALL || t == HcclCMDType::HCCL_CMD_ALLTOALLV ||
           t == HcclCMDType::HCCL_CMD_ALLTOALLVC;
}

// Pure data movement has no fold order to preserve: in FUSED mode the contract itself is launched on the
// ragged-copy kernels (one read and one write per delivered byte), with the tables of all ranks.
HcclResult LaunchDataMove(World *w, const std::vector<OpParam> &params, void *stream)
{
    const u32 n = w->rankSize;
    std::vector<const void *> send(n);
    std::vector<void *> recv(n);
    for (u32 r = 0; r < n; ++r) {
        send[r] = params[r].inputPtr;
        recv[r] = params[r].outputPtr;
    }
    const HcclCMDType t = params[0].opType;
    if (t == HcclCMDType::HCCL_CMD_ALLGATHER || t == HcclCMDType::HCCL_CMD_ALLGATHER_V) {
        std::vector<u64> counts(n);
        std::vector<u64> displs(n);
        for (u32 r = 0; r < n; ++r) {
            if (t == HcclCMDType::HCCL_CMD_ALLGATHER) {
                counts[r] = params[0].DataDes.count;
                displs[r] = r * params[0].DataDes.count;
            } else {
                counts[r] = params[0].vDataDes.counts[r];
                displs[r] = params[0].vDataDes.displs[r];
            }
        }
        const int dt = (t == HcclCMDType::HCCL_CMD_ALLGATHER) ? params[0].DataDes.dataType : params[0].vDataDes.dataType;
        return static_cast<HcclResult>(
            hcclx_allgatherv(send.data(), recv.data(), counts.data(), displs.data(), n, dt, 0, stream));
    }
    std::vector<u64> sc(static_cast<size_t>(n) * n);
    std::vector<u64> sd(static_cast<size_t>(n) * n);
    std::vector<u64> rd(static_cast<size_t>(n) * n);
    for (u32 i = 0; i < n; ++i) {
        for (u32 j = 0; j < n; ++j) {
            sc[i * n + j] = params[i].all2AllVDataDes.sendCounts[j];
            sd[i * n + j] = params[i].all2AllVDataDes.sdispls[j];
            rd[i * n + j] = params[i].all2AllVDataDes.rdispls[j];
        }
    }
    return static_cast<HcclResult>(hcclx_alltoallv(send.data(), recv.data(), sc.data(), sd.data(), rd.data(), n,
                                                   params[0].all2AllVDataDes.sendType, 0, stream));
}

}  // namespace

namespace {
HcclResult RunCollectiveOnStream(World *w, std::vector<OpParam> &params);

// Ranks may pass different streams.  The collective runs on the stream of the last rank; it first waits
// for everything the other ranks' streams hold so far (their inputs), and those streams then wait for it.
HcclResult JoinStreams(const std::vector<OpParam> &params, hipStream_t launch, bool before)
{
    std::vector<hipStream_t> others;
    for (const OpParam &p : params) {
        hipStream_t s = static_cast<hipStream_t>(p.stream);
        if (s != launch && std::find(others.begin(), others.end(), s) == others.end()) others.push_back(s);
    }
    for (hipStream_t s : others) {
        hipEvent_t ev;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) return HCCL_E_RUNTIME;
        const hipError_t e1 = hipEventRecord(ev, before ? s : launch);
        const hipError_t e2 = hipStreamWaitEvent(before ? launch : s, ev, 0);
        (void)hipEventDestroy(ev);  // released once the recorded work has passed it
        if (e1 != hipSuccess || e2 != hipSuccess) return HCCL_E_RUNTIME;
    }
    return HCCL_SUCCESS;
}
}  // namespace

HcclResult RunCollective(World *w, std::vector<OpParam> &params)
{
    if (w->dryRun) {
        w->lastLaunches = 0;
        return RunCollectiveOnStream(w, params);
    }
    hipStream_t launch = static_cast<hipStream_t>(params[w->rankSize - 1].stream);
    CHK_RET(JoinStreams(params, launch, true));
    // everything a collective launches is launched by this host thread: the kernels it took are the difference
    // of the library's per-thread count (a fold whose result fans out is two, a large ragged gather several)
    const uint64_t kernelsBefore = hcclx_kernels_launched();
    const HcclResult res = RunCollectiveOnStream(w, params);
    w->lastLaunches = static_cast<u32>(hcclx_kernels_launched() - kernelsBefore);
    CHK_RET(JoinStreams(params, launch, false));
    return res;
}

namespace {
HcclResult RunCollectiveOnStream(World *w, std::vector<OpParam> &params)
{
    const u32 n = w->rankSize;
    // every rank must have issued the same collective with the same operands
    for (u32 r = 1; r < n; ++r) {
        CHK_PRT_RET(!SameOperands(params[0], params[r]),
                    HCCL_ERROR("[RunCollective] rank %u issued a different collective than rank 0", r), HCCL_E_PARA);
    }
    const HcclCMDType type = params[0].opType;
    if (IsDataMove(type)) {
        // what i sends to j must be what j expects from i
        for (u32 i = 0; i < n && type != HcclCMDType::HCCL_CMD_ALLGATHER && type != HcclCMDType::HCCL_CMD_ALLGATHER_V;
             ++i) {
            for (u32 j = 0; j < n; ++j) {
                CHK_PRT_RET(params[i].all2AllVDataDes.sendCounts[j] != params[j].all2AllVDataDes.recvCounts[i],
                            HCCL_ERROR("[RunCollective] sendCounts[%u][%u] != recvCounts[%u][%u]", i, j, j, i),
                            HCCL_E_PARA);
            }
        }
    }

    // algorithm: forced for this world, asked for by HCCL_ALGO, or the selector's choice
    std::string algName = GetForcedAlgorithm(w, type);
    if (algName.empty()) {
        const HcclDataType dt = params[0].DataDes.dataType;
        const bool cpuReduce = dt == HCCL_DATA_TYPE_INT64 || dt == HCCL_DATA_TYPE_UINT64 || dt == HCCL_DATA_TYPE_FP64 ||
                               params[0].reduceType == HCCL_REDUCE_PROD;
        algName = AlgNameFromConfig(w->algoConfig, type, cpuReduce);
    }
    if (algName.empty()) {
        TopoInfoWithNetLayerDetails topo;
        topo.userRankSize = n;
        topo.topoLevelNums = w->topoLevels;
        topo.level0Topo = w->topoShape;
        topo.localNetInsSizeOfLayer0 = w->devicesPerServer ? w->devicesPerServer : n;
        CHK_RET(ExecuteSelector().Run(params[0], &topo, algName));
    }
    w->lastAlgName = algName;
    w->lastWasFused = false;
    w->lastPlanCacheHit = 0;
    w->lastFusedSegments = 0;
    w->lastLevels = 0;
    void *stream = params[n - 1].stream;

    const int dtype = params[0].DataDes.dataType;
    const int op = params[0].reduceType;
    const bool fused = (w->mode == ExecMode::FUSED);
    if (fused && !w->dryRun && !w->traceText && !w->check && IsDataMove(type)) {
        w->lastWasFused = true;
        return LaunchDataMove(w, params, stream);
    }
    std::vector<u64> shape;
    std::vector<u64> key;
    bool separate = false;
    if (!w->dryRun && !w->traceText && !w->check) {
        PlanCache &cache = w->planCache;
        shape = ShapeKey(params, algName, w->cclBytes);
        shape.push_back(fused ? 1 : 0);
        shape.push_back(static_cast<u64>(w->linkProtocol));   // read and write mode record different steps
        key = PlanKey(shape, params);
        if (!cache.retired.empty()) ReapRetired(cache, false);
        if (CachedPlan *c = FindPlan(cache, key)) {
            if (c->lastStream != stream) c->manyStreams = true;
            c->lastStream = stream;
            w->lastWasFused = c->fused;
            w->lastLevels = c->levels;
            w->lastFusedSegments = c->segments;
            w->lastPlanCacheHit = 1;
            return LaunchPlans(w, c->plans, stream);
        }
        // Everything below allocates tables or sends them through the pinned ring: none of it may be recorded into
        // a graph (the graph would replay a copy from a ring slot that has long been reused).
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) == hipSuccess &&
            capturing != hipStreamCaptureStatusNone) {
            HCCL_ERROR("[RunCollective] %s on a capturing stream has no plan for these buffers yet: run the same "
                       "collective on the same buffers once before the capture", algName.c_str());
            return HCCL_E_NOT_SUPPORT;
        }
        separate = BuffersAreSeparate(params);
        if (ShapePlan *sp = separate ? FindShape(cache, shape) : nullptr) {
            // The same collective on other buffers: the plan it had, with every pointer moved along with its buffer.
            std::vector<HostPart> parts;
            Rebase(*sp, params, parts);
            w->lastWasFused = sp->fused;
            w->lastLevels = sp->levels;
            w->lastFusedSegments = sp->segments;
            w->lastPlanCacheHit = 2;
            // Small plans go through the descriptor ring (no allocation).  Beyond the size the runtime copies inline,
            // a table of the plan's own, uploaded on the library's stream, is cheaper than a copy queued on the
            // caller's (16-rank mesh-chunk, 72 KB: 50 against 146 us; 32-rank, 1.1 MB: 0.25 against 0.85 ms), and
            // buffers that have come by before are worth their own tables anyway.
            constexpr u64 kThroughTheRingUpTo = 16 * 1024;
            if (!SeenBefore(cache, HashKey(key)) && sp->hostBytes <= kThroughTheRingUpTo) return LaunchParts(w, parts, stream);
            CachedPlan c;
            c.key = key;
            c.fused = sp->fused;
            c.levels = sp->levels;
            c.segments = sp->segments;
            const HcclResult made = CreatePlans(parts, c.plans);
            if (made != HCCL_SUCCESS) {
                DropPlans(c.plans, c.buffers);
                return made;
            }
            return LaunchAndKeep(w, std::move(c), stream);
        }
    }

    // expand: every rank's executor + template records its steps
    g_phase.Start();
    auto lap = [](const char *what) { g_phase.Lap(what); };
    // A fused pass never touches the scratch buffers (their addresses only name intermediate values while the
    // schedule is traced), so they stand for themselves as address ranges until a schedule has to run step by step.
    std::vector<Node> order;
    u32 numLevels = 0;
    bool recordedOnMemory = false;
    auto expand = [&](bool scratchMemory) -> HcclResult {
        CHK_RET(w->EnsureScratch(scratchMemory));
        recordedOnMemory = w->scratchIsMemory;
        lap("scratch");
        w->ResetRecording();
        for (u32 r = 0; r < n; ++r) {
            params[r].algName = algName;
            std::unique_ptr<InsCollAlgBase> exec = CollAlgExecRegistryV2::Instance().GetAlgExec(type, algName);
            CHK_PRT_RET(exec == nullptr, HCCL_ERROR("[RunCollective] no executor named %s", algName.c_str()),
                        HCCL_E_NOT_SUPPORT);
            AlgResourceCtxSerializable resCtx;
            const u64 threadNum = exec->CalcThreadNum(params[r], r, n);
            FillResources(w, r, static_cast<u32>(threadNum), resCtx);
            CHK_RET(exec->Orchestrate(params[r], resCtx));
        }
        lap("record");
        CHK_RET(BuildOrder(w, order, numLevels, w->check ? &w->lastCheck : nullptr));
        w->lastLevels = numLevels;
        if (g_phase.on) {
            size_t items = 0;
            for (auto &perRank : w->threads) {
                for (auto &t : perRank) items += t->items.size();
            }
            std::fprintf(stderr, "[timing] %zu recorded items, %zu data steps, %u levels\n", items, order.size(), numLevels);
        }
        lap("order");
        return HCCL_SUCCESS;
    };
    const u32 esz = IsDataMove(type) ? 1 : DATATYPE_SIZE_TABLE[dtype];
    const int foldType = IsDataMove(type) ? HCCL_DATA_TYPE_INT8 : dtype;
    std::string *text = (w->traceText || w->dryRun) ? &w->lastTrace : nullptr;
    w->lastTrace.clear();
    w->lastCheck = CheckReport();

    // A template whose steps grow with the cube of the rank count may state its result in closed form: then nothing
    // is recorded, ordered or traced.  Only among buffers that lie apart (what the steps amount to does not depend
    // on where they are then), and never when the schedule itself is to be checked.
    std::vector<Fold> folds;
    bool haveFolds = false;
    const bool plain = !w->dryRun && !w->traceText && !w->check;
    if ((fused || w->dryRun || w->traceText) && !w->check && !IsDataMove(type) &&
        (w->closedForm == 2 || (w->closedForm == 1 && plain)) && (plain ? separate : BuffersAreSeparate(params))) {
        std::unique_ptr<InsCollAlgBase> exec = CollAlgExecRegistryV2::Instance().GetAlgExec(type, algName);
        std::vector<ClosedFold> closed;
        params[0].algName = algName;
        if (exec != nullptr && exec->ClosedForm(params[0], n, w->cclBytes, closed)) {
            if (FoldsFromClosedForm(closed, params, dtype, op, folds, text)) {
                haveFolds = true;
            } else {   // a tree that no kernel evaluates: the recorded steps decide how it runs
                folds.clear();
                if (text) text->clear();
            }
            lap("closedform");
        }
    }
    if (!haveFolds) CHK_RET(expand(!fused && !w->dryRun));

    if (fused || w->dryRun || w->traceText || w->check) {
        bool ok = true;
        if (!haveFolds) {
            Tracer tr;
            for (const Node &nd : order) {
                const TaskItem &it = *nd.item;
                if (it.kind == ItemKind::COPY) {
                    tr.Copy(reinterpret_cast<u64>(it.dst), reinterpret_cast<u64>(it.src), it.bytes);
                } else {
                    tr.Reduce(reinterpret_cast<u64>(it.dst), reinterpret_cast<u64>(it.src), it.bytes);
                }
            }
            lap("trace");
            if (w->check) {
                CheckSemantics(tr, params, w->lastCheck);
                CHK_PRT_RET(w->lastCheck.races != 0 || w->lastCheck.semanticErrors != 0,
                            HCCL_ERROR("[schedule check] %s", w->lastCheck.firstProblem.c_str()), HCCL_E_INTERNAL);
            }
            std::string checkedText;
            std::string *traceOut = text ? text : (w->check ? &checkedText : nullptr);
            ok = FoldsFromTrace(tr, params, foldType, op, folds, traceOut);
            // A template that also states its result in closed form is planned from that statement when the check
            // is off: so the check holds the statement against what the recorded steps amount to, piece by piece
            // and in the same association order.
            if (ok && w->check && !IsDataMove(type) && BuffersAreSeparate(params)) {
                std::unique_ptr<InsCollAlgBase> exec = CollAlgExecRegistryV2::Instance().GetAlgExec(type, algName);
                std::vector<ClosedFold> closed;
                std::vector<Fold> stated;
                std::string statedText;
                params[0].algName = algName;
                if (exec != nullptr && exec->ClosedForm(params[0], n, w->cclBytes, closed) &&
                    FoldsFromClosedForm(closed, params, dtype, op, stated, &statedText) && statedText != *traceOut) {
                    // the first line that differs names the piece
                    size_t at = 0;
                    while (at < statedText.size() && at < traceOut->size() && statedText[at] == (*traceOut)[at]) ++at;
                    const size_t from = statedText.rfind('\n', at ? at - 1 : 0);
                    const size_t lineStart = (from == std::string::npos || at == 0) ? 0 : from + 1;
                    const size_t lineEnd = statedText.find('\n', lineStart);
                    w->lastCheck.semanticErrors++;
                    if (w->lastCheck.firstProblem.empty()) {
                        w->lastCheck.firstProblem = "the template's closed form is not what its recorded steps amount to; it states: " +
                                                    statedText.substr(lineStart, lineEnd == std::string::npos ? std::string::npos
                                                                                                             : lineEnd - lineStart);
                    }
                    HCCL_ERROR("[schedule check] %s", w->lastCheck.firstProblem.c_str());
                    return HCCL_E_INTERNAL;
                }
            }
        }
        FusedPlan plan;
        ok = ok && BuildFusedPlan(params, folds, esz, plan, haveFolds);
        lap("fusedplan");
        w->lastFusedSegments =
            static_cast<u32>(plan.chainSegs.size() + plan.selfSegs.size() + plan.copySegs.size() + plan.treeSegs.size() +
                             plan.wideSegs.size() + plan.wideTreeSegs.size() + plan.wideSelfSegs.size() +
                             plan.stagedSelfSegs.size());
        if (w->dryRun) {
            w->lastWasFused = ok;
            return HCCL_SUCCESS;
        }
        if (ok && fused) {
            std::vector<HostPart> parts;
            auto add = [&](std::vector<hcclx_seg_t> &segs, int dt, int mode) {
                if (segs.empty()) return;
                parts.emplace_back();
                parts.back().dtype = dt;
                parts.back().op = op;
                parts.back().mode = mode;
                parts.back().segs = std::move(segs);
            };
            auto addWide = [&](std::vector<hcclx_wide_seg_t> &segs, int mode) {
                if (segs.empty()) return;
                parts.emplace_back();
                parts.back().wide = true;
                parts.back().dtype = foldType;
                parts.back().op = op;
                parts.back().mode = mode;
                parts.back().wideSegs = std::move(segs);
            };
            add(plan.selfSegs, foldType, HCCLX_FOLD_SELF_FIRST);
            add(plan.chainSegs, foldType, HCCLX_FOLD_CHAIN);
            add(plan.copySegs, HCCL_DATA_TYPE_INT8, HCCLX_FOLD_CHAIN);
            add(plan.treeSegs, foldType, HCCLX_FOLD_TREE);
            addWide(plan.wideSegs, HCCLX_FOLD_CHAIN);
            addWide(plan.wideTreeSegs, HCCLX_FOLD_TREE);
            addWide(plan.wideSelfSegs, HCCLX_FOLD_SELF_FIRST);
            CachedPlan c;
            c.key = key;
            c.levels = numLevels;
            c.segments = w->lastFusedSegments;
            const bool stagedOutputs = !plan.stagedSelfSegs.empty();
            if (stagedOutputs) {
                // outputs that go through a staging buffer of the plan's own: kept with its addresses only
                char *staging = nullptr;
                if (hipMalloc(reinterpret_cast<void **>(&staging), plan.stagingBytes) != hipSuccess) return HCCL_E_RUNTIME;
                c.buffers.push_back(staging);
                for (hcclx_wide_seg_t &seg : plan.stagedSelfSegs) {
                    for (uint32_t j = 0; j < seg.ndst; ++j) seg.dst[j] = staging + reinterpret_cast<u64>(seg.dst[j]);
                }
                addWide(plan.stagedSelfSegs, HCCLX_FOLD_SELF_FIRST);
                std::vector<hcclx_seg_t> copies;
                for (const FusedPlan::StagedCopy &sc : plan.stagedCopies) {
                    hcclx_seg_t cp;
                    std::memset(&cp, 0, sizeof(cp));
                    cp.count = sc.bytes;
                    cp.nsrc = 1;
                    cp.ndst = 1;
                    cp.src[0] = staging + sc.offset;
                    cp.dst[0] = reinterpret_cast<void *>(sc.dst);
                    copies.push_back(cp);
                }
                // launched last: every read of the inputs is queued in front of it
                add(copies, HCCL_DATA_TYPE_INT8, HCCLX_FOLD_CHAIN);
            }
            const HcclResult made = CreatePlans(parts, c.plans);
            if (made != HCCL_SUCCESS) {
                DropPlans(c.plans, c.buffers);
                return made;
            }
            lap("tables");
            w->lastWasFused = true;
            const HcclResult res = LaunchAndKeep(w, std::move(c), stream);
            lap("launch");
            if (res == HCCL_SUCCESS && separate && !stagedOutputs) {
                KeepShape(w->planCache, shape, std::move(parts), params, true, numLevels, w->lastFusedSegments);
            }
            return res;
        }
    }
    if (!recordedOnMemory) CHK_RET(expand(true));   // recorded (again) against scratch buffers that exist
    std::vector<HostPart> parts;
    BuildStepParts(order, numLevels, foldType, op, parts);
    CachedPlan c;
    c.key = key;
    c.fused = false;
    c.levels = numLevels;
    const HcclResult made = CreatePlans(parts, c.plans);
    if (made != HCCL_SUCCESS) {
        DropPlans(c.plans, c.buffers);
        return made;
    }
    const HcclResult res = LaunchAndKeep(w, std::move(c), stream);
    if (res == HCCL_SUCCESS && separate) KeepShape(w->planCache, shape, std::move(parts), params, false, numLevels, 0);
    return res;
}

}  // namespace

}  // namespace ops_hccl
