// Virtual-rank world: creation, the recording primitive backend and the rank rendezvous.
#include "vcomm.h"

#include <atomic>

#include <algorithm>
#include <cstring>

#include "hcclx.h"
#include "hcomm_primitives.h"
#include "schedule.h"

namespace ops_hccl {

namespace {

std::mutex g_worldsMu;
std::vector<World *> g_worlds;

// Notify indices a thread or channel may use (the templates stay below 4 * ranks).
constexpr u32 kMaxNotifyIdx = 4096;

// The number of the notify identity `idx` of a table (a channel direction or a thread), assigned on first use and
// kept for the life of the world.
bool SlotOf(World *w, std::vector<u32> &table, u32 idx, u64 &slot)
{
    if (idx >= kMaxNotifyIdx) return false;
    if (idx >= table.size()) table.resize(idx + 1, 0);
    if (table[idx] == 0) {
        w->recordSeq.push_back(0);
        w->waitSeq.push_back(0);
        table[idx] = static_cast<u32>(w->recordSeq.size());
    }
    slot = table[idx] - 1;
    return true;
}

VThread *AsThread(ThreadHandle h) { return reinterpret_cast<VThread *>(h); }
VChannel *AsChannel(ChannelHandle h) { return reinterpret_cast<VChannel *>(h); }

int32_t RecordData(ThreadHandle thread, ItemKind kind, void *dst, const void *src, u64 bytes, u64 count, int dtype,
                   int op)
{
    VThread *t = AsThread(thread);
    if (t == nullptr) return HCCL_E_PTR;
    if (bytes == 0) return HCCL_SUCCESS;
    if (dst == nullptr || src == nullptr) return HCCL_E_PTR;
    TaskItem it;
    it.kind = kind;
    it.dst = static_cast<char *>(dst);
    it.src = static_cast<const char *>(src);
    it.bytes = bytes;
    it.count = count;
    it.dtype = static_cast<u8>(dtype);
    it.op = static_cast<u8>(op);
    t->items.push_back(it);
    return HCCL_SUCCESS;
}

int32_t RecordNotify(VThread *t, ItemKind kind, u64 key)
{
    World *w = t->world;
    TaskItem it;
    it.kind = kind;
    it.key = key;
    it.seq = (kind == ItemKind::NOTIFY_RECORD) ? w->recordSeq[key]++ : w->waitSeq[key]++;
    t->items.push_back(it);
    return HCCL_SUCCESS;
}

int32_t ReduceArgsOk(HcommDataType dt, HcommReduceOp op)
{
    if (dt < 0 || dt >= HCCL_DATA_TYPE_RESERVED) return HCCL_E_PARA;
    if (op < HCCL_REDUCE_SUM || op > HCCL_REDUCE_MIN) return HCCL_E_PARA;
    return HCCL_SUCCESS;
}

}  // namespace

World::~World()
{
    for (char *p : cclBuf) {
        if (p && scratchIsMemory) (void)hipFree(p);
    }
    if (!dryRun && (!planCache.lru.empty() || !planCache.retired.empty())) (void)hipDeviceSynchronize();
    for (RetiredPlan &r : planCache.retired) {
        if (r.event) (void)hipEventDestroy(static_cast<hipEvent_t>(r.event));
        for (hcclx_plan *p : r.plans) (void)hcclx_plan_destroy(p);
        for (void *b : r.buffers) (void)hipFree(b);
    }
    for (CachedPlan &c : planCache.lru) {
        for (hcclx_plan *p : c.plans) (void)hcclx_plan_destroy(p);
        for (void *b : c.buffers) (void)hipFree(b);
    }
}

// Placeholder scratch addresses: non-canonical, so they can never collide with memory of the process, one
// non-overlapping terabyte per rank.
static char *ScratchPlaceholder(u32 rank)
{
    return reinterpret_cast<char *>(0x7000000000000000ull + static_cast<u64>(rank) * (1ull << 40));
}

HcclResult World::EnsureScratch(bool memory)
{
    if (!memory || dryRun) {
        for (u32 r = 0; r < rankSize; ++r) {
            if (cclBuf[r] == nullptr) cclBuf[r] = ScratchPlaceholder(r);
        }
        return HCCL_SUCCESS;
    }
    if (scratchIsMemory) return HCCL_SUCCESS;
    std::vector<char *> made(rankSize, nullptr);
    for (u32 r = 0; r < rankSize; ++r) {
        const hipError_t e = hipMalloc(reinterpret_cast<void **>(&made[r]), cclBytes);
        if (e != hipSuccess) {
            HCCL_ERROR("scratch buffer of rank %u: %s", r, hipGetErrorString(e));
            for (char *p : made) {
                if (p) (void)hipFree(p);
            }
            return HCCL_E_MEMORY;
        }
    }
    cclBuf = made;
    scratchIsMemory = true;
    return HCCL_SUCCESS;
}

void World::ResetRecording()
{
    std::fill(recordSeq.begin(), recordSeq.end(), 0u);
    std::fill(waitSeq.begin(), waitSeq.end(), 0u);
    for (auto &perRank : threads) {
        for (auto &t : perRank) t->items.clear();
    }
}

HcclResult WorldCreate(u32 rankSize, u64 cclBytes, bool dryRun, std::vector<HcclComm> &comms)
{
    if (rankSize == 0 || rankSize > 64) return HCCL_E_PARA;
    // the ReduceScatter executor keeps 1 MiB of the buffer back; leave room for at least one aligned slot per rank
    if (cclBytes < 1024 * 1024 + 128ull * 64) return HCCL_E_PARA;
    World *w = new World;
    w->rankSize = rankSize;
    w->cclBytes = cclBytes;
    w->dryRun = dryRun;
    if (hipGetDevice(&w->device) != hipSuccess) w->device = -1;  // a host-only process can still record
    if (const char *m = std::getenv("HCCL_VRANK_EXEC_MODE")) {
        if (std::strcmp(m, "step") == 0) w->mode = ExecMode::STEP;
    }
    if (const char *b = std::getenv("HCCL_VRANK_BLOCKING")) w->blocking = (std::atoi(b) != 0);
    if (const char *c = std::getenv("HCCL_VRANK_CHECK")) w->check = (std::atoi(c) != 0);
    if (const char *l = std::getenv("HCCL_VRANK_LINK_PROTOCOL")) {
        if (std::strcmp(l, "pcie") == 0) w->linkProtocol = CommProtocol::COMM_PROTOCOL_PCIE;
        if (std::strcmp(l, "roce") == 0) w->linkProtocol = CommProtocol::COMM_PROTOCOL_ROCE;
    }
    if (const char *c = std::getenv("HCCL_VRANK_CLOSED_FORM")) w->closedForm = std::max(0, std::min(2, std::atoi(c)));
    {
        u8 level = static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_DISABLE);
        if (const char *d = std::getenv("HCCL_DETERMINISTIC")) {
            if (ParseDeterministic(d, level) != HCCL_SUCCESS) {
                delete w;
                return HCCL_E_PARA;
            }
        }
        SetExternalInputHcclDeterministic(level);
    }
    if (const char *a = std::getenv("HCCL_ALGO")) {
        const HcclResult rc = SetHcclAlgoConfig(a, w->algoConfig);
        if (rc != HCCL_SUCCESS) {
            delete w;
            return rc;
        }
    }
    w->cclBuf.assign(rankSize, nullptr);
    w->queue.resize(rankSize);
    w->launched.assign(rankSize, 0);
    w->lastResult.assign(rankSize, HCCL_SUCCESS);
    w->threads.resize(rankSize);
    w->channels.resize(rankSize);
    comms.clear();
    for (u32 r = 0; r < rankSize; ++r) {
        w->ranks.emplace_back(new RankComm{w, r});
        for (u32 t = 0; t < rankSize + 1; ++t) {  // mesh templates use one thread per rank
            w->threads[r].emplace_back(new VThread);
            VThread *vt = w->threads[r].back().get();
            vt->world = w;
            vt->rank = r;
            vt->index = t;
        }
        for (u32 p = 0; p < rankSize; ++p) {
            w->channels[r].emplace_back(new VChannel{w, r, p, {}});
        }
        comms.push_back(w->ranks.back().get());
    }
    std::lock_guard<std::mutex> lock(g_worldsMu);
    g_worlds.push_back(w);
    return HCCL_SUCCESS;
}

RankComm *AsRankComm(HcclComm comm)
{
    RankComm *rc = static_cast<RankComm *>(comm);
    if (rc == nullptr) return nullptr;
    std::lock_guard<std::mutex> lock(g_worldsMu);
    for (World *w : g_worlds) {
        if (rc->world == w && rc->rank < w->rankSize && w->ranks[rc->rank].get() == rc) return rc;
    }
    return nullptr;
}

HcclResult WorldDestroyRank(HcclComm comm)
{
    RankComm *rc = AsRankComm(comm);
    if (rc == nullptr) return HCCL_E_PTR;
    World *w = rc->world;
    {
        std::lock_guard<std::mutex> lock(w->mu);
        w->launched[rc->rank] = ~0ull;  // marks the rank handle as destroyed
        for (u64 v : w->launched) {
            if (v != ~0ull) return HCCL_SUCCESS;
        }
    }
    {
        std::lock_guard<std::mutex> lock(g_worldsMu);
        for (size_t i = 0; i < g_worlds.size(); ++i) {
            if (g_worlds[i] == w) {
                g_worlds.erase(g_worlds.begin() + i);
                break;
            }
        }
    }
    delete w;
    return HCCL_SUCCESS;
}

void FillResources(World *w, u32 rank, u32 threadNum, AlgResourceCtxSerializable &resCtx)
{
    resCtx.topoInfo.userRank = rank;
    resCtx.topoInfo.userRankSize = w->rankSize;
    resCtx.subCommRanks.assign(1, std::vector<u32>());
    for (u32 r = 0; r < w->rankSize; ++r) resCtx.subCommRanks[0].push_back(r);  // TopoMatch1D: ranks 0..N-1
    resCtx.cclMem.addr = w->cclBuf[rank];
    resCtx.cclMem.size = w->cclBytes;
    resCtx.threads.clear();
    for (u32 t = 0; t < threadNum && t < w->threads[rank].size(); ++t) {
        resCtx.threads.push_back(reinterpret_cast<ThreadHandle>(w->threads[rank][t].get()));
    }
    resCtx.channels.clear();
    for (u32 p = 0; p < w->rankSize; ++p) {
        if (p == rank) continue;
        ChannelInfo ch;
        ch.isValid = true;
        ch.remoteRank = p;
        ch.protocol = w->linkProtocol;
        ch.notifyNum = 3;
        ch.portGroupSize = 1;
        ch.handle = reinterpret_cast<ChannelHandle>(w->channels[rank][p].get());
        ch.remoteCclMem.addr = w->cclBuf[p];
        ch.remoteCclMem.size = w->cclBytes;
        resCtx.channels[p].push_back(ch);
    }
}

HcclResult SubmitOp(RankComm *rc, const OpParam &param)
{
    World *w = rc->world;
    std::unique_lock<std::mutex> lock(w->mu);
    QueuedOp q;
    q.param = param;
    w->queue[rc->rank].push_back(std::move(q));
    const u64 myTicket = w->launched[rc->rank] + w->queue[rc->rank].size();  // collective number of this call

    bool all = true;
    for (u32 r = 0; r < w->rankSize; ++r) all = all && !w->queue[r].empty();
    while (all) {
        std::vector<OpParam> params;
        for (u32 r = 0; r < w->rankSize; ++r) {
            params.push_back(std::move(w->queue[r].front().param));
            w->queue[r].pop_front();
        }
        const HcclResult res = RunCollective(w, params);
        for (u32 r = 0; r < w->rankSize; ++r) {
            w->launched[r]++;
            w->lastResult[r] = res;
        }
        w->cv.notify_all();
        all = true;
        for (u32 r = 0; r < w->rankSize; ++r) all = all && !w->queue[r].empty();
    }
    if (w->launched[rc->rank] >= myTicket) return w->lastResult[rc->rank];
    if (!w->blocking) return HCCL_SUCCESS;  // queued; the last rank to arrive launches
    w->cv.wait(lock, [&] { return w->launched[rc->rank] >= myTicket; });
    return w->lastResult[rc->rank];
}

}  // namespace ops_hccl

// ---------------------------------------------------------------------------------------------------
// the primitive ABI: every call is recorded on its thread
// ---------------------------------------------------------------------------------------------------
using namespace ops_hccl;

extern "C" {

int32_t HcommLocalCopyOnThread(ThreadHandle thread, void *dst, const void *src, uint64_t len)
{
    return RecordData(thread, ItemKind::COPY, dst, src, len, len, HCCL_DATA_TYPE_INT8, 0);
}

int32_t HcommLocalReduceOnThread(ThreadHandle thread, void *dst, const void *src, uint64_t count,
                                 HcommDataType dataType, HcommReduceOp reduceOp)
{
    if (ReduceArgsOk(dataType, reduceOp) != HCCL_SUCCESS) return HCCL_E_PARA;
    return RecordData(thread, ItemKind::REDUCE, dst, src, count * DATATYPE_SIZE_TABLE[dataType], count, dataType,
                      reduceOp);
}

int32_t HcommWriteOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src, uint64_t len)
{
    if (AsChannel(channel) == nullptr) return HCCL_E_PTR;
    return RecordData(thread, ItemKind::COPY, dst, src, len, len, HCCL_DATA_TYPE_INT8, 0);
}

int32_t HcommReadOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src, uint64_t len)
{
    if (AsChannel(channel) == nullptr) return HCCL_E_PTR;
    return RecordData(thread, ItemKind::COPY, dst, src, len, len, HCCL_DATA_TYPE_INT8, 0);
}

int32_t HcommWriteReduceOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                 uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp)
{
    if (AsChannel(channel) == nullptr) return HCCL_E_PTR;
    if (ReduceArgsOk(dataType, reduceOp) != HCCL_SUCCESS) return HCCL_E_PARA;
    return RecordData(thread, ItemKind::REDUCE, dst, src, count * DATATYPE_SIZE_TABLE[dataType], count, dataType,
                      reduceOp);
}

int32_t HcommReadReduceOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                uint64_t count, HcommDataType dataType, HcommReduceOp reduceOp)
{
    return HcommWriteReduceOnThread(thread, channel, dst, src, count, dataType, reduceOp);
}

int32_t HcommChannelNotifyRecordOnThread(ThreadHandle thread, ChannelHandle channel, uint32_t remoteNotifyIdx)
{
    VThread *t = AsThread(thread);
    VChannel *c = AsChannel(channel);
    if (t == nullptr || c == nullptr) return HCCL_E_PTR;
    if (c->world != t->world) return HCCL_E_PARA;   // a handle of another world would index past this world's tables
    u64 slot = 0;
    if (!SlotOf(t->world, c->notifySlot, remoteNotifyIdx, slot)) return HCCL_E_PARA;
    return RecordNotify(t, ItemKind::NOTIFY_RECORD, slot);
}

int32_t HcommChannelNotifyWaitOnThread(ThreadHandle thread, ChannelHandle channel, uint32_t localNotifyIdx,
                                       uint32_t timeout)
{
    (void)timeout;
    VThread *t = AsThread(thread);
    VChannel *c = AsChannel(channel);
    if (t == nullptr || c == nullptr) return HCCL_E_PTR;
    World *w = t->world;
    if (c->world != w || c->remoteRank >= w->rankSize || c->localRank >= w->rankSize) return HCCL_E_PARA;
    // the same identity as the record on the sender's side of the link
    VChannel *sender = w->channels[c->remoteRank][c->localRank].get();
    u64 slot = 0;
    if (!SlotOf(w, sender->notifySlot, localNotifyIdx, slot)) return HCCL_E_PARA;
    return RecordNotify(t, ItemKind::NOTIFY_WAIT, slot);
}

int32_t HcommThreadNotifyRecordOnThread(ThreadHandle thread, ThreadHandle dstThread, uint32_t dstNotifyIdx)
{
    VThread *t = AsThread(thread);
    VThread *d = AsThread(dstThread);
    if (t == nullptr || d == nullptr) return HCCL_E_PTR;
    if (d->world != t->world) return HCCL_E_PARA;   // as above
    u64 slot = 0;
    if (!SlotOf(t->world, d->notifySlot, dstNotifyIdx, slot)) return HCCL_E_PARA;
    return RecordNotify(t, ItemKind::NOTIFY_RECORD, slot);
}

int32_t HcommThreadNotifyWaitOnThread(ThreadHandle thread, uint32_t notifyIdx, uint32_t timeout)
{
    (void)timeout;
    VThread *t = AsThread(thread);
    if (t == nullptr) return HCCL_E_PTR;
    u64 slot = 0;
    if (!SlotOf(t->world, t->notifySlot, notifyIdx, slot)) return HCCL_E_PARA;
    return RecordNotify(t, ItemKind::NOTIFY_WAIT, slot);
}

// The waits every verb of the reference's wrapper tries first (hcomm_primitives_dl.cc:155-173): the time-out is the
// process-wide one set with HcommSetNotifyWaitTimeOut.  A recorded wait has no clock, so the value is only kept.
namespace {
std::atomic<uint32_t> g_notifyWaitTimeout{0};
std::atomic<uint32_t> g_threadResAcquireTimeout{0};
}  // namespace

int32_t HcommSetNotifyWaitTimeOut(uint32_t timeOut)
{
    g_notifyWaitTimeout.store(timeOut);
    return HCCL_SUCCESS;
}

int32_t HcommThreadResAcquireTimeOut(uint32_t timeOut)
{
    g_threadResAcquireTimeout.store(timeOut);
    return HCCL_SUCCESS;
}

int32_t HcommThreadNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, uint32_t notifyIdx)
{
    return HcommThreadNotifyWaitOnThread(thread, notifyIdx, g_notifyWaitTimeout.load());
}

int32_t HcommChannelNotifyWaitOnThreadWithDefaultTimeout(ThreadHandle thread, ChannelHandle channel,
                                                         uint32_t localNotifyIdx)
{
    return HcommChannelNotifyWaitOnThread(thread, channel, localNotifyIdx, g_notifyWaitTimeout.load());
}

int32_t HcommWriteWithNotifyNbiOnThread(ThreadHandle thread, ChannelHandle channel, void *dst, const void *src,
                                        uint64_t len, uint32_t remoteNotifyIdx)
{
    const int32_t rc = HcommWriteOnThread(thread, channel, dst, src, len);
    if (rc != HCCL_SUCCESS) return rc;
    return HcommChannelNotifyRecordOnThread(thread, channel, remoteNotifyIdx);
}

int32_t HcommChannelFenceOnThread(ThreadHandle thread, ChannelHandle channel)
{
    // the steps of a thread are recorded, and later ordered, in program order: a fence adds nothing
    VThread *t = AsThread(thread);
    VChannel *c = AsChannel(channel);
    if (t == nullptr || c == nullptr) return HCCL_E_PTR;
    return c->world == t->world ? HCCL_SUCCESS : HCCL_E_PARA;
}

int32_t HcommBatchTransferOnThread(ThreadHandle thread, ChannelHandle channel,
                                   const HcclHcommBatchTransferDesc *transferDescs, uint32_t transferDescNum)
{
    if (AsThread(thread) == nullptr || AsChannel(channel) == nullptr) return HCCL_E_PTR;
    if (transferDescNum != 0 && transferDescs == nullptr) return HCCL_E_PTR;
    for (uint32_t i = 0; i < transferDescNum; ++i) {
        const HcclHcommBatchTransferDesc &d = transferDescs[i];
        int32_t rc = HCCL_SUCCESS;
        switch (d.transType) {
            case HCCL_HCOMM_TRANSFER_TYPE_WRITE:
                rc = HcommWriteOnThread(thread, channel, d.transferInfo.write.dst, d.transferInfo.write.src,
                                        d.transferInfo.write.len);
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_READ:
                rc = HcommReadOnThread(thread, channel, d.transferInfo.read.dst, d.transferInfo.read.src,
                                       d.transferInfo.read.len);
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE:
                rc = HcommWriteReduceOnThread(thread, channel, d.transferInfo.reduce.dst, d.transferInfo.reduce.src,
                                              d.transferInfo.reduce.count, d.transferInfo.reduce.dataType,
                                              d.transferInfo.reduce.reduceOp);
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_READ_REDUCE:
                rc = HcommReadReduceOnThread(thread, channel, d.transferInfo.reduce.dst, d.transferInfo.reduce.src,
                                             d.transferInfo.reduce.count, d.transferInfo.reduce.dataType,
                                             d.transferInfo.reduce.reduceOp);
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_WRITE_WITH_NOTIFY:
                rc = HcommWriteOnThread(thread, channel, d.transferInfo.writeWithNotify.dst,
                                        d.transferInfo.writeWithNotify.src, d.transferInfo.writeWithNotify.len);
                if (rc == HCCL_SUCCESS) {
                    rc = HcommChannelNotifyRecordOnThread(thread, channel, d.transferInfo.writeWithNotify.notifyIdx);
                }
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_WRITE_REDUCE_WITH_NOTIFY:
                rc = HcommWriteReduceOnThread(thread, channel, d.transferInfo.writeReduceWithNotify.dst,
                                              d.transferInfo.writeReduceWithNotify.src,
                                              d.transferInfo.writeReduceWithNotify.count,
                                              d.transferInfo.writeReduceWithNotify.dataType,
                                              d.transferInfo.writeReduceWithNotify.reduceOp);
                if (rc == HCCL_SUCCESS) {
                    rc = HcommChannelNotifyRecordOnThread(thread, channel, d.transferInfo.writeReduceWithNotify.notifyIdx);
                }
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_RECORD:
                rc = HcommChannelNotifyRecordOnThread(thread, channel, d.transferInfo.notifyRecord.notifyIdx);
                break;
            case HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_WAIT:
            case HCCL_HCOMM_TRANSFER_TYPE_NOTIFY_WAIT_WITH_DEFAULT_TIMEOUT:
                rc = HcommChannelNotifyWaitOnThread(thread, channel, d.transferInfo.notifyRecord.notifyIdx, 0);
                break;
            default:
                return HCCL_E_PARA;
        }
        if (rc != HCCL_SUCCESS) return rc;
    }
    return HCCL_SUCCESS;
}

int32_t HcommBatchModeStart(const char *batchTag)
{
    (void)batchTag;
    return HCCL_SUCCESS;
}

int32_t HcommBatchModeEnd(const char *batchTag)
{
    (void)batchTag;
    return HCCL_SUCCESS;
}

int32_t HcommThreadJoin(ThreadHandle thread, uint32_t timeout)
{
    (void)thread;
    (void)timeout;
    return HCCL_SUCCESS;
}

}  // extern "C"
