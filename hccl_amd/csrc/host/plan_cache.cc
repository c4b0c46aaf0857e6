// Plan keys, the two plan caches, moving a plan to other buffers, launching.
#include <algorithm>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "schedule_internal.h"

namespace ops_hccl {
namespace sched {

// What the plan of a collective depends on apart from where the buffers lie, as plain numbers (a string would cost
// more to build than the launch).  The last words say which ranks run in place.
std::vector<u64> ShapeKey(const std::vector<OpParam> &params, const std::string &alg, u64 cclBytes)
{
    const OpParam &p0 = params[0];
    std::vector<u64> key;
    key.reserve(10 + 2 * p0.vDataDes.counts.size() + 2 * params.size());
    key.push_back(static_cast<u64>(p0.opType));
    key.push_back(std::hash<std::string>()(alg));
    key.push_back(static_cast<u64>(p0.DataDes.dataType));
    key.push_back(static_cast<u64>(p0.reduceType));
    key.push_back(p0.DataDes.count);
    key.push_back(cclBytes);
    key.push_back(p0.vDataDes.counts.size());
    key.insert(key.end(), p0.vDataDes.counts.begin(), p0.vDataDes.counts.end());
    key.insert(key.end(), p0.vDataDes.displs.begin(), p0.vDataDes.displs.end());
    // The AlltoAll family: what moves is in every rank's tables, not in the extents (an expert router changes the
    // counts every step while the buffers stay where they are).
    if (p0.opType == HcclCMDType::HCCL_CMD_ALLTOALL || p0.opType == HcclCMDType::HCCL_CMD_ALLTOALLV ||
        p0.opType == HcclCMDType::HCCL_CMD_ALLTOALLVC) {
        key.push_back(static_cast<u64>(p0.all2AllVDataDes.sendType));
        for (const OpParam &p : params) {
            const auto &d = p.all2AllVDataDes;
            key.push_back(d.sendCounts.size());
            key.insert(key.end(), d.sendCounts.begin(), d.sendCounts.end());
            key.insert(key.end(), d.sdispls.begin(), d.sdispls.end());
            key.insert(key.end(), d.recvCounts.begin(), d.recvCounts.end());
            key.insert(key.end(), d.rdispls.begin(), d.rdispls.end());
        }
    }
    for (const OpParam &p : params) {
        key.push_back(p.inputSize);
        key.push_back(p.outputSize);
        key.push_back(p.inputPtr == p.outputPtr ? 1 : 0);
    }
    return key;
}

// The shape and the addresses: what a plan with its tables in device memory is found by.
std::vector<u64> PlanKey(const std::vector<u64> &shape, const std::vector<OpParam> &params)
{
    std::vector<u64> key = shape;
    for (const OpParam &p : params) {
        key.push_back(reinterpret_cast<u64>(p.inputPtr));
        key.push_back(reinterpret_cast<u64>(p.outputPtr));
    }
    return key;
}

// True when no two of the ranks' buffers overlap, a rank's input being the same as its own output aside: then the
// recorded schedule, its trace and the plan made from it are the same wherever the buffers lie, and a plan made for
// one set of addresses serves another by shifting every pointer with its buffer.
bool BuffersAreSeparate(const std::vector<OpParam> &params)
{
    struct R {
        u64 lo, hi;
    };
    std::vector<R> r;
    r.reserve(2 * params.size());
    for (const OpParam &p : params) {
        const u64 in = reinterpret_cast<u64>(p.inputPtr);
        const u64 out = reinterpret_cast<u64>(p.outputPtr);
        if (in == out) {
            const u64 size = std::max(p.inputSize, p.outputSize);
            if (size) r.push_back({in, in + size});
            continue;
        }
        if (p.inputSize != 0) r.push_back({in, in + p.inputSize});
        if (p.outputSize != 0) r.push_back({out, out + p.outputSize});
    }
    std::sort(r.begin(), r.end(), [](const R &a, const R &b) { return a.lo < b.lo; });
    for (size_t i = 1; i < r.size(); ++i) {
        if (r[i].lo < r[i - 1].hi) return false;
    }
    return true;
}

// For every pointer of a shape plan's parts, in the order segments hold them (sources, then destinations), which of
// the ranks' buffers it points into: 1 + its index in `buffers`, or 0 for a pointer outside them (the scratch
// buffers of step plans, which belong to the world and stay where they are).  False when the plan cannot be moved
// with its buffers: a run that starts in a buffer and ends beyond it (it would straddle two buffers that only
// happened to lie back to back), or a run of a fused plan, which has no scratch buffers, that lies in none.
static bool FindOwners(ShapePlan &sp)
{
    struct Range {
        u64 lo, hi;
        uint16_t owner;
    };
    std::vector<Range> ranges;
    for (size_t b = 0; b < sp.buffers.size(); b += 2) {
        const ShapePlan::Buffer &in = sp.buffers[b];
        const ShapePlan::Buffer &out = sp.buffers[b + 1];
        if (in.base == out.base) {   // in place: one buffer, as long as the longer of the two
            const u64 size = std::max(in.size, out.size);
            if (size) ranges.push_back({in.base, in.base + size, static_cast<uint16_t>(b + 1)});
            continue;
        }
        if (in.size) ranges.push_back({in.base, in.base + in.size, static_cast<uint16_t>(b + 1)});
        if (out.size) ranges.push_back({out.base, out.base + out.size, static_cast<uint16_t>(b + 2)});
    }
    std::sort(ranges.begin(), ranges.end(), [](const Range &a, const Range &b) { return a.lo < b.lo; });
    // Segments of one plan mostly name the ranks in the same order, so the range the pointer at the same place of
    // the segment before fell into is tried first; the search is for the others.
    auto rangeOf = [&](const void *p, size_t guess) -> size_t {
        const u64 a = reinterpret_cast<u64>(p);
        if (guess < ranges.size() && a >= ranges[guess].lo && a < ranges[guess].hi) return guess;
        auto it = std::upper_bound(ranges.begin(), ranges.end(), a, [](u64 v, const Range &m) { return v < m.lo; });
        if (it == ranges.begin()) return ranges.size();
        --it;
        return a < it->hi ? static_cast<size_t>(it - ranges.begin()) : ranges.size();
    };
    sp.owners.assign(sp.parts.size(), {});
    std::vector<size_t> guess(2 * HCCLX_MAX_WIDE_FAN, ranges.size());
    bool movable = true;
    for (size_t i = 0; i < sp.parts.size(); ++i) {
        std::vector<uint16_t> &own = sp.owners[i];
        const u64 esz = hcclx_dtype_size(sp.parts[i].dtype);
        auto each = [&](const auto &segs) {
            for (const auto &g : segs) {
                for (uint32_t k = 0; k < g.nsrc + g.ndst; ++k) {
                    const void *p = k < g.nsrc ? g.src[k] : g.dst[k - g.nsrc];
                    size_t &at = guess[k < g.nsrc ? k : HCCLX_MAX_WIDE_FAN + k - g.nsrc];
                    at = rangeOf(p, at);
                    own.push_back(at < ranges.size() ? ranges[at].owner : 0);
                    if (g.count == 0) continue;
                    if (at < ranges.size()) {
                        if (reinterpret_cast<u64>(p) + g.count * esz > ranges[at].hi) movable = false;
                    } else if (sp.fused) {
                        movable = false;
                    }
                }
            }
        };
        each(sp.parts[i].segs);
        each(sp.parts[i].wideSegs);
    }
    return movable;
}

// Moves the pointers of a shape plan's parts from the buffers it was made for to those of `params`: every pointer
// goes along with the buffer it points into.
void Rebase(const ShapePlan &sp, const std::vector<OpParam> &params, std::vector<HostPart> &parts)
{
    std::vector<int64_t> delta(1 + sp.buffers.size(), 0);   // by owner; 0 = stays
    for (size_t r = 0; r < params.size(); ++r) {
        delta[1 + 2 * r] = static_cast<int64_t>(reinterpret_cast<u64>(params[r].inputPtr) - sp.buffers[2 * r].base);
        delta[2 + 2 * r] = static_cast<int64_t>(reinterpret_cast<u64>(params[r].outputPtr) - sp.buffers[2 * r + 1].base);
    }
    auto shift = [&](const void *p, uint16_t owner) -> void * {
        return reinterpret_cast<void *>(reinterpret_cast<u64>(p) + static_cast<u64>(delta[owner]));
    };
    parts = sp.parts;
    for (size_t i = 0; i < parts.size(); ++i) {
        const uint16_t *own = sp.owners[i].data();
        auto each = [&](auto &segs) {
            for (auto &g : segs) {
                for (uint32_t k = 0; k < g.nsrc; ++k) g.src[k] = shift(g.src[k], *own++);
                for (uint32_t k = 0; k < g.ndst; ++k) g.dst[k] = shift(g.dst[k], *own++);
            }
        };
        each(parts[i].segs);
        each(parts[i].wideSegs);
    }
}

// Device-resident plans of a list of parts.
HcclResult CreatePlans(const std::vector<HostPart> &parts, std::vector<hcclx_plan *> &plans)
{
    for (const HostPart &hp : parts) {
        hcclx_plan *p = nullptr;
        const int rc = hp.wide ? hcclx_plan_create_wide(hp.wideSegs.data(), static_cast<uint32_t>(hp.wideSegs.size()), hp.dtype,
                                                        hp.op, hp.mode, &p)
                               : hcclx_plan_create(hp.segs.data(), static_cast<uint32_t>(hp.segs.size()), hp.dtype, hp.op,
                                                   hp.mode, &p);
        if (rc != HCCL_SUCCESS) return static_cast<HcclResult>(rc);
        plans.push_back(p);
    }
    return HCCL_SUCCESS;
}

// The same parts launched once, their tables travelling through the descriptor ring: no allocation, no plan kept.
HcclResult LaunchParts(World *w, const std::vector<HostPart> &parts, void *stream)
{
    (void)w;
    for (const HostPart &hp : parts) {
        const int rc = hp.wide ? hcclx_fold_wide(hp.wideSegs.data(), static_cast<uint32_t>(hp.wideSegs.size()), hp.dtype, hp.op,
                                                 hp.mode, stream)
                               : hcclx_fold(hp.segs.data(), static_cast<uint32_t>(hp.segs.size()), hp.dtype, hp.op, hp.mode,
                                            stream);
        if (rc != HCCL_SUCCESS) return static_cast<HcclResult>(rc);
    }
    return HCCL_SUCCESS;
}

HcclResult LaunchPlans(World *w, const std::vector<hcclx_plan *> &plans, void *stream)
{
    (void)w;
    for (hcclx_plan *p : plans) {
        const int rc = hcclx_plan_launch(p, stream);
        if (rc != HCCL_SUCCESS) return static_cast<HcclResult>(rc);
    }
    return HCCL_SUCCESS;
}

void DropPlans(std::vector<hcclx_plan *> &plans, std::vector<void *> &buffers)
{
    for (hcclx_plan *q : plans) (void)hcclx_plan_destroy(q);
    plans.clear();
    for (void *b : buffers) (void)hipFree(b);
    buffers.clear();
}

u64 HashKey(const std::vector<u64> &key)
{
    u64 h = 1469598103934665603ull;   // FNV-1a over the words
    for (u64 w : key) {
        h ^= w;
        h *= 1099511628211ull;
    }
    return h;
}

// Frees the retired plans whose kernels have finished.
void ReapRetired(PlanCache &cache, bool wait)
{
    size_t kept = 0;
    for (RetiredPlan &r : cache.retired) {
        hipEvent_t ev = static_cast<hipEvent_t>(r.event);
        bool done = (ev == nullptr);
        if (!done) {
            done = wait ? (hipEventSynchronize(ev) == hipSuccess) : (hipEventQuery(ev) == hipSuccess);
        }
        if (done) {
            if (ev) (void)hipEventDestroy(ev);
            DropPlans(r.plans, r.buffers);
        } else {
            cache.retired[kept++] = std::move(r);
        }
    }
    cache.retired.resize(kept);
}

CachedPlan *FindPlan(PlanCache &cache, const std::vector<u64> &key)
{
    auto range = cache.index.equal_range(HashKey(key));
    for (auto it = range.first; it != range.second; ++it) {
        if (it->second->key == key) {
            cache.lru.splice(cache.lru.begin(), cache.lru, it->second);   // most recently used first
            return &*it->second;
        }
    }
    return nullptr;
}

ShapePlan *FindShape(PlanCache &cache, const std::vector<u64> &shape)
{
    auto range = cache.shapeIndex.equal_range(HashKey(shape));
    for (auto it = range.first; it != range.second; ++it) {
        if (it->second->key == shape) {
            cache.shapes.splice(cache.shapes.begin(), cache.shapes, it->second);
            return &*it->second;
        }
    }
    return nullptr;
}

// True when this address key was launched from a shape plan before (among the last few dozen such launches);
// remembers it otherwise.
bool SeenBefore(PlanCache &cache, u64 hash)
{
    constexpr size_t kRemembered = 64;
    if (std::find(cache.seenOnce.begin(), cache.seenOnce.end(), hash) != cache.seenOnce.end()) return true;
    if (cache.seenOnce.size() < kRemembered) {
        cache.seenOnce.push_back(hash);
    } else {
        cache.seenOnce[cache.seenAt] = hash;
        cache.seenAt = (cache.seenAt + 1) % kRemembered;
    }
    return false;
}

// Keeps the host side of a plan so that the same collective on other buffers need not be planned again.
void KeepShape(PlanCache &cache, const std::vector<u64> &shape, std::vector<HostPart> &&parts,
               const std::vector<OpParam> &params, bool fused, u32 levels, u32 segments)
{
    if (shape.empty() || FindShape(cache, shape) != nullptr) return;
    ShapePlan sp;
    sp.key = shape;
    sp.parts = std::move(parts);
    sp.fused = fused;
    sp.levels = levels;
    sp.segments = segments;
    sp.hostBytes = shape.size() * sizeof(u64);
    for (const HostPart &hp : sp.parts) {
        sp.hostBytes += hp.segs.size() * sizeof(hcclx_seg_t) + hp.wideSegs.size() * sizeof(hcclx_wide_seg_t);
    }
    if (sp.hostBytes > kShapeCacheBytes / 4) return;   // one plan must not push most of the others out
    for (const OpParam &p : params) {
        sp.buffers.push_back({reinterpret_cast<u64>(p.inputPtr), p.inputSize});
        sp.buffers.push_back({reinterpret_cast<u64>(p.outputPtr), p.outputSize});
    }
    if (!FindOwners(sp)) return;   // planned for its addresses only
    for (const std::vector<uint16_t> &own : sp.owners) sp.hostBytes += own.size() * sizeof(uint16_t);
    cache.shapeBytes += sp.hostBytes;
    cache.shapes.push_front(std::move(sp));
    cache.shapeIndex.emplace(HashKey(shape), cache.shapes.begin());
    while (cache.shapes.size() > 1 && (cache.shapes.size() > kShapeCacheEntries || cache.shapeBytes > kShapeCacheBytes)) {
        auto victim = std::prev(cache.shapes.end());
        auto range = cache.shapeIndex.equal_range(HashKey(victim->key));
        for (auto it = range.first; it != range.second; ++it) {
            if (it->second == victim) {
                cache.shapeIndex.erase(it);
                break;
            }
        }
        cache.shapeBytes -= victim->hostBytes;
        cache.shapes.erase(victim);
    }
}

// Launches a freshly built plan and, when it has a key, keeps it for the next identical collective.  A plan that
// is not kept is destroyed once its kernels have finished.
HcclResult LaunchAndKeep(World *w, CachedPlan &&c, void *stream)
{
    PlanCache &cache = w->planCache;
    const HcclResult res = LaunchPlans(w, c.plans, stream);
    if (c.key.empty() || res != HCCL_SUCCESS) {
        (void)hipDeviceSynchronize();
        DropPlans(c.plans, c.buffers);
        return res;
    }
    c.lastStream = stream;
    c.tableBytes = 0;
    for (hcclx_plan *p : c.plans) c.tableBytes += hcclx_plan_table_bytes(p);
    cache.bytes += c.tableBytes;
    cache.lru.push_front(std::move(c));
    cache.index.emplace(HashKey(cache.lru.front().key), cache.lru.begin());
    while (cache.lru.size() > 1 && (cache.lru.size() > kPlanCacheEntries || cache.bytes > kPlanCacheBytes)) {
        auto victim = std::prev(cache.lru.end());
        auto range = cache.index.equal_range(HashKey(victim->key));
        for (auto it = range.first; it != range.second; ++it) {
            if (it->second == victim) {
                cache.index.erase(it);
                break;
            }
        }
        RetiredPlan r;
        r.plans = std::move(victim->plans);
        r.buffers = std::move(victim->buffers);
        hipEvent_t ev = nullptr;
        if (!victim->manyStreams && hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess &&
            hipEventRecord(ev, static_cast<hipStream_t>(victim->lastStream)) == hipSuccess) {
            r.event = ev;
        } else {
            if (ev) (void)hipEventDestroy(ev);
            (void)hipDeviceSynchronize();   // no single event covers it: make sure nothing still reads the tables
        }
        cache.bytes -= victim->tableBytes;
        cache.lru.erase(victim);
        cache.retired.push_back(std::move(r));
    }
    return res;
}


}  // namespace sched
}  // namespace ops_hccl
