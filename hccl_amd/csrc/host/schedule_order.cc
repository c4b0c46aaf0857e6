// Recorded steps -> dependency levels (and the race check); the launch lists of the step-by-step mode.
#include <algorithm>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "schedule_internal.h"

namespace ops_hccl {
namespace sched {

PhaseTimer g_phase;

// ---------------------------------------------------------------------------------------------------
// dependency order of the recorded steps
// ---------------------------------------------------------------------------------------------------
namespace {

bool IsDataOp(const TaskItem &it) { return it.kind == ItemKind::COPY || it.kind == ItemKind::REDUCE; }

// Flattens every thread's items into `order` (a topological order) and gives each data step a level:
// steps of one level do not depend on each other.  Fails when a wait has no matching record (the
// schedule would hang) or the dependencies form a cycle.
// With `report`, also looks for data races: two steps that the handshakes leave unordered and that touch
// the same bytes, at least one of them writing.  Up to kExhaustiveSteps steps every such pair is tested
// for a dependency path; beyond that only steps of the same level (which are unordered by construction).
constexpr size_t kExhaustiveSteps = 4096;

// A step is followed by the next one of its thread and, when it is a record, by the wait it releases: records
// and waits of one identity pair up one to one.
struct Succ {
    int n = 0;
    int to[2] = {-1, -1};
    std::vector<int> more;   // a record that several waits matched (a malformed schedule): kept so that it is reported
    void Add(int id)
    {
        if (n < 2) {
            to[n] = id;
        } else {
            more.push_back(id);
        }
        ++n;
    }
    template <typename F> void Each(F &&f) const
    {
        for (int k = 0; k < n && k < 2; ++k) f(to[k]);
        for (int id : more) f(id);
    }
};

}  // namespace

HcclResult BuildOrder(World *w, std::vector<Node> &order, u32 &numLevels, CheckReport *report)
{
    struct Flat {
        const TaskItem *item;
        int prev;   // previous item of the same thread
        int match;  // for a wait: the record that releases it
        u32 level;
        u32 indeg;
    };
    std::vector<Flat> flat;
    size_t total = 0;
    for (auto &perRank : w->threads) {
        for (auto &t : perRank) total += t->items.size();
    }
    flat.reserve(total);
    for (auto &perRank : w->threads) {
        for (auto &t : perRank) {
            int prev = -1;
            for (const TaskItem &it : t->items) {
                const int id = static_cast<int>(flat.size());
                flat.push_back({&it, prev, -1, 0, 0});
                prev = id;
            }
        }
    }
    // The records of one notify identity in the order they were made: recordAt[first[identity] + n] is the n-th.
    const size_t identities = w->recordSeq.size();
    std::vector<u32> first(identities + 1, 0);
    for (size_t k = 0; k < identities; ++k) first[k + 1] = first[k] + w->recordSeq[k];
    std::vector<int> recordAt(first[identities], -1);
    for (int id = 0; id < static_cast<int>(flat.size()); ++id) {
        const TaskItem &it = *flat[id].item;
        if (it.kind == ItemKind::NOTIFY_RECORD) recordAt[first[it.key] + it.seq] = id;
    }
    std::vector<Succ> succ(flat.size());
    for (int id = 0; id < static_cast<int>(flat.size()); ++id) {
        Flat &f = flat[id];
        if (f.prev >= 0) {
            succ[f.prev].Add(id);
            f.indeg++;
        }
        if (f.item->kind == ItemKind::NOTIFY_WAIT) {
            CHK_PRT_RET(f.item->key >= identities || f.item->seq >= w->recordSeq[f.item->key],
                        HCCL_ERROR("[schedule] a notify wait has no matching record"), HCCL_E_INTERNAL);
            f.match = recordAt[first[f.item->key] + f.item->seq];
            succ[f.match].Add(id);
            f.indeg++;
        }
    }
    std::vector<int> ready;
    for (int id = 0; id < static_cast<int>(flat.size()); ++id) {
        if (flat[id].indeg == 0) ready.push_back(id);
    }
    order.clear();
    numLevels = 0;
    size_t head = 0;
    while (head < ready.size()) {
        const int id = ready[head++];
        const Flat &f = flat[id];
        if (IsDataOp(*f.item)) {
            order.push_back({f.item, f.level});
            numLevels = std::max(numLevels, f.level + 1);
        }
        const u32 out = f.level + (IsDataOp(*f.item) ? 1 : 0);
        succ[id].Each([&](int s) {
            flat[s].level = std::max(flat[s].level, out);
            if (--flat[s].indeg == 0) ready.push_back(s);
        });
    }
    CHK_PRT_RET(head != flat.size(), HCCL_ERROR("[schedule] the recorded handshakes deadlock"), HCCL_E_INTERNAL);
    if (report != nullptr) {
        // data steps, numbered in topological order
        std::vector<int> dataId(flat.size(), -1);
        std::vector<int> dataFlat;
        for (int id : ready) {
            if (IsDataOp(*flat[id].item)) {
                dataId[id] = static_cast<int>(dataFlat.size());
                dataFlat.push_back(id);
            }
        }
        const size_t nd = dataFlat.size();
        report->steps = static_cast<u32>(nd);
        report->levels = numLevels;
        for (int id : dataFlat) (flat[id].item->kind == ItemKind::COPY ? report->copies : report->reduces)++;
        report->exhaustive = nd <= kExhaustiveSteps;
        // reach[id]: the data steps that come after flat node id (bit set), built backwards over the order
        const size_t words = (nd + 63) / 64;
        std::vector<std::vector<uint64_t>> reach;
        if (report->exhaustive) {
            reach.assign(flat.size(), std::vector<uint64_t>(words, 0));
            for (size_t k = ready.size(); k-- > 0;) {
                const int id = ready[k];
                succ[id].Each([&](int sx) {
                    for (size_t wd = 0; wd < words; ++wd) reach[id][wd] |= reach[sx][wd];
                    if (dataId[sx] >= 0) reach[id][dataId[sx] / 64] |= 1ull << (dataId[sx] % 64);
                });
            }
        }
        auto ordered = [&](int a, int b) {   // flat ids of two data steps
            if (!report->exhaustive) return flat[a].level != flat[b].level;
            const int da = dataId[a];
            const int db = dataId[b];
            return ((reach[a][db / 64] >> (db % 64)) & 1ull) != 0 || ((reach[b][da / 64] >> (da % 64)) & 1ull) != 0;
        };
        struct Access {
            u64 lo, hi;
            int id;
            bool write;
        };
        std::vector<Access> acc;
        for (int id : dataFlat) {
            const TaskItem &it = *flat[id].item;
            if (it.bytes == 0) continue;
            // a copy onto itself (the first step of an in-place collective) changes no byte: neither a read
            // nor a write that could race
            if (it.kind == ItemKind::COPY && it.dst == it.src) continue;
            const u64 d = reinterpret_cast<u64>(it.dst);
            const u64 sA = reinterpret_cast<u64>(it.src);
            acc.push_back({d, d + it.bytes, id, true});
            acc.push_back({sA, sA + it.bytes, id, false});
        }
        std::sort(acc.begin(), acc.end(), [](const Access &a, const Access &b) { return a.lo < b.lo; });
        std::vector<size_t> active;
        for (size_t k = 0; k < acc.size(); ++k) {
            size_t keep = 0;
            for (size_t a : active) {
                if (acc[a].hi > acc[k].lo) active[keep++] = a;
            }
            active.resize(keep);
            for (size_t a : active) {
                if (acc[a].id == acc[k].id || (!acc[a].write && !acc[k].write)) continue;
                if (ordered(acc[a].id, acc[k].id)) continue;
                if (report->races++ == 0) {
                    std::ostringstream os;
                    os << "race: steps " << dataId[acc[a].id] << " and " << dataId[acc[k].id]
                       << " are not ordered and overlap at address 0x" << std::hex << std::max(acc[a].lo, acc[k].lo);
                    report->firstProblem = os.str();
                }
            }
            active.push_back(k);
        }
    }
    // by level, steps of one level in the order found above (a counting sort)
    std::vector<u32> at(numLevels + 1, 0);
    for (const Node &nd : order) at[nd.level + 1]++;
    for (u32 l = 0; l < numLevels; ++l) at[l + 1] += at[l];
    std::vector<Node> sorted(order.size());
    for (const Node &nd : order) sorted[at[nd.level]++] = nd;
    order.swap(sorted);
    return HCCL_SUCCESS;
}

// ---------------------------------------------------------------------------------------------------
// STEP mode: every recorded copy / reduce is launched, one fold launch per level and kind
// ---------------------------------------------------------------------------------------------------
// STEP mode: the recorded steps as they are, level by level; the copies of a level are one launch and its
// reduce steps another.  The launches are built as plans so that a repeated collective only replays them.
void BuildStepParts(const std::vector<Node> &order, u32 numLevels, int dtype, int op, std::vector<HostPart> &parts)
{
    size_t i = 0;
    for (u32 level = 0; level < numLevels; ++level) {
        HostPart copies;
        copies.dtype = HCCL_DATA_TYPE_INT8;
        copies.mode = HCCLX_FOLD_CHAIN;
        HostPart reduces;
        reduces.dtype = dtype;
        reduces.op = op;
        reduces.mode = HCCLX_FOLD_CHAIN;
        for (; i < order.size() && order[i].level == level; ++i) {
            const TaskItem &it = *order[i].item;
            hcclx_seg_t s;
            std::memset(&s, 0, sizeof(s));
            if (it.kind == ItemKind::COPY) {
                s.count = it.bytes;
                s.nsrc = 1;
                s.ndst = 1;
                s.src[0] = it.src;
                s.dst[0] = it.dst;
                copies.segs.push_back(s);
            } else {
                s.count = it.count;
                s.nsrc = 2;  // dst = src (+) dst: the accumulator comes first in fold order
                s.ndst = 1;
                s.src[0] = it.dst;
                s.src[1] = it.src;
                s.dst[0] = it.dst;
                reduces.segs.push_back(s);
            }
        }
        if (!copies.segs.empty()) parts.push_back(std::move(copies));
        if (!reduces.segs.empty()) parts.push_back(std::move(reduces));
    }
}


}  // namespace sched
}  // namespace ops_hccl
