// What the pieces of the schedule pipeline share (schedule.h describes the pipeline):
//   schedule_order.cc   recorded steps -> dependency levels, race check; the step-by-step launch lists
//   schedule_fuse.cc    levelled steps -> symbolic trace -> folds -> fused launch lists; closed forms; semantics check
//   plan_cache.cc       keys, the two plan caches, moving a plan to other buffers, launching
//   schedule.cc         RunCollective: selection, rendezvous of streams, the order in which the above is tried
#pragma once
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

#include "hcclx.h"
#include "schedule.h"

namespace ops_hccl {
namespace sched {

// HCCL_VRANK_TIMING=1 prints what each phase of planning a collective took (stderr).
struct PhaseTimer {
    const bool on = std::getenv("HCCL_VRANK_TIMING") != nullptr;
    std::chrono::steady_clock::time_point last = std::chrono::steady_clock::now();
    void Start() { if (on) last = std::chrono::steady_clock::now(); }
    void Lap(const char *what)
    {
        if (!on) return;
        const auto now = std::chrono::steady_clock::now();
        std::fprintf(stderr, "[timing] %-12s %8.3f ms\n", what, std::chrono::duration<double, std::milli>(now - last).count());
        last = now;
    }
};
extern PhaseTimer g_phase;


// ---------------------------------------------------------------------------------------------------
// dependency order of the recorded steps (schedule_order.cc)
// ---------------------------------------------------------------------------------------------------
struct Node {
    const TaskItem *item = nullptr;
    u32 level = 0;
};

// Flattens every thread's items into `order` (a topological order) and gives each data step a level; with `report`
// also looks for data races.  Fails when a wait has no matching record or the handshakes deadlock.
HcclResult BuildOrder(World *w, std::vector<Node> &order, u32 &numLevels, CheckReport *report = nullptr);
// STEP mode: the recorded steps as launch lists, per level the copies and then the reduce steps.
void BuildStepParts(const std::vector<Node> &order, u32 numLevels, int dtype, int op, std::vector<HostPart> &parts);

// ---------------------------------------------------------------------------------------------------
// FUSED mode: symbolic execution (schedule_fuse.cc)
// ---------------------------------------------------------------------------------------------------
// An expression gives a byte stream: value(e, off).  Expression 0 is memory as it was when the collective
// started: value(0, off) = mem[off] (off is an absolute address).  Any other expression is one reduce
// step: value(e, off) = value(src, off + srcShift) (+) value(dst, off + dstShift).
struct Expr {
    int src = -1;
    int dst = -1;
    u64 srcShift = 0;
    u64 dstShift = 0;
};

struct Piece {
    u64 len = 0;
    int expr = 0;
    u64 shift = 0;  // value at address a of the piece = value(expr, a - start + shift)
};

struct Sub {
    u64 start;
    u64 len;
    int expr;
    u64 shift;
};

class Tracer {
public:
    Tracer() { exprs_.push_back(Expr()); }

    void Copy(u64 dst, u64 src, u64 len)
    {
        const std::vector<Sub> from = Lookup(src, len);
        Erase(dst, len);
        for (const Sub &s : from) {
            Piece p;
            p.len = s.len;
            p.expr = s.expr;
            p.shift = s.shift;
            mem_[dst + (s.start - src)] = p;
        }
    }

    void Reduce(u64 dst, u64 src, u64 len)
    {
        const std::vector<Sub> a = Lookup(src, len);
        const std::vector<Sub> b = Lookup(dst, len);
        Erase(dst, len);
        size_t ia = 0;
        size_t ib = 0;
        u64 off = 0;
        while (off < len) {
            const Sub &sa = a[ia];
            const Sub &sb = b[ib];
            const u64 endA = sa.start - src + sa.len;
            const u64 endB = sb.start - dst + sb.len;
            const u64 end = std::min(endA, endB);
            Expr e;
            e.src = sa.expr;
            e.srcShift = sa.shift + (off - (sa.start - src));
            e.dst = sb.expr;
            e.dstShift = sb.shift + (off - (sb.start - dst));
            exprs_.push_back(e);
            Piece p;
            p.len = end - off;
            p.expr = static_cast<int>(exprs_.size()) - 1;
            p.shift = 0;
            mem_[dst + off] = p;
            off = end;
            if (off == endA) ++ia;
            if (off == endB) ++ib;
        }
    }

    // The pieces that cover [addr, addr + len): written ranges as recorded, untouched ranges as memory.
    std::vector<Sub> Lookup(u64 addr, u64 len) const
    {
        std::vector<Sub> out;
        u64 cur = addr;
        const u64 end = addr + len;
        auto it = mem_.upper_bound(addr);
        if (it != mem_.begin()) {
            auto pv = std::prev(it);
            if (pv->first + pv->second.len > addr) it = pv;
        }
        while (cur < end) {
            if (it == mem_.end() || it->first >= end) {
                out.push_back({cur, end - cur, 0, cur});
                break;
            }
            if (it->first > cur) {
                out.push_back({cur, it->first - cur, 0, cur});
                cur = it->first;
            }
            const u64 pEnd = std::min(end, it->first + it->second.len);
            out.push_back({cur, pEnd - cur, it->second.expr, it->second.shift + (cur - it->first)});
            cur = pEnd;
            ++it;
        }
        return out;
    }

    const Expr &At(int e) const { return exprs_[e]; }
    // A reduce step that no memory piece holds yet (closed forms build their trees from these).
    int AddExpr(const Expr &e)
    {
        exprs_.push_back(e);
        return static_cast<int>(exprs_.size()) - 1;
    }

private:
    void Split(u64 addr)
    {
        auto it = mem_.upper_bound(addr);
        if (it == mem_.begin()) return;
        --it;
        if (it->first < addr && it->first + it->second.len > addr) {
            Piece tail = it->second;
            const u64 cut = addr - it->first;
            tail.len -= cut;
            tail.shift += cut;
            it->second.len = cut;
            mem_[addr] = tail;
        }
    }

    void Erase(u64 addr, u64 len)
    {
        Split(addr);
        Split(addr + len);
        mem_.erase(mem_.lower_bound(addr), mem_.lower_bound(addr + len));
    }

    std::map<u64, Piece> mem_;
    std::vector<Expr> exprs_;
};

// One output piece flattened to a fold: source addresses in fold order.
struct Fold {
    std::vector<u64> src;
    std::vector<u64> dsts;    // every output piece that holds this value
    u64 bytes = 0;
    bool chain = true;        // false: a tree that no chain reproduces
    bool fits = true;         // false: a tree too large for the tree kernels
    u32 levels = 0;           // tree: levels below the root
    std::vector<u8> prog;     // tree: (dst register, src register) per step over src[] as registers;
                              // chain: empty, or one byte per source, non-zero = that step is acc (+) src
};

// The ranks' input buffers sorted by address, to find the one an address lies in without walking all ranks.
struct InputRanges {
    struct Range {
        u64 base;
        u64 size;
        u32 rank;
    };
    std::vector<Range> sorted;
    u64 longest = 1;   // no buffer that starts more than this below an address can hold it
    explicit InputRanges(const std::vector<OpParam> &params)
    {
        for (size_t r = 0; r < params.size(); ++r) {
            sorted.push_back({reinterpret_cast<u64>(params[r].inputPtr), params[r].inputSize, static_cast<u32>(r)});
            longest = std::max<u64>(longest, params[r].inputSize);
        }
        std::sort(sorted.begin(), sorted.end(), [](const Range &a, const Range &b) { return a.base < b.base; });
    }
    // The input buffer that holds [addr, addr + bytes), or nullptr.  Buffers that start at or below addr are
    // tried from the nearest one down (in-place and overlapping operands may nest).
    const Range *Find(u64 addr, u64 bytes) const
    {
        auto it = std::upper_bound(sorted.begin(), sorted.end(), addr,
                                   [](u64 v, const Range &x) { return v < x.base; });
        while (it != sorted.begin()) {
            --it;
            if (it->base + longest <= addr) break;
            if (addr + bytes <= it->base + it->size) return &*it;
        }
        return nullptr;
    }
};

struct FusedPlan {
    std::vector<hcclx_seg_t> chainSegs;
    std::vector<hcclx_seg_t> selfSegs;
    std::vector<hcclx_seg_t> copySegs;
    std::vector<hcclx_seg_t> treeSegs;
    std::vector<hcclx_wide_seg_t> wideSegs;       // chains over more than HCCLX_MAX_FAN sources
    std::vector<hcclx_wide_seg_t> wideTreeSegs;   // trees with more leaves or levels than the 16-slot kernel holds
    std::vector<hcclx_wide_seg_t> wideSelfSegs;   // the per-rank orders of the one-shot templates among 17 .. 64 ranks
    // The same in place (outputs overwrite inputs): the wide kernel computes its outputs sixteen at a time in
    // different workgroups, so they go to a staging buffer first (dst[] hold byte offsets into it) and are copied
    // to their places by a second launch.
    struct StagedCopy {
        u64 offset;
        u64 dst;
        u64 bytes;
    };
    std::vector<hcclx_wide_seg_t> stagedSelfSegs;
    std::vector<StagedCopy> stagedCopies;
    u64 stagingBytes = 0;
};

// Output pieces beyond which a schedule is run step by step instead of being fused.
constexpr size_t kMaxFusedPieces = 400000;


// The folds of a traced schedule: one per distinct value among the output pieces.  Returns false when the schedule
// cannot be fused (a floating-point tree with more than six levels or 64 leaves, or too many pieces).
bool FoldsFromTrace(const Tracer &tr, const std::vector<OpParam> &params, int dtype, int op, std::vector<Fold> &folds,
                    std::string *text);
// The folds of a collective that its executor and template state in closed form, and, with `text`, the trace they
// stand for.
bool FoldsFromClosedForm(const std::vector<ClosedFold> &closed, const std::vector<OpParam> &params, int dtype, int op,
                         std::vector<Fold> &folds, std::string *text);
// The fused launch lists of the folds; false when they cannot run as one pass.  `stated`: the folds come from a
// closed form (their sources are input pieces and no two of them are the same value).
bool BuildFusedPlan(const std::vector<OpParam> &params, std::vector<Fold> &folds, u32 esz, FusedPlan &plan,
                    bool stated = false);
// Every output piece against the contract of the collective.
void CheckSemantics(const Tracer &tr, const std::vector<OpParam> &params, CheckReport &rep);

// ---------------------------------------------------------------------------------------------------
// plans and their caches (plan_cache.cc)
// ---------------------------------------------------------------------------------------------------
std::vector<u64> ShapeKey(const std::vector<OpParam> &params, const std::string &alg, u64 cclBytes);
std::vector<u64> PlanKey(const std::vector<u64> &shape, const std::vector<OpParam> &params);
bool BuffersAreSeparate(const std::vector<OpParam> &params);
void Rebase(const ShapePlan &sp, const std::vector<OpParam> &params, std::vector<HostPart> &parts);
HcclResult CreatePlans(const std::vector<HostPart> &parts, std::vector<hcclx_plan *> &plans);
HcclResult LaunchParts(World *w, const std::vector<HostPart> &parts, void *stream);
HcclResult LaunchPlans(World *w, const std::vector<hcclx_plan *> &plans, void *stream);
void DropPlans(std::vector<hcclx_plan *> &plans, std::vector<void *> &buffers);
u64 HashKey(const std::vector<u64> &key);
void ReapRetired(PlanCache &cache, bool wait);
CachedPlan *FindPlan(PlanCache &cache, const std::vector<u64> &key);
ShapePlan *FindShape(PlanCache &cache, const std::vector<u64> &shape);
bool SeenBefore(PlanCache &cache, u64 hash);
void KeepShape(PlanCache &cache, const std::vector<u64> &shape, std::vector<HostPart> &&parts,
               const std::vector<OpParam> &params, bool fused, u32 levels, u32 segments);
HcclResult LaunchAndKeep(World *w, CachedPlan &&c, void *stream);

}  // namespace sched
}  // namespace ops_hccl
