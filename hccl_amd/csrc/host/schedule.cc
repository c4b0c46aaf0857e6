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

namespace {

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
PhaseTimer g_phase;

bool IsDataOp(const TaskItem &it) { return it.kind == ItemKind::COPY || it.kind == ItemKind::REDUCE; }

// ---------------------------------------------------------------------------------------------------
// dependency order of the recorded steps
// ---------------------------------------------------------------------------------------------------
struct Node {
    const TaskItem *item = nullptr;
    u32 level = 0;
};

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

HcclResult BuildOrder(World *w, std::vector<Node> &order, u32 &numLevels, CheckReport *report = nullptr)
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

// ---------------------------------------------------------------------------------------------------
// FUSED mode: symbolic execution
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

bool IsFloatType(int dt)
{
    return dt == HCCL_DATA_TYPE_FP16 || dt == HCCL_DATA_TYPE_FP32 || dt == HCCL_DATA_TYPE_FP64 ||
           dt == HCCL_DATA_TYPE_BFP16;
}

void CollectLeaves(const Tracer &tr, int e, u64 shift, std::vector<u64> &out)
{
    if (e == 0) {
        out.push_back(shift);
        return;
    }
    const Expr &x = tr.At(e);
    CollectLeaves(tr, x.dst, shift + x.dstShift, out);
    CollectLeaves(tr, x.src, shift + x.srcShift, out);
}

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

// An input byte as the trace names it: "x<rank>@<offset>", the lowest rank whose input holds the address, as a
// reader of the trace expects for shared buffers.
std::string LeafText(u64 addr, const InputRanges &inputs)
{
    const InputRanges::Range *best = nullptr;
    auto it = std::upper_bound(inputs.sorted.begin(), inputs.sorted.end(), addr,
                               [](u64 v, const InputRanges::Range &x) { return v < x.base; });
    while (it != inputs.sorted.begin()) {
        --it;
        if (it->base + inputs.longest <= addr) break;
        if (addr < it->base + std::max<u64>(it->size, 1) && (best == nullptr || it->rank < best->rank)) best = &*it;
    }
    if (best == nullptr) return "?";
    return "x" + std::to_string(best->rank) + "@" + std::to_string(addr - best->base);
}

std::string ExprText(const Tracer &tr, int e, u64 shift, const InputRanges &inputs)
{
    if (e == 0) return LeafText(shift, inputs);
    const Expr &x = tr.At(e);
    return "(" + ExprText(tr, x.src, shift + x.srcShift, inputs) + "+" + ExprText(tr, x.dst, shift + x.dstShift, inputs) +
           ")";
}

// Post-order walk of a tree expression: leaves are numbered dst side first, so the value of every node
// ends up in the register of its left-most leaf and the root in register 0.  Returns that register and
// the number of levels below the node through *levels.
u32 EmitTree(const Tracer &tr, int e, u64 shift, Fold &f, u32 *levels)
{
    if (e == 0) {
        f.src.push_back(shift);
        *levels = 0;
        return static_cast<u32>(f.src.size()) - 1;
    }
    const Expr &x = tr.At(e);
    u32 ld = 0;
    u32 ls = 0;
    const u32 rd = EmitTree(tr, x.dst, shift + x.dstShift, f, &ld);
    const u32 rs = EmitTree(tr, x.src, shift + x.srcShift, f, &ls);
    f.prog.push_back(static_cast<u8>(rd));
    f.prog.push_back(static_cast<u8>(rs));
    *levels = std::max(ld, ls) + 1;
    return rd;
}

// Turns the expression of a piece into a fold.  A left-deep spine "leaf (+) acc" is a chain as it
// stands.  Integer arithmetic (wrap-around sum and product, max, min) is associative and commutative, so
// any tree equals the chain of its leaves.  For floating types IEEE addition and multiplication are
// commutative but not associative: "acc (+) leaf" still equals "leaf (+) acc" bit for bit (NaN payloads
// aside), other tree shapes do not flatten; max/min additionally depend on operand order for NaN and
// signed zeros: there a step "acc (+) leaf" is marked, and the chain kernels swap its operands.
Fold Flatten(const Tracer &tr, int e, u64 shift, int dtype, int op)
{
    Fold f;
    if (!IsFloatType(dtype)) {
        CollectLeaves(tr, e, shift, f.src);
        return f;
    }
    const bool commutes = (op == HCCL_REDUCE_SUM || op == HCCL_REDUCE_PROD);
    std::vector<u64> rev;  // leaves from the outermost step inwards
    std::vector<u8> revSwap;
    bool anySwap = false;
    int cur = e;
    u64 sh = shift;
    while (cur != 0) {
        const Expr &x = tr.At(cur);
        if (x.src == 0) {
            rev.push_back(sh + x.srcShift);
            revSwap.push_back(0);
            sh += x.dstShift;
            cur = x.dst;
        } else if (x.dst == 0) {
            rev.push_back(sh + x.dstShift);
            revSwap.push_back(commutes ? 0 : 1);
            anySwap = anySwap || !commutes;
            sh += x.srcShift;
            cur = x.src;
        } else {
            // not a spine: keep the tree as it is, for the kernels that evaluate trees of up to four levels
            // (six in the wide kernel) in registers
            f.chain = false;
            u32 levels = 0;
            (void)EmitTree(tr, e, shift, f, &levels);
            f.levels = levels;
            f.fits = (f.src.size() <= HCCLX_MAX_WIDE_FAN && levels <= 6);
            return f;
        }
    }
    f.src.push_back(sh);
    for (auto it = rev.rbegin(); it != rev.rend(); ++it) f.src.push_back(*it);
    if (anySwap) {
        f.prog.push_back(0);
        for (auto it = revSwap.rbegin(); it != revSwap.rend(); ++it) f.prog.push_back(*it);
    }
    return f;
}

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

bool Overlaps(u64 a, u64 alen, u64 b, u64 blen) { return a < b + blen && b < a + alen; }

// The folds of a traced schedule: one per distinct value among the output pieces.  Returns false when the schedule
// cannot be fused (a floating-point tree with more than six levels or 64 leaves, or too many pieces).
bool FoldsFromTrace(const Tracer &tr, const std::vector<OpParam> &params, int dtype, int op, std::vector<Fold> &folds,
                    std::string *text)
{
    // One fold per distinct value: output pieces that hold the same expression (the copies an AllReduce hands to
    // every rank) are destinations of one fold, flattened once.
    struct PieceKey {
        int expr;
        u64 shift, len;
        bool operator==(const PieceKey &o) const { return expr == o.expr && shift == o.shift && len == o.len; }
    };
    struct PieceHash {
        size_t operator()(const PieceKey &k) const
        {
            u64 h = static_cast<u64>(k.expr) * 0x9E3779B97F4A7C15ull;
            h ^= (k.shift + 0x9E3779B97F4A7C15ull + (h << 6) + (h >> 2));
            h ^= (k.len + 0x9E3779B97F4A7C15ull + (h << 6) + (h >> 2));
            return static_cast<size_t>(h);
        }
    };
    std::unordered_map<PieceKey, size_t, PieceHash> byPiece;
    bool allFit = true;
    size_t pieces = 0;
    const InputRanges inputs(params);
    for (size_t r = 0; r < params.size(); ++r) {
        const u64 out = reinterpret_cast<u64>(params[r].outputPtr);
        if (params[r].outputSize == 0) continue;
        for (const Sub &s : tr.Lookup(out, params[r].outputSize)) {
            if (s.expr == 0 && s.shift == s.start) continue;  // never written: stays as it is
            if (text) {
                std::ostringstream os;
                os << "rank " << r << " out[" << (s.start - out) << "," << s.len << ") = "
                   << ExprText(tr, s.expr, s.shift, inputs) << "\n";
                *text += os.str();
            }
            if (++pieces > kMaxFusedPieces) return false;   // more pieces than one pass is worth planning for
            auto found = byPiece.emplace(PieceKey{s.expr, s.shift, s.len}, folds.size());
            if (found.second) {
                Fold f = Flatten(tr, s.expr, s.shift, dtype, op);
                f.bytes = s.len;
                if (!f.fits) allFit = false;
                folds.push_back(std::move(f));
            }
            folds[found.first->second].dsts.push_back(s.start);
        }
    }
    g_phase.Lap(" flatten");
    return allFit;
}

// The folds of a collective that its executor and template state in closed form, and, with `text`, the trace they
// stand for: the same lines the recorded steps give when traced.
void FoldsFromClosedForm(const std::vector<ClosedFold> &closed, const std::vector<OpParam> &params, std::vector<Fold> &folds,
                         std::string *text)
{
    const InputRanges inputs(params);
    struct Line {
        u32 rank;
        u64 offset;
        size_t fold;
    };
    std::vector<Line> lines;
    folds.reserve(closed.size());
    for (const ClosedFold &c : closed) {
        Fold f;
        f.bytes = c.bytes;
        for (const ClosedFold::Ref &s : c.src) f.src.push_back(reinterpret_cast<u64>(params[s.rank].inputPtr) + s.offset);
        for (const ClosedFold::Ref &d : c.dst) {
            f.dsts.push_back(reinterpret_cast<u64>(params[d.rank].outputPtr) + d.offset);
            if (text) lines.push_back({d.rank, d.offset, folds.size()});
        }
        folds.push_back(std::move(f));
    }
    if (text == nullptr) return;
    std::sort(lines.begin(), lines.end(),
              [](const Line &a, const Line &b) { return a.rank != b.rank ? a.rank < b.rank : a.offset < b.offset; });
    for (const Line &l : lines) {
        const Fold &f = folds[l.fold];
        std::string expr = LeafText(f.src[0], inputs);
        for (size_t k = 1; k < f.src.size(); ++k) expr = "(" + LeafText(f.src[k], inputs) + "+" + expr + ")";
        std::ostringstream os;
        os << "rank " << l.rank << " out[" << l.offset << "," << f.bytes << ") = " << expr << "\n";
        *text += os.str();
    }
}

// Builds the fused launch plan from the folds.  Returns false when they cannot run as one pass (a source that is
// not an input, or an output that overlaps another fold's source); the caller then runs the steps one by one.
bool BuildFusedPlan(const std::vector<OpParam> &params, std::vector<Fold> &folds, u32 esz, FusedPlan &plan)
{
    const InputRanges inputs(params);
    // every source must be input data (or an output that the same fold overwrites in place)
    for (const Fold &f : folds) {
        for (u64 a : f.src) {
            if (inputs.Find(a, f.bytes) == nullptr) return false;
        }
    }
    // Different expressions may still read the same sources in the same order (pieces that were reduced by
    // different steps of equal shape): they become one fold with all the destinations.
    {
        std::map<std::vector<u64>, size_t> bySrc;
        std::vector<Fold> merged;
        for (Fold &f : folds) {
            std::vector<u64> key = f.src;
            key.push_back(f.bytes);
            for (u8 b : f.prog) key.push_back(b);  // same sources, different tree: different value
            auto found = bySrc.emplace(std::move(key), merged.size());
            if (found.second) {
                merged.push_back(std::move(f));
            } else {
                Fold &into = merged[found.first->second];
                into.dsts.insert(into.dsts.end(), f.dsts.begin(), f.dsts.end());
            }
        }
        folds.swap(merged);
    }
    g_phase.Lap(" bysrc");
    // Find groups of N single-destination folds over the same N sources where fold j starts from source j and then
    // takes the others in a common order: the per-rank order of the one-shot templates, computed in one pass.
    std::map<std::vector<u64>, std::vector<size_t>> bySet;
    for (size_t i = 0; i < folds.size(); ++i) {
        const Fold &f = folds[i];
        if (f.dsts.size() != 1) continue;
        if (!f.chain || !f.prog.empty() || f.src.size() < 2 || f.src.size() > HCCLX_MAX_WIDE_FAN) continue;
        std::vector<u64> key = f.src;
        std::sort(key.begin(), key.end());
        key.push_back(f.bytes);
        bySet[key].push_back(i);
    }
    std::vector<bool> taken(folds.size(), false);
    std::vector<bool> staged(folds.size(), false);   // written by the second launch: cannot race with what the first reads
    std::vector<int> group(folds.size(), -1);
    for (auto &kv : bySet) {
        const std::vector<size_t> &grp = kv.second;
        const size_t n = folds[grp[0]].src.size();
        if (grp.size() != n || n < 2) continue;
        for (size_t cand : grp) {  // the fold whose own source comes first in the common order
            const std::vector<u64> &base = folds[cand].src;
            std::vector<int> owner(n, -1);
            bool ok = true;
            for (size_t g : grp) {
                const std::vector<u64> &s = folds[g].src;
                size_t j = 0;
                while (j < n && base[j] != s[0]) ++j;
                if (j == n || owner[j] != -1) {
                    ok = false;
                    break;
                }
                size_t pos = 1;
                for (size_t k = 0; k < n && ok; ++k) {
                    if (k == j) continue;
                    if (s[pos++] != base[k]) ok = false;
                }
                if (!ok) break;
                owner[j] = static_cast<int>(g);
            }
            if (!ok) continue;
            if (n > HCCLX_MAX_FAN) {
                // the wide kernel computes the outputs sixteen at a time in different workgroups, so none of
                // them may overwrite a source: an in-place collective writes to a staging buffer first
                bool clash = false;
                for (size_t j = 0; j < n && !clash; ++j) {
                    for (size_t k = 0; k < n && !clash; ++k) {
                        clash = Overlaps(folds[owner[j]].dsts[0], folds[owner[j]].bytes, base[k], folds[cand].bytes);
                    }
                }
                hcclx_wide_seg_t seg;
                std::memset(&seg, 0, sizeof(seg));
                seg.count = folds[cand].bytes / esz;
                seg.nsrc = static_cast<uint32_t>(n);
                seg.ndst = static_cast<uint32_t>(n);
                for (size_t j = 0; j < n; ++j) {
                    const Fold &fj = folds[owner[j]];
                    seg.src[j] = reinterpret_cast<const void *>(base[j]);
                    seg.dst[j] = reinterpret_cast<void *>(fj.dsts[0]);
                    taken[owner[j]] = true;
                    if (clash) {
                        seg.dst[j] = reinterpret_cast<void *>(plan.stagingBytes);
                        plan.stagedCopies.push_back({plan.stagingBytes, fj.dsts[0], fj.bytes});
                        plan.stagingBytes += (fj.bytes + 255) & ~static_cast<u64>(255);
                        staged[owner[j]] = true;
                    }
                }
                if (clash) {
                    plan.stagedSelfSegs.push_back(seg);
                    break;
                }
                plan.wideSelfSegs.push_back(seg);
                break;
            }
            hcclx_seg_t seg;
            std::memset(&seg, 0, sizeof(seg));
            seg.count = folds[cand].bytes / esz;
            seg.nsrc = static_cast<uint32_t>(n);
            seg.ndst = static_cast<uint32_t>(n);
            for (size_t j = 0; j < n; ++j) {
                seg.src[j] = reinterpret_cast<const void *>(base[j]);
                seg.dst[j] = reinterpret_cast<void *>(folds[owner[j]].dsts[0]);
                taken[owner[j]] = true;
                group[owner[j]] = static_cast<int>(plan.selfSegs.size());
            }
            plan.selfSegs.push_back(seg);
            break;
        }
    }
    g_phase.Lap(" selfgroups");
    // A destination may coincide exactly with a source of its own fold, or of a fold of the same
    // self-first group (every thread reads all sources of an element before it writes any destination):
    // that is an in-place collective.  Any other overlap between what one fold writes and what another
    // reads would be a race inside a single pass.
    // Every source lies in a rank's input and every destination in a rank's output: when no output buffer touches
    // an input buffer there is nothing to look for.
    bool apart = true;
    for (size_t r = 0; r < params.size() && apart; ++r) {
        if (params[r].outputSize == 0) continue;
        const u64 lo = reinterpret_cast<u64>(params[r].outputPtr);
        const u64 hi = lo + params[r].outputSize;
        for (const InputRanges::Range &in : inputs.sorted) {
            if (in.base >= hi) break;
            if (in.size != 0 && in.base + in.size > lo) {
                apart = false;
                break;
            }
        }
    }
    if (!apart) {
        struct Read {
            u64 addr;
            u64 bytes;
            size_t fold;
        };
        std::vector<Read> reads;
        u64 longest = 0;
        for (size_t j = 0; j < folds.size(); ++j) {
            for (u64 a : folds[j].src) reads.push_back({a, folds[j].bytes, j});
            longest = std::max(longest, folds[j].bytes);
        }
        std::sort(reads.begin(), reads.end(), [](const Read &x, const Read &y) { return x.addr < y.addr; });
        for (size_t i = 0; i < folds.size(); ++i) {
            if (staged[i]) continue;
            for (u64 dst : folds[i].dsts) {
                // reads that can reach into [dst, dst + bytes) start after dst - longest
                const u64 from = dst > longest ? dst - longest : 0;
                auto it = std::lower_bound(reads.begin(), reads.end(), from,
                                           [](const Read &x, u64 v) { return x.addr < v; });
                for (; it != reads.end() && it->addr < dst + folds[i].bytes; ++it) {
                    if (!Overlaps(dst, folds[i].bytes, it->addr, it->bytes)) continue;
                    const size_t j = it->fold;
                    const bool sameUnit = (i == j) || (group[i] != -1 && group[i] == group[j]);
                    if (sameUnit && it->addr == dst) continue;
                    return false;
                }
            }
        }
    }
    g_phase.Lap(" overlaps");
    for (size_t i = 0; i < folds.size(); ++i) {
        if (taken[i]) continue;
        const Fold &f = folds[i];
        if (f.src.size() > HCCLX_MAX_FAN || (1u << f.levels) > HCCLX_MAX_FAN) {
            // more ranks than the register-resident kernels take: the wide kernels
            if (f.src.size() > HCCLX_MAX_WIDE_FAN) return false;
            for (size_t at = 0; at < f.dsts.size(); at += HCCLX_MAX_WIDE_FAN) {
                hcclx_wide_seg_t seg;
                std::memset(&seg, 0, sizeof(seg));
                seg.count = f.bytes / esz;
                seg.nsrc = static_cast<uint32_t>(f.src.size());
                for (size_t k = 0; k < f.src.size(); ++k) seg.src[k] = reinterpret_cast<const void *>(f.src[k]);
                for (size_t d = at; d < f.dsts.size() && d < at + HCCLX_MAX_WIDE_FAN; ++d) {
                    seg.dst[seg.ndst++] = reinterpret_cast<void *>(f.dsts[d]);
                }
                if (f.chain) {
                    if (!f.prog.empty()) std::memcpy(seg.prog, f.prog.data(), f.prog.size());
                    plan.wideSegs.push_back(seg);
                } else {
                    std::memcpy(seg.prog, f.prog.data(), f.prog.size());
                    plan.wideTreeSegs.push_back(seg);
                }
            }
            continue;
        }
        for (size_t at = 0; at < f.dsts.size(); at += HCCLX_MAX_FAN) {
            hcclx_seg_t seg;
            std::memset(&seg, 0, sizeof(seg));
            seg.nsrc = static_cast<uint32_t>(f.src.size());
            for (size_t k = 0; k < f.src.size(); ++k) seg.src[k] = reinterpret_cast<const void *>(f.src[k]);
            for (size_t d = at; d < f.dsts.size() && d < at + HCCLX_MAX_FAN; ++d) {
                seg.dst[seg.ndst++] = reinterpret_cast<void *>(f.dsts[d]);
            }
            if (f.src.size() == 1) {
                seg.count = f.bytes;  // a copy: counted in bytes
                plan.copySegs.push_back(seg);
            } else if (!f.chain) {
                seg.count = f.bytes / esz;
                std::memcpy(seg.prog, f.prog.data(), f.prog.size());
                plan.treeSegs.push_back(seg);
            } else {
                seg.count = f.bytes / esz;
                if (!f.prog.empty()) std::memcpy(seg.prog, f.prog.data(), f.prog.size());
                plan.chainSegs.push_back(seg);
            }
        }
    }
    return true;
}

// Every output piece against the contract of the collective (what the reference's semantics checkers
// demand of a recorded task list: test/st/algorithm/utils/src/hccl_verifier/semantics_check/).
void CheckSemantics(const Tracer &tr, const std::vector<OpParam> &params, CheckReport &rep)
{
    const u32 n = static_cast<u32>(params.size());
    const HcclCMDType type = params[0].opType;
    auto problem = [&](u32 rank, u64 off, const std::string &what) {
        if (rep.semanticErrors++ == 0 && rep.firstProblem.empty()) {
            std::ostringstream os;
            os << "rank " << rank << " output byte " << off << ": " << what;
            rep.firstProblem = os.str();
        }
    };
    auto inputOf = [&](u64 addr, u32 &rank, u64 &off) {
        for (u32 k = 0; k < n; ++k) {
            const u64 base = reinterpret_cast<u64>(params[k].inputPtr);
            if (addr >= base && addr < base + std::max<u64>(params[k].inputSize, 1)) {
                rank = k;
                off = addr - base;
                return true;
            }
        }
        return false;
    };
    const bool reduceOp = type == HcclCMDType::HCCL_CMD_ALLREDUCE || type == HcclCMDType::HCCL_CMD_REDUCE_SCATTER ||
                          type == HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V;
    for (u32 r = 0; r < n; ++r) {
        const OpParam &p = params[r];
        const u64 out = reinterpret_cast<u64>(p.outputPtr);
        const u64 esz = reduceOp ? DATATYPE_SIZE_TABLE[p.DataDes.dataType] : 1;
        // expected source of output byte `off`: rank (or every rank for a reduction) and input offset;
        // false = this byte is not part of the result and must stay untouched
        auto expect = [&](u64 off, u32 &srcRank, u64 &srcOff) {
            switch (type) {
                case HcclCMDType::HCCL_CMD_ALLREDUCE:
                    srcOff = off;
                    return off < p.DataDes.count * esz;
                case HcclCMDType::HCCL_CMD_REDUCE_SCATTER:
                    srcOff = r * p.outputSize + off;
                    return true;
                case HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V:
                    srcOff = p.vDataDes.displs[r] * esz + off;
                    return off < p.vDataDes.counts[r] * esz;
                case HcclCMDType::HCCL_CMD_ALLGATHER:
                    srcRank = static_cast<u32>(off / p.inputSize);
                    srcOff = off % p.inputSize;
                    return true;
                case HcclCMDType::HCCL_CMD_ALLGATHER_V: {
                    const u64 ez = DATATYPE_SIZE_TABLE[p.vDataDes.dataType];
                    for (u32 k = 0; k < n; ++k) {
                        const u64 lo = p.vDataDes.displs[k] * ez;
                        if (off >= lo && off < lo + p.vDataDes.counts[k] * ez) {
                            srcRank = k;
                            srcOff = off - lo;
                            return true;
                        }
                    }
                    return false;
                }
                default: {   // the AlltoAll family
                    const u64 ez = DATATYPE_SIZE_TABLE[p.all2AllVDataDes.recvType];
                    for (u32 k = 0; k < n; ++k) {
                        const u64 lo = p.all2AllVDataDes.rdispls[k] * ez;
                        if (off >= lo && off < lo + p.all2AllVDataDes.recvCounts[k] * ez) {
                            srcRank = k;
                            srcOff = params[k].all2AllVDataDes.sdispls[r] * ez + (off - lo);
                            return true;
                        }
                    }
                    return false;
                }
            }
        };
        for (const Sub &s : tr.Lookup(out, std::max<u64>(p.outputSize, 0))) {
            const u64 off = s.start - out;
            const bool untouched = (s.expr == 0 && s.shift == s.start);
            // a piece is uniform only if the expectation does not change inside it: test both ends
            for (u64 probe : {off, off + s.len - 1}) {
                u32 wantRank = 0;
                u64 wantOff = 0;
                const bool part = expect(probe, wantRank, wantOff);
                const u64 delta = probe - off;
                if (!part) {
                    if (!untouched) problem(r, probe, "written, but not part of the result");
                    continue;
                }
                if (untouched) {
                    // in place: the byte already holds the right input only for a copy from the same address
                    u32 k = 0;
                    u64 o = 0;
                    if (!reduceOp && inputOf(s.start + delta, k, o) && k == wantRank && o == wantOff) continue;
                    problem(r, probe, "never written");
                    continue;
                }
                std::vector<u64> leaves;
                CollectLeaves(tr, s.expr, s.shift + delta, leaves);
                if (!reduceOp) {
                    u32 k = 0;
                    u64 o = 0;
                    if (leaves.size() != 1 || !inputOf(leaves[0], k, o) || k != wantRank || o != wantOff) {
                        problem(r, probe, "copied from the wrong place");
                    }
                    continue;
                }
                std::vector<u32> seen(n, 0);
                bool ok = leaves.size() == n;
                for (u64 a : leaves) {
                    u32 k = 0;
                    u64 o = 0;
                    if (!inputOf(a, k, o) || o != wantOff) {
                        ok = false;
                        break;
                    }
                    seen[k]++;
                }
                for (u32 k = 0; k < n && ok; ++k) ok = seen[k] == 1;
                if (!ok) problem(r, probe, "not the reduction of every rank's element at the matching offset");
            }
        }
    }
}

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

// Moves the pointers of a shape plan's parts from the buffers it was made for to those of `params`.  Pointers
// outside the ranks' buffers (the scratch buffers of step plans, which belong to the world) stay.
void Rebase(const ShapePlan &sp, const std::vector<OpParam> &params, std::vector<HostPart> &parts)
{
    struct Move {
        u64 lo, hi;
        int64_t delta;
    };
    std::vector<Move> moves;
    for (size_t r = 0; r < params.size(); ++r) {
        const ShapePlan::Buffer &in = sp.buffers[2 * r];
        const ShapePlan::Buffer &out = sp.buffers[2 * r + 1];
        const u64 newIn = reinterpret_cast<u64>(params[r].inputPtr);
        const u64 newOut = reinterpret_cast<u64>(params[r].outputPtr);
        if (in.base == out.base) {   // in place: one buffer, as long as the longer of the two
            const u64 size = std::max(in.size, out.size);
            if (size) moves.push_back({in.base, in.base + size, static_cast<int64_t>(newIn - in.base)});
            continue;
        }
        if (in.size) moves.push_back({in.base, in.base + in.size, static_cast<int64_t>(newIn - in.base)});
        if (out.size) moves.push_back({out.base, out.base + out.size, static_cast<int64_t>(newOut - out.base)});
    }
    std::sort(moves.begin(), moves.end(), [](const Move &a, const Move &b) { return a.lo < b.lo; });
    auto shift = [&](const void *p) -> void * {
        const u64 a = reinterpret_cast<u64>(p);
        auto it = std::upper_bound(moves.begin(), moves.end(), a, [](u64 v, const Move &m) { return v < m.lo; });
        if (it == moves.begin()) return const_cast<void *>(p);
        --it;
        return a < it->hi ? reinterpret_cast<void *>(a + it->delta) : const_cast<void *>(p);
    };
    parts = sp.parts;
    for (HostPart &hp : parts) {
        for (hcclx_seg_t &g : hp.segs) {
            for (uint32_t k = 0; k < g.nsrc; ++k) g.src[k] = shift(g.src[k]);
            for (uint32_t k = 0; k < g.ndst; ++k) g.dst[k] = shift(g.dst[k]);
        }
        for (hcclx_wide_seg_t &g : hp.wideSegs) {
            for (uint32_t k = 0; k < g.nsrc; ++k) g.src[k] = shift(g.src[k]);
            for (uint32_t k = 0; k < g.ndst; ++k) g.dst[k] = shift(g.dst[k]);
        }
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
    w->lastLaunches = 0;
    for (const HostPart &hp : parts) {
        const int rc = hp.wide ? hcclx_fold_wide(hp.wideSegs.data(), static_cast<uint32_t>(hp.wideSegs.size()), hp.dtype, hp.op,
                                                 hp.mode, stream)
                               : hcclx_fold(hp.segs.data(), static_cast<uint32_t>(hp.segs.size()), hp.dtype, hp.op, hp.mode,
                                            stream);
        if (rc != HCCL_SUCCESS) return static_cast<HcclResult>(rc);
        w->lastLaunches++;
    }
    return HCCL_SUCCESS;
}

HcclResult LaunchPlans(World *w, const std::vector<hcclx_plan *> &plans, void *stream)
{
    w->lastLaunches = 0;
    for (hcclx_plan *p : plans) {
        const int rc = hcclx_plan_launch(p, stream);
        if (rc != HCCL_SUCCESS) return static_cast<HcclResult>(rc);
        w->lastLaunches++;
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
    w->lastLaunches = 1;
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
    if (w->dryRun) return RunCollectiveOnStream(w, params);
    hipStream_t launch = static_cast<hipStream_t>(params[w->rankSize - 1].stream);
    CHK_RET(JoinStreams(params, launch, true));
    const HcclResult res = RunCollectiveOnStream(w, params);
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
            if (!SeenBefore(cache, HashKey(key))) return LaunchParts(w, parts, stream);
            // these buffers have come by before: they are worth tables of their own in device memory
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
            FoldsFromClosedForm(closed, params, folds, text);
            haveFolds = true;
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
            ok = FoldsFromTrace(tr, params, foldType, op, folds, text);
        }
        FusedPlan plan;
        ok = ok && BuildFusedPlan(params, folds, esz, plan);
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
