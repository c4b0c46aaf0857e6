// Levelled steps -> symbolic trace -> folds -> fused launch lists; closed forms; the semantics check.
#include <algorithm>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "schedule_internal.h"

namespace ops_hccl {
namespace sched {

// ---------------------------------------------------------------------------------------------------
// FUSED mode: symbolic execution
// ---------------------------------------------------------------------------------------------------
namespace {

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

bool Overlaps(u64 a, u64 alen, u64 b, u64 blen) { return a < b + blen && b < a + alen; }

}  // namespace

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
// stand for: the same lines the recorded steps give when traced.  Returns false when a tree among them cannot be
// fused (as FoldsFromTrace does); the caller then records the steps.
bool FoldsFromClosedForm(const std::vector<ClosedFold> &closed, const std::vector<OpParam> &params, int dtype, int op,
                         std::vector<Fold> &folds, std::string *text)
{
    const InputRanges inputs(params);
    // which operand the accumulated value is only shows in the bits of floating-point MAX and MIN (as in Flatten)
    const bool orderShows = IsFloatType(dtype) && op != HCCL_REDUCE_SUM && op != HCCL_REDUCE_PROD;
    struct Line {
        u32 rank;
        u64 offset;
        size_t fold;
    };
    std::vector<Line> lines;
    std::vector<std::string> treeText;   // per fold, for trees
    Tracer tr;                            // holds the reduce steps of the trees; no memory piece is ever written
    bool allFit = true;
    folds.reserve(closed.size());
    for (const ClosedFold &c : closed) {
        // the pieces a template names must lie inside the buffers of the call
        for (const ClosedFold::Ref &s : c.src) {
            if (s.rank >= params.size() || s.offset + c.bytes > params[s.rank].inputSize) return false;
        }
        for (const ClosedFold::Ref &d : c.dst) {
            if (d.rank >= params.size() || d.offset + c.bytes > params[d.rank].outputSize) return false;
        }
        Fold f;
        if (c.tree.empty()) {
            for (const ClosedFold::Ref &s : c.src) f.src.push_back(reinterpret_cast<u64>(params[s.rank].inputPtr) + s.offset);
            if (c.accIsSource && orderShows && c.src.size() > 1) {
                f.prog.assign(c.src.size(), 1);
                f.prog[0] = 0;
            }
            if (text) treeText.emplace_back();
        } else {
            // the tree as reduce steps over memory as it was (expression 0), then flattened as a traced piece is
            const size_t leaves = c.src.size();
            std::vector<int> made;
            made.reserve(c.tree.size());
            auto operand = [&](u32 child, int &expr, u64 &shift) {
                if (child < leaves) {
                    expr = 0;
                    shift = reinterpret_cast<u64>(params[c.src[child].rank].inputPtr) + c.src[child].offset;
                } else {
                    expr = made[child - leaves];
                    shift = 0;
                }
            };
            for (const ClosedFold::Step &st : c.tree) {
                Expr e;
                operand(st.srcChild, e.src, e.srcShift);
                operand(st.dstChild, e.dst, e.dstShift);
                made.push_back(tr.AddExpr(e));
            }
            f = Flatten(tr, made.back(), 0, dtype, op);
            if (!f.fits) allFit = false;
            if (text) treeText.push_back(ExprText(tr, made.back(), 0, inputs));
        }
        f.bytes = c.bytes;
        for (const ClosedFold::Ref &d : c.dst) {
            f.dsts.push_back(reinterpret_cast<u64>(params[d.rank].outputPtr) + d.offset);
            if (text) lines.push_back({d.rank, d.offset, folds.size()});
        }
        folds.push_back(std::move(f));
    }
    if (text == nullptr) return allFit;
    std::sort(lines.begin(), lines.end(),
              [](const Line &a, const Line &b) { return a.rank != b.rank ? a.rank < b.rank : a.offset < b.offset; });
    for (const Line &l : lines) {
        const ClosedFold &c = closed[l.fold];
        std::string expr = treeText[l.fold];
        if (c.tree.empty()) {
            auto leaf = [&](size_t k) {
                return LeafText(reinterpret_cast<u64>(params[c.src[k].rank].inputPtr) + c.src[k].offset, inputs);
            };
            expr = leaf(0);
            for (size_t k = 1; k < c.src.size(); ++k) {
                expr = c.accIsSource ? "(" + expr + "+" + leaf(k) + ")" : "(" + leaf(k) + "+" + expr + ")";
            }
        }
        std::ostringstream os;
        os << "rank " << l.rank << " out[" << l.offset << "," << c.bytes << ") = " << expr << "\n";
        *text += os.str();
    }
    return allFit;
}

// Builds the fused launch plan from the folds.  Returns false when they cannot run as one pass (a source that is
// not an input, or an output that overlaps another fold's source); the caller then runs the steps one by one.
bool BuildFusedPlan(const std::vector<OpParam> &params, std::vector<Fold> &folds, u32 esz, FusedPlan &plan, bool stated)
{
    const InputRanges inputs(params);
    // every source must be input data (or an output that the same fold overwrites in place); the sources of folds
    // stated in closed form are pieces of the inputs by construction
    for (const Fold &f : folds) {
        if (stated) break;
        for (u64 a : f.src) {
            if (inputs.Find(a, f.bytes) == nullptr) return false;
        }
    }
    // Different expressions may still read the same sources in the same order (pieces that were reduced by
    // different steps of equal shape): they become one fold with all the destinations.  (A closed form names every
    // value once.)
    if (!stated) {
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


}  // namespace sched
}  // namespace ops_hccl
