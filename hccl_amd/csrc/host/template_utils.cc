#include <algorithm>

#include "template_base.h"

namespace ops_hccl {

u32 GetNHRStepNum(u32 rankSize)
{
    u32 nSteps = 0;
    for (u32 tmp = rankSize - 1; tmp != 0; tmp >>= 1, nSteps++) {
    }
    return nSteps;
}

HcclResult GetAlgRank(u32 virtRank, const std::vector<u32> &rankIds, u32 &algRank)
{
    auto it = std::find(rankIds.begin(), rankIds.end(), virtRank);
    CHK_PRT_RET(it == rankIds.end(), HCCL_ERROR("[GetAlgRank] Invalid virtual Rank!"), HCCL_E_PARA);
    algRank = static_cast<u32>(it - rankIds.begin());
    return HCCL_SUCCESS;
}

std::vector<SliceInfo> SplitDataByRank(u64 count, u32 sliceNum, u64 dataTypeSize)
{
    std::vector<SliceInfo> out;
    const u64 sliceCount = RoundUp(count, sliceNum);
    u64 offsetCount = 0;
    for (u32 i = 0; i < sliceNum; ++i) {
        const u64 cur = (count - offsetCount > sliceCount) ? sliceCount : count - offsetCount;
        out.emplace_back(offsetCount * dataTypeSize, cur * dataTypeSize, cur);
        offsetCount += cur;
    }
    return out;
}

void GetNHRReduceScatterSteps(u32 n, u32 me, std::vector<NHRStepInfo> &steps)
{
    const u32 nSteps = GetNHRStepNum(n);
    steps.assign(nSteps, NHRStepInfo());
    for (u32 step = 0; step < nSteps; ++step) {
        const u32 delta = 1u << step;
        NHRStepInfo &s = steps[step];
        s.step = step;
        s.myRank = me;
        s.toRank = (me + n - delta) % n;
        s.fromRank = (me + delta) % n;
        s.nSlices = (n - 1 + (1u << step)) / (1u << (step + 1));
        const u32 dSlice = 1u << (step + 1);
        u32 tx = s.toRank;
        u32 rx = me;
        for (u32 i = 0; i < s.nSlices; ++i) {
            s.txSliceIdxs.push_back(tx);
            s.rxSliceIdxs.push_back(rx);
            tx = (tx + n - dSlice % n) % n;
            rx = (rx + n - dSlice % n) % n;
        }
    }
}

void GetNHRAllGatherSteps(u32 n, u32 me, std::vector<NHRStepInfo> &steps)
{
    const u32 nSteps = GetNHRStepNum(n);
    steps.assign(nSteps, NHRStepInfo());
    for (u32 step = 0; step < nSteps; ++step) {
        const u32 delta = 1u << (nSteps - 1 - step);
        NHRStepInfo &s = steps[step];
        s.step = step;
        s.myRank = me;
        s.toRank = (me + delta) % n;
        s.fromRank = (me + n - delta % n) % n;
        s.nSlices = (n - 1 + delta) / (1u << (nSteps - step));
        const u32 dSlice = 1u << (nSteps - step);
        u32 tx = me;
        u32 rx = (me + n - delta % n) % n;
        for (u32 i = 0; i < s.nSlices; ++i) {
            s.txSliceIdxs.push_back(tx);
            s.rxSliceIdxs.push_back(rx);
            tx = (tx + n - dSlice % n) % n;
            rx = (rx + n - dSlice % n) % n;
        }
    }
}

SliceValues::SliceValues(u32 ranks)
{
    nodes_.resize(ranks);
    held_.resize(ranks);
    for (u32 r = 0; r < ranks; ++r) {
        nodes_[r].rank = r;
        held_[r] = static_cast<int>(r);
    }
}

void SliceValues::Reduce(u32 dstRank, u32 srcRank)
{
    Node n;
    n.src = held_[srcRank];
    n.dst = held_[dstRank];
    nodes_.push_back(n);
    staged_.emplace_back(dstRank, static_cast<int>(nodes_.size()) - 1);
}

void SliceValues::Copy(u32 dstRank, u32 srcRank) { staged_.emplace_back(dstRank, held_[srcRank]); }

void SliceValues::EndRound()
{
    for (const auto &s : staged_) held_[s.first] = s.second;
    staged_.clear();
}

// Children first; returns the number the node has in f (a leaf: its place in f.src; an inner node: f.src.size() of
// the finished fold is not known yet, so inner nodes are numbered from kInner up and renumbered by Emit).
constexpr u32 kInner = 1u << 30;
u32 SliceValues::EmitNode(int node, u64 inOffset, ClosedFold &f) const
{
    const Node &n = nodes_[node];
    if (n.src < 0) {
        f.src.push_back({n.rank, inOffset});
        return static_cast<u32>(f.src.size()) - 1;
    }
    ClosedFold::Step st;
    st.dstChild = EmitNode(n.dst, inOffset, f);
    st.srcChild = EmitNode(n.src, inOffset, f);
    f.tree.push_back(st);
    return kInner + static_cast<u32>(f.tree.size()) - 1;
}

void SliceValues::Emit(u32 r, u64 inOffset, ClosedFold &f) const
{
    f.src.clear();
    f.tree.clear();
    (void)EmitNode(held_[r], inOffset, f);
    const u32 leaves = static_cast<u32>(f.src.size());
    for (ClosedFold::Step &st : f.tree) {
        if (st.srcChild >= kInner) st.srcChild = st.srcChild - kInner + leaves;
        if (st.dstChild >= kInner) st.dstChild = st.dstChild - kInner + leaves;
    }
}

}  // namespace ops_hccl
