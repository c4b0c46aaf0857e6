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

}  // namespace ops_hccl
