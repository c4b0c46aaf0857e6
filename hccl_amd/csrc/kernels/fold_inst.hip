// One data type's instantiations of the fold kernel.  Built once per type with
//   -DHCCLX_DT=<HcclDataType enumerator> -DHCCLX_NAME=<suffix> -DHCCLX_ORDERED=<0|1>
// HCCLX_ORDERED=1 (floating types) also builds the self-first and tree modes; for integers every fold
// order gives the same bits, so the launcher maps those modes onto the chain kernel.
// With -DHCCLX_COPY the unit holds the byte copy kernel instead (one source, many destinations).
#include "fold.h"

namespace hcclx {

template <int DT, int OP, int MAXN, int MODE>
static hipError_t launch_one(const FoldLaunch &l)
{
    HCCLX_LAUNCH((k_fold<DT, OP, MAXN, MODE>), dim3(l.grid), dim3(kFoldThreads), l.nseg * sizeof(uint64_t), l.stream,
                       l.tile_end, static_cast<const SegDev *>(l.segs), l.nseg, l.total_tiles, l.store_policy, l.uniform_tiles);
    return hipGetLastError();
}

template <int DT, int OP, int MODE, int NFIX>
static hipError_t launch_waves_n(const FoldLaunch &l)
{
    const bool direct = l.nseg <= kFoldDirectSegs || l.uniform_tiles != 0;
    const size_t lds = waves_lds_bytes(static_cast<int>(l.waves)) + (direct ? 0 : l.nseg * sizeof(uint64_t));
    HCCLX_LAUNCH((k_fold_waves<DT, OP, MODE, NFIX>), dim3(static_cast<uint32_t>(l.total_tiles)), dim3(l.waves * kWaveLanes), lds,
                 l.stream, l.tile_end, static_cast<const SegDev *>(l.segs), l.nseg, l.pieces, l.store_policy, l.uniform_tiles);
    return hipGetLastError();
}

// The self-first orders get an instance per rank count up to twelve (the widest the launch policy takes by itself);
// chains, and wider or mixed launches, run on the instance that reads the count per segment.
template <int DT, int OP, int MODE>
static hipError_t launch_waves(const FoldLaunch &l)
{
    if constexpr (MODE == kFoldSelfFirst) {
        switch (l.waves_fixed) {
            case 2: return launch_waves_n<DT, OP, MODE, 2>(l);
            case 3: return launch_waves_n<DT, OP, MODE, 3>(l);
            case 4: return launch_waves_n<DT, OP, MODE, 4>(l);
            case 5: return launch_waves_n<DT, OP, MODE, 5>(l);
            case 6: return launch_waves_n<DT, OP, MODE, 6>(l);
            case 7: return launch_waves_n<DT, OP, MODE, 7>(l);
            case 8: return launch_waves_n<DT, OP, MODE, 8>(l);
            case 9: return launch_waves_n<DT, OP, MODE, 9>(l);
            case 10: return launch_waves_n<DT, OP, MODE, 10>(l);
            case 11: return launch_waves_n<DT, OP, MODE, 11>(l);
            case 12: return launch_waves_n<DT, OP, MODE, 12>(l);
            case 13: return launch_waves_n<DT, OP, MODE, 13>(l);
            case 14: return launch_waves_n<DT, OP, MODE, 14>(l);
            case 15: return launch_waves_n<DT, OP, MODE, 15>(l);
            case 16: return launch_waves_n<DT, OP, MODE, 16>(l);
            default: return launch_waves_n<DT, OP, MODE, 0>(l);
        }
    } else if constexpr (MODE == kFoldChain) {
        return launch_waves_n<DT, OP, MODE, 0>(l);
    } else {
        return hipErrorInvalidValue;
    }
}

template <int DT, int OP, int MODE, int U>
static hipError_t launch_wide_u(const FoldLaunch &l)
{
    HCCLX_LAUNCH((k_fold_wide<DT, OP, MODE, U>), dim3(l.grid), dim3(kFoldThreads), l.nseg * sizeof(uint64_t), l.stream,
                       l.tile_end, static_cast<const SegWide *>(l.segs), l.nseg, l.total_tiles, l.xcd_remap, l.store_policy, l.uniform_tiles);
    return hipGetLastError();
}

template <int DT, int OP, int MODE>
static hipError_t launch_wide(const FoldLaunch &l)
{
    if constexpr (MODE == kFoldChain) {
        return l.wide_unroll == kWideUnrollOne ? launch_wide_u<DT, OP, MODE, kWideUnrollOne>(l)
                                               : launch_wide_u<DT, OP, MODE, kWideUnrollMany>(l);
    } else {
        return launch_wide_u<DT, OP, MODE, 1>(l);
    }
}

#ifdef HCCLX_COPY

hipError_t fold_dispatch_copy(const FoldLaunch &l)
{
    return launch_one<HCCL_DATA_TYPE_INT8, HCCL_REDUCE_SUM, 1, kFoldChain>(l);
}

#else

template <int OP, int MODE>
static hipError_t by_fan(int maxn, const FoldLaunch &l)
{
    if (l.waves != 0 && maxn <= kMaxFan) return launch_waves<HCCLX_DT, OP, MODE>(l);
    switch (maxn) {
        case 2: return launch_one<HCCLX_DT, OP, 2, MODE>(l);
        case 4: return launch_one<HCCLX_DT, OP, 4, MODE>(l);
        case 8: return launch_one<HCCLX_DT, OP, 8, MODE>(l);
        case 16: return launch_one<HCCLX_DT, OP, 16, MODE>(l);
        case kMaxWideFan: return launch_wide<HCCLX_DT, OP, MODE>(l);
        default: return hipErrorInvalidValue;
    }
}

template <int MODE>
static hipError_t by_op(int op, int maxn, const FoldLaunch &l)
{
    switch (op) {
        case HCCL_REDUCE_SUM: return by_fan<HCCL_REDUCE_SUM, MODE>(maxn, l);
        case HCCL_REDUCE_PROD: return by_fan<HCCL_REDUCE_PROD, MODE>(maxn, l);
        case HCCL_REDUCE_MAX: return by_fan<HCCL_REDUCE_MAX, MODE>(maxn, l);
        case HCCL_REDUCE_MIN: return by_fan<HCCL_REDUCE_MIN, MODE>(maxn, l);
        default: return hipErrorInvalidValue;
    }
}

#define HCCLX_CAT_(a, b) a##b
#define HCCLX_CAT(a, b) HCCLX_CAT_(a, b)

hipError_t HCCLX_CAT(fold_dispatch_, HCCLX_NAME)(int op, int maxn, int mode, const FoldLaunch &l)
{
    if (mode == kFoldChain) {
        return by_op<kFoldChain>(op, maxn, l);
    }
#if HCCLX_ORDERED
    if (mode == kFoldSelfFirst) {
        return by_op<kFoldSelfFirst>(op, maxn, l);
    }
    if (mode == kFoldTree) {
        return by_op<kFoldTree>(op, maxn, l);
    }
#endif
    return hipErrorInvalidValue;
}

#endif

}  // namespace hcclx
