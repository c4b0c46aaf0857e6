// Ragged data movement of the V collectives: AlltoAllV pack/unpack and AllGatherV, for n virtual ranks
// whose buffers live in one GPU.
//
// Reference behaviour restated (one copy instead of the reference's pack -> CCL slot -> unpack pair):
//   AlltoAllV  in_i[sdispls_i[j] .. +sendCounts_i[j])  ->  out_j[rdispls_j[i] .. )
//              src/ops/all_to_all_v/template/aicpu/ins_temp_all_to_all_v_mesh_1D.cc:304-308 (pack into the
//              peer's CCL slot), :431-438 (unpack), :161-170 (self block)
//   AllGatherV out_j[displs[i] .. +counts[i]) = in_i[0 .. counts[i])   for all i, j
//              src/ops/all_gather_v/template/aicpu/ins_temp_all_gather_v_mesh_1D.cc:97-242;
//              contract include/hccl.h:120-135
//
// The count/displacement tables stay on the device.  Each workgroup stages the per-block tile counts in
// LDS, turns them into an inclusive prefix with a wavefront scan, and then walks tile numbers in a
// grid-stride loop, locating a tile's (source, destination) block by binary search in LDS.  No host
// round trip is needed when the tables come from an on-device router.
//
// Bound: HBM bandwidth.  Algorithmic bytes: AlltoAllV 2 x payload; AllGatherV (1 + n) x payload moved,
// 2n x payload delivered.
#include "fold.h"
#include "vops.h"

namespace hcclx {

namespace {

__device__ __forceinline__ uint64_t wave_inclusive_scan(uint64_t v)
{
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t lo = __shfl_up(static_cast<uint32_t>(v), d, 64);
        const uint32_t hi = __shfl_up(static_cast<uint32_t>(v >> 32), d, 64);
        if (lane >= d) v += (static_cast<uint64_t>(hi) << 32) | lo;
    }
    return v;
}

// In place: s_tab[0..m) (per-block tile counts) becomes its inclusive prefix sum.  m <= 4096.
// Each thread sums a contiguous run, a wavefront scan orders the 64 runs of a wave, and the four wave
// totals are combined through LDS.
__device__ void block_inclusive_scan(uint64_t *s_tab, uint32_t m, uint64_t *s_wave)
{
    const uint32_t per = (m + kThreads - 1) / kThreads;
    const uint32_t b = threadIdx.x * per;
    const uint32_t e = (b + per < m) ? b + per : m;
    uint64_t sum = 0;
    for (uint32_t i = b; i < e; ++i) sum += s_tab[i];
    const uint64_t incl = wave_inclusive_scan(sum);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) s_wave[wave] = incl;
    __syncthreads();
    uint64_t base = incl - sum;
    for (int w = 0; w < wave; ++w) base += s_wave[w];
    for (uint32_t i = b; i < e; ++i) {
        base += s_tab[i];
        s_tab[i] = base;
    }
    __syncthreads();
}

__device__ __forceinline__ uint32_t find_block(const uint64_t *s_end, uint32_t m, uint64_t t)
{
    uint32_t lo = 0;
    uint32_t hi = m - 1;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (s_end[mid] > t) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    return __builtin_amdgcn_readfirstlane(lo);
}

// One tile of a block copy: tile `tl` of a block of `bytes` bytes from src to dst[0..ndst) (all
// destinations share dst[0]'s alignment modulo 16, or lose only speed if they do not).
// kCached: the source is read with ordinary loads, so that workgroups that copy the same tile to another
// destination shortly afterwards find it in the L2; otherwise it streams past the caches.
template <bool kCached>
__device__ __forceinline__ u32x4 ld16c(const char *p)
{
    if constexpr (kCached) {
        return ld16_cached(p);
    } else {
        return ld16(p);
    }
}

template <int kCopyUnroll, bool kCached = false, typename DstFn>
__device__ __forceinline__ void copy_tile(const char *src, uint64_t dst0, uint64_t bytes, uint64_t tl, uint32_t ndst,
                                          DstFn dst_of)
{
    constexpr uint64_t kTileVecs = 256ull * kCopyUnroll;
    const uint64_t head = v_head_of(bytes, dst0);
    const uint64_t body = bytes - head;
    const uint64_t nvec = body / 16;
    const uint32_t shift = v_shift_of(head, dst0);
    // in the first tile of a shifted grid v0 wraps below zero for the vectors in front of the block and
    // fails the bound check below
    const uint64_t v0 = tl * kTileVecs + threadIdx.x - shift;
    const char *sb = src + head;
    if (tl * kTileVecs >= shift && (tl + 1) * kTileVecs - shift <= nvec) {
        u32x4 r[kCopyUnroll];
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) r[u] = ld16c<kCached>(sb + (v0 + static_cast<uint64_t>(u) * kThreads) * 16);
        for (uint32_t d = 0; d < ndst; ++d) {
            char *db = dst_of(d) + head;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) st16(db + (v0 + static_cast<uint64_t>(u) * kThreads) * 16, r[u]);
        }
        return;
    }
    // first or last tile of the block: the vectors inside it; the last one also moves head and tail bytes
    u32x4 r[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) {
        const uint64_t vi = v0 + static_cast<uint64_t>(u) * kThreads;
        if (vi < nvec) r[u] = ld16c<kCached>(sb + vi * 16);
    }
    const uint64_t tail = body - nvec * 16;
    char edge = 0;
    uint64_t edge_off = 0;
    const bool has_edge = tl == (nvec + shift) / kTileVecs && threadIdx.x < head + tail;
    if (has_edge) {
        edge_off = (threadIdx.x < head) ? threadIdx.x : head + nvec * 16 + (threadIdx.x - head);
        edge = src[edge_off];
    }
    for (uint32_t d = 0; d < ndst; ++d) {
        char *dp = dst_of(d);
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) {
            const uint64_t vi = v0 + static_cast<uint64_t>(u) * kThreads;
            if (vi < nvec) st16(dp + head + vi * 16, r[u]);
        }
        if (has_edge) dp[edge_off] = edge;
    }
}

template <typename Ptrs, typename Tabs>
__global__ void __launch_bounds__(kThreads)
k_alltoallv(Ptrs ptrs, Tabs tabs, uint32_t n, uint32_t esz, uint32_t tiles_per_block)
{
    extern __shared__ uint64_t s_end[];  // n*n entries, then 4 wave totals
    const uint32_t m = n * n;
    uint64_t *s_wave = s_end + m;
    for (uint32_t p = threadIdx.x; p < m; p += kThreads) {
        const uint32_t i = p / n;
        const uint32_t j = p - i * n;
        const uint64_t dst = reinterpret_cast<uint64_t>(ptrs.recv[j]) + tabs.rdispl(j * n + i) * esz;
        s_end[p] = v_tiles_of(tabs.count(p) * esz, dst, kA2avUnroll);
    }
    __syncthreads();
    block_inclusive_scan(s_end, m, s_wave);
    const uint64_t total = s_end[m - 1];

    // A workgroup takes runs of tiles_per_block consecutive tiles, so that the table set-up above is
    // paid once per run.
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * tiles_per_block;
    for (uint64_t run = static_cast<uint64_t>(blockIdx.x) * tiles_per_block; run < total; run += stride)
    for (uint64_t t = run; t < run + tiles_per_block && t < total; ++t) {
        const uint32_t p = find_block(s_end, m, t);
        const uint64_t tl = uniform64(t - (p ? s_end[p - 1] : 0));
        const uint32_t i = p / n;
        const uint32_t j = p - i * n;
        const uint64_t bytes = tabs.count(p) * esz;
        const char *src = ptrs.send[i] + tabs.sdispl(p) * esz;
        char *dst = ptrs.recv[j] + tabs.rdispl(j * n + i) * esz;
        copy_tile<kA2avUnroll>(src, reinterpret_cast<uint64_t>(dst), bytes, tl, 1, [=](uint32_t) { return dst; });
    }
}

// One tile per workgroup; the block of a tile is found in the host-made prefix that rides in the kernel
// arguments.  Every index below is wave-uniform, so the table reads are scalar loads.
template <int UNROLL>
__global__ void __launch_bounds__(kThreads)
k_alltoallv_direct(VRankPtrs16 ptrs, A2avTablesDirect tabs, uint32_t n, uint32_t esz)
{
    const uint32_t t = blockIdx.x;
    uint32_t lo = 0;
    uint32_t hi = n * n - 1;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (tabs.tile_end[mid] > t) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    const uint32_t p = lo;
    const uint64_t tl = t - (p ? tabs.tile_end[p - 1] : 0);
    const uint32_t i = p / n;
    const uint32_t j = p - i * n;
    const uint64_t bytes = static_cast<uint64_t>(tabs.send_counts[p]) * esz;
    const char *src = ptrs.send[i] + static_cast<uint64_t>(tabs.sdispls[p]) * esz;
    char *dst = ptrs.recv[j] + static_cast<uint64_t>(tabs.rdispls[p]) * esz;
    copy_tile<UNROLL>(src, reinterpret_cast<uint64_t>(dst), bytes, tl, 1, [=](uint32_t) { return dst; });
}

// One tile per workgroup; its block is found in the host-made list (every index is wave-uniform: scalar loads).
template <int UNROLL>
__global__ void __launch_bounds__(kThreads)
k_copy_blocks(const CopyBlock *__restrict__ blocks, uint32_t nblocks)
{
    const uint64_t t = blockIdx.x;
    uint32_t lo = 0;
    uint32_t hi = nblocks - 1;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (blocks[mid].tile_end > t) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    const uint64_t tl = t - (lo ? blocks[lo - 1].tile_end : 0);
    const char *src = blocks[lo].src;
    char *dst = blocks[lo].dst;
    const uint64_t bytes = blocks[lo].bytes;
    copy_tile<UNROLL>(src, reinterpret_cast<uint64_t>(dst), bytes, tl, 1, [=](uint32_t) { return dst; });
}

// One source run to several places, one place at a time.  Job blockIdx.y copies `bytes` bytes from src to its
// destinations dsts[job * nd + 0 .. ndst): blockIdx.x = d * slots + tile, and workgroups start in the order of
// their numbers, so a run (a few MiB) is written to its first destination, then to the second, and so on.  At any
// moment the GPU therefore writes ONE output instead of n at once, which HBM takes a third faster (measured: one
// source to eight outputs 4.8 -> 6.9 TB/s at the pins); the re-reads of the run come from the L2, not from HBM.
// The place of a workgroup follows from its number by arithmetic and two independent scalar loads: a table search
// in front of an 8 KiB tile costs a fifth of the kernel's time.  Jobs with fewer tiles or destinations than the
// launch's widest leave workgroups that exit at once; the host groups jobs of similar length per launch.
__global__ void __launch_bounds__(kThreads)
k_phased_copy(const PhasedJob *__restrict__ jobs, char *const *__restrict__ dsts, uint32_t slots, uint32_t nd)
{
    const uint32_t j = blockIdx.y;
    const uint32_t d = blockIdx.x / slots;
    const uint64_t tl = blockIdx.x - d * slots;
    const PhasedJob job = jobs[j];
    char *dst = dsts[static_cast<uint64_t>(j) * nd + d];
    if (d >= job.ndst || tl >= job.tiles) return;
    // tiles are laid out for the first destination's alignment; the others share it or lose only speed
    copy_tile<kPhasedUnroll, true>(job.src, job.dst0, job.bytes, tl, 1, [=](uint32_t) { return dst; });
}

template <typename Tabs>
__global__ void __launch_bounds__(kThreads)
k_allgatherv(VRankPtrs ptrs, Tabs tabs, uint32_t n, uint32_t esz, uint32_t tiles_per_block)
{
    extern __shared__ uint64_t s_end[];  // n entries, then 4 wave totals
    uint64_t *s_wave = s_end + n;
    for (uint32_t i = threadIdx.x; i < n; i += kThreads) {
        const uint64_t dst = reinterpret_cast<uint64_t>(ptrs.recv[0]) + tabs.displ(i) * esz;
        s_end[i] = v_tiles_of(tabs.count(i) * esz, dst, kAgvUnroll);
    }
    __syncthreads();
    block_inclusive_scan(s_end, n, s_wave);
    const uint64_t total = s_end[n - 1];

    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * tiles_per_block;
    for (uint64_t run = static_cast<uint64_t>(blockIdx.x) * tiles_per_block; run < total; run += stride)
    for (uint64_t t = run; t < run + tiles_per_block && t < total; ++t) {
        const uint32_t i = find_block(s_end, n, t);
        const uint64_t tl = uniform64(t - (i ? s_end[i - 1] : 0));
        const uint64_t bytes = tabs.count(i) * esz;
        const uint64_t off = tabs.displ(i) * esz;
        const char *src = ptrs.send[i];
        copy_tile<kAgvUnroll>(src, reinterpret_cast<uint64_t>(ptrs.recv[0]) + off, bytes, tl, n,
                  [&](uint32_t d) { return ptrs.recv[d] + off; });
    }
}

}  // namespace

hipError_t launch_alltoallv(const VRankPtrs &ptrs, const uint64_t *send_counts, const uint64_t *sdispls,
                            const uint64_t *rdispls, uint32_t n, uint32_t esz, uint32_t grid, uint32_t tiles_per_block,
                            hipStream_t stream)
{
    const size_t lds = (static_cast<size_t>(n) * n + 4) * sizeof(uint64_t);
    const A2avTablesPtr tabs{send_counts, sdispls, rdispls};
    HCCLX_LAUNCH((k_alltoallv<VRankPtrs, A2avTablesPtr>), dim3(grid), dim3(kThreads), lds, stream, ptrs, tabs, n,
                       esz, tiles_per_block);
    return hipGetLastError();
}

hipError_t launch_copy_blocks(const CopyBlock *blocks, uint32_t nblocks, uint32_t grid, int unroll, hipStream_t stream)
{
    if (unroll == 1) {
        HCCLX_LAUNCH((k_copy_blocks<1>), dim3(grid), dim3(kThreads), 0, stream, blocks, nblocks);
    } else if (unroll == 2) {
        HCCLX_LAUNCH((k_copy_blocks<2>), dim3(grid), dim3(kThreads), 0, stream, blocks, nblocks);
    } else {
        HCCLX_LAUNCH((k_copy_blocks<4>), dim3(grid), dim3(kThreads), 0, stream, blocks, nblocks);
    }
    return hipGetLastError();
}

__global__ void __launch_bounds__(kThreads) k_phased_copy_inline(PhasedInline tab, uint32_t slots, uint32_t nd)
{
    const uint32_t j = blockIdx.y;
    const uint32_t d = blockIdx.x / slots;
    const uint64_t tl = blockIdx.x - d * slots;
    const PhasedJob &job = tab.jobs[j];
    if (d >= job.ndst || d >= nd || tl >= job.tiles) return;
    char *dst = tab.base[d] + job.dst0;
    copy_tile<kPhasedUnroll, true>(job.src, reinterpret_cast<uint64_t>(tab.base[0]) + job.dst0, job.bytes, tl, 1,
                                   [=](uint32_t) { return dst; });
}

hipError_t launch_phased_copy_inline(const PhasedInline &tab, uint32_t njobs, uint32_t slots, uint32_t nd, hipStream_t stream)
{
    HCCLX_LAUNCH(k_phased_copy_inline, dim3(slots * nd, njobs), dim3(kThreads), 0, stream, tab, slots, nd);
    return hipGetLastError();
}

hipError_t launch_phased_copy(const PhasedJob *jobs, char *const *dsts, uint32_t njobs, uint32_t slots, uint32_t nd,
                              hipStream_t stream)
{
    HCCLX_LAUNCH(k_phased_copy, dim3(slots * nd, njobs), dim3(kThreads), 0, stream, jobs, dsts, slots, nd);
    return hipGetLastError();
}

hipError_t launch_alltoallv_direct(const VRankPtrs16 &ptrs, const A2avTablesDirect &tabs, uint32_t n, uint32_t esz,
                                   uint32_t grid, int unroll, hipStream_t stream)
{
    if (unroll == 1) {
        HCCLX_LAUNCH((k_alltoallv_direct<1>), dim3(grid), dim3(kThreads), 0, stream, ptrs, tabs, n, esz);
    } else if (unroll == 2) {
        HCCLX_LAUNCH((k_alltoallv_direct<2>), dim3(grid), dim3(kThreads), 0, stream, ptrs, tabs, n, esz);
    } else {
        HCCLX_LAUNCH((k_alltoallv_direct<4>), dim3(grid), dim3(kThreads), 0, stream, ptrs, tabs, n, esz);
    }
    return hipGetLastError();
}

// One wavefront per row of n <= 64 counts: displs = exclusive prefix sum, totals[row] = the row's sum.
__global__ void __launch_bounds__(64)
k_displs_from_counts(const uint64_t *__restrict__ counts, uint32_t n, uint64_t *__restrict__ displs,
                     uint64_t *__restrict__ totals)
{
    const uint64_t row = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint64_t c = lane < n ? counts[row * n + lane] : 0;
    const uint64_t incl = wave_inclusive_scan(c);
    if (lane < n) displs[row * n + lane] = incl - c;
    if (totals != nullptr && lane == n - 1) totals[row] = incl;
}

hipError_t launch_displs_from_counts(const uint64_t *counts, uint32_t rows, uint32_t n, uint64_t *displs, uint64_t *totals,
                                     hipStream_t stream)
{
    HCCLX_LAUNCH(k_displs_from_counts, dim3(rows), dim3(64), 0, stream, counts, n, displs, totals);
    return hipGetLastError();
}

hipError_t launch_allgatherv(const VRankPtrs &ptrs, const uint64_t *counts, const uint64_t *displs, uint32_t n,
                             uint32_t esz, uint32_t grid, uint32_t tiles_per_block, hipStream_t stream)
{
    const size_t lds = (static_cast<size_t>(n) + 4) * sizeof(uint64_t);
    const AgvTablesPtr tabs{counts, displs};
    HCCLX_LAUNCH((k_allgatherv<AgvTablesPtr>), dim3(grid), dim3(kThreads), lds, stream, ptrs, tabs, n, esz,
                       tiles_per_block);
    return hipGetLastError();
}

hipError_t launch_allgatherv_inline(const VRankPtrs &ptrs, const AgvTablesInline &tabs, uint32_t n, uint32_t esz,
                                    uint32_t grid, uint32_t tiles_per_block, hipStream_t stream)
{
    const size_t lds = (static_cast<size_t>(n) + 4) * sizeof(uint64_t);
    HCCLX_LAUNCH((k_allgatherv<AgvTablesInline>), dim3(grid), dim3(kThreads), lds, stream, ptrs, tabs, n, esz,
                       tiles_per_block);
    return hipGetLastError();
}

}  // namespace hcclx
