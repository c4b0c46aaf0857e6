// The caller side of an MoE AlltoAllV, for n virtual ranks at once: routing tables from per-entry
// destinations (stable grouping by destination rank), the row gather that packs the send buffers, and the
// inverse that combines what comes back.  C-ABI entry points: hcclx_moe_* in include/hcclx.h.
//
// The reference has no such step: its AlltoAllV takes finished send buffers and tables.  The nearest code is
// the staging either side of the transfer, PreCopy / PostCopy of InsTempAlltoAllVMesh1D
// (src/ops/all_to_all_v/template/aicpu/ins_temp_all_to_all_v_mesh_1D.cc:412-440).
//
// Bound: HBM bandwidth (pack / combine move rows of several KiB); the routing kernels touch 4 bytes per
// entry and are latency-bound.  Algorithmic bytes: pack 2 x entries x row bytes; combine (topk + 1) x
// tokens x row bytes.  hcclx_moe_dispatch and hcclx_moe_gather_combine do pack + AlltoAllV, and AlltoAllV back
// + combine, in one pass each: the rows go straight to (come straight from) the place the AlltoAllV would
// have put them, which halves the traffic of either direction.
#include "hcclx.h"
#include "hcclx_internal.h"
#include "kernels/elem.h"
#include "kernels/fold.h"

#include <cstring>

using namespace hcclx;

namespace {

constexpr uint32_t kMoeMaxRanks = 64;
constexpr uint32_t kMoeChunk = 256;        // entries per workgroup of the routing kernels
constexpr uint32_t kDropped = 0xffffffffu;  // perm value of an entry whose destination is out of range

struct MoeConstPtrs {
    const void *p[kMoeMaxRanks];
};
struct MoePtrs {
    void *p[kMoeMaxRanks];
};

__device__ __forceinline__ const MoePtrs &as_mutable_dev(const MoeConstPtrs &c)
{
    return reinterpret_cast<const MoePtrs &>(c);   // same layout; the landing addresses are only read through
}

// Workspace layout (uint32): base[n][n][chunks] (chunk fastest) -- first the per-chunk histogram, then,
// in place, its exclusive prefix over the chunks -- followed by row_start[n][n].
__host__ __device__ inline uint32_t chunks_of(uint32_t entries) { return (entries + kMoeChunk - 1) / kMoeChunk; }

__global__ void __launch_bounds__(kMoeChunk)
k_moe_hist(MoeConstPtrs dest, uint32_t n, uint32_t entries, uint32_t chunks, uint32_t *base)
{
    __shared__ uint32_t s_hist[kMoeMaxRanks];
    const uint32_t c = blockIdx.x;
    const uint32_t i = blockIdx.y;
    if (threadIdx.x < kMoeMaxRanks) s_hist[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t e = c * kMoeChunk + threadIdx.x;
    if (e < entries) {
        const int32_t d = static_cast<const int32_t *>(dest.p[i])[e];
        if (d >= 0 && static_cast<uint32_t>(d) < n) atomicAdd(&s_hist[d], 1u);
    }
    __syncthreads();
    if (threadIdx.x < n) base[(static_cast<uint64_t>(i) * n + threadIdx.x) * chunks + c] = s_hist[threadIdx.x];
}

__device__ __forceinline__ uint32_t wave_scan_u32(uint32_t v)
{
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

// One workgroup per rank i: every (i, d) histogram row becomes its exclusive prefix over the chunks (a
// wavefront scans 64 chunks at a time); the row totals give send counts and displacements.
__global__ void __launch_bounds__(256)
k_moe_scan(uint32_t n, uint32_t chunks, uint64_t row_elems, uint32_t *base, uint32_t *row_start, uint64_t *send_counts,
           uint64_t *sdispls, uint64_t *recv_counts)
{
    __shared__ uint32_t s_total[kMoeMaxRanks];
    const uint32_t i = blockIdx.x;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    for (uint32_t d = wave; d < n; d += 4) {
        uint32_t *row = base + (static_cast<uint64_t>(i) * n + d) * chunks;
        uint32_t running = 0;
        for (uint32_t c0 = 0; c0 < chunks; c0 += 64) {
            const uint32_t c = c0 + lane;
            const uint32_t v = c < chunks ? row[c] : 0;
            const uint32_t incl = wave_scan_u32(v);
            if (c < chunks) row[c] = running + incl - v;
            running += __shfl(incl, 63, 64);
        }
        if (lane == 0) s_total[d] = running;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t start = 0;
        for (uint32_t d = 0; d < n; ++d) {
            const uint32_t t = s_total[d];
            row_start[i * n + d] = start;
            send_counts[i * n + d] = static_cast<uint64_t>(t) * row_elems;
            sdispls[i * n + d] = static_cast<uint64_t>(start) * row_elems;
            recv_counts[d * n + i] = static_cast<uint64_t>(t) * row_elems;
            start += t;
        }
    }
}

// perm[e] = first row of the destination's group + entries of earlier chunks with that destination + rank of
// e among the entries of its own chunk with that destination (index order: the grouping is stable).
__global__ void __launch_bounds__(kMoeChunk)
k_moe_perm(MoeConstPtrs dest, MoePtrs perm, uint32_t n, uint32_t entries, uint32_t chunks, const uint32_t *base,
           const uint32_t *row_start, const uint64_t *send_counts, uint64_t *rdispls)
{
    // one workgroup also writes rdispls[j][i] = what ranks 0 .. i-1 send to rank j (the send counts are complete:
    // the scan kernel ran before this one)
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < n) {
        const uint32_t j = threadIdx.x;
        uint64_t run = 0;
        for (uint32_t i = 0; i < n; ++i) {
            rdispls[j * n + i] = run;
            run += send_counts[i * n + j];
        }
    }
    __shared__ uint32_t s_cnt[4][kMoeMaxRanks];
    const uint32_t c = blockIdx.x;
    const uint32_t i = blockIdx.y;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t e = c * kMoeChunk + threadIdx.x;
    int32_t d = -1;
    if (e < entries) d = static_cast<const int32_t *>(dest.p[i])[e];
    const bool valid = d >= 0 && static_cast<uint32_t>(d) < n;
    uint32_t rank = 0;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (uint32_t dd = 0; dd < n; ++dd) {
        const unsigned long long m = __ballot(valid && static_cast<uint32_t>(d) == dd);
        if (valid && static_cast<uint32_t>(d) == dd) rank = __popcll(m & below);
        if (lane == 0) s_cnt[wave][dd] = __popcll(m);
    }
    __syncthreads();
    if (e < entries) {
        uint32_t out = kDropped;
        if (valid) {
            uint32_t off = rank;
            for (uint32_t w = 0; w < wave; ++w) off += s_cnt[w][d];
            out = row_start[i * n + d] + base[(static_cast<uint64_t>(i) * n + d) * chunks + c] + off;
        }
        static_cast<uint32_t *>(perm.p[i])[e] = out;
    }
}

// The scan and permutation kernels in one launch, for tables small enough that every workgroup can afford to sum
// its rank's rows of the per-chunk histogram itself (at most kFusedChunks chunks per rank and kFusedCells histogram
// cells in all): two dependent launches instead of three.  Workgroup (c, i): per destination the entries of rank i
// in all chunks and in the chunks before c (one wavefront per destination, one lane per chunk), from them the first
// row of each destination's group, then the permutation of chunk c as in k_moe_perm.  The workgroups of chunk 0
// write their rank's rows of the count and displacement tables; workgroup (0, 0) also sums every rank's rows and
// writes rdispls.  base keeps the raw histogram.
constexpr uint32_t kFusedChunks = 64;
constexpr uint32_t kFusedCells = 16384;

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v)
{
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}

__global__ void __launch_bounds__(kMoeChunk)
k_moe_scan_perm(MoeConstPtrs dest, MoePtrs perm, uint32_t n, uint32_t entries, uint32_t chunks, uint64_t row_elems,
                const uint32_t *base, uint64_t *send_counts, uint64_t *sdispls, uint64_t *recv_counts, uint64_t *rdispls)
{
    __shared__ uint32_t s_total[kMoeMaxRanks];
    __shared__ uint32_t s_before[kMoeMaxRanks];
    __shared__ uint32_t s_start[kMoeMaxRanks];
    __shared__ uint32_t s_cnt[4][kMoeMaxRanks];
    __shared__ uint32_t s_all[kMoeMaxRanks * kMoeMaxRanks];   // workgroup (0, 0): entries of rank i for destination j
    const uint32_t c = blockIdx.x;
    const uint32_t i = blockIdx.y;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    for (uint32_t d = wave; d < n; d += 4) {
        const uint32_t v = lane < chunks ? base[(static_cast<uint64_t>(i) * n + d) * chunks + lane] : 0;
        const uint32_t total = wave_sum_u32(v);
        const uint32_t before = wave_sum_u32(lane < c ? v : 0);
        if (lane == 0) {
            s_total[d] = total;
            s_before[d] = before;
        }
    }
    if (c == 0 && i == 0) {
        for (uint32_t cell = threadIdx.x; cell < n * n; cell += kMoeChunk) {
            uint32_t t = 0;
            for (uint32_t k = 0; k < chunks; ++k) t += base[static_cast<uint64_t>(cell) * chunks + k];
            s_all[cell] = t;
        }
    }
    __syncthreads();
    if (wave == 0) {
        const uint32_t t = lane < n ? s_total[lane] : 0;
        const uint32_t incl = wave_scan_u32(t);
        s_start[lane] = incl - t;
        if (c == 0 && lane < n) {
            send_counts[i * n + lane] = static_cast<uint64_t>(t) * row_elems;
            sdispls[i * n + lane] = static_cast<uint64_t>(incl - t) * row_elems;
            recv_counts[lane * n + i] = static_cast<uint64_t>(t) * row_elems;
        }
    }
    if (c == 0 && i == 0 && threadIdx.x < n) {
        const uint32_t j = threadIdx.x;
        uint64_t run = 0;
        for (uint32_t r = 0; r < n; ++r) {
            rdispls[j * n + r] = run * row_elems;
            run += s_all[r * n + j];
        }
    }
    const uint32_t e = c * kMoeChunk + threadIdx.x;
    int32_t d = -1;
    if (e < entries) d = static_cast<const int32_t *>(dest.p[i])[e];
    const bool valid = d >= 0 && static_cast<uint32_t>(d) < n;
    uint32_t rank = 0;
    const unsigned long long below = (1ull << lane) - 1ull;
    for (uint32_t dd = 0; dd < n; ++dd) {
        const unsigned long long m = __ballot(valid && static_cast<uint32_t>(d) == dd);
        if (valid && static_cast<uint32_t>(d) == dd) rank = __popcll(m & below);
        if (lane == 0) s_cnt[wave][dd] = __popcll(m);
    }
    __syncthreads();
    if (e < entries) {
        uint32_t out = kDropped;
        if (valid) {
            uint32_t off = rank;
            for (uint32_t w = 0; w < wave; ++w) off += s_cnt[w][d];
            out = s_start[d] + s_before[d] + off;
        }
        static_cast<uint32_t *>(perm.p[i])[e] = out;
    }
}

// Row gather / scatter: 512 vectors of 16 bytes per workgroup, rows of vpr vectors.
//   PACK:    packed[perm[e]] = tokens[e / topk]      (g runs over entries x vpr)
//   UNPACK:  out[t] = packed[perm[t]]                (topk == 1; g runs over tokens x vpr)
template <bool PACK>
__global__ void __launch_bounds__(256)
k_moe_rows(MoeConstPtrs src, MoeConstPtrs perm, MoePtrs dst, uint32_t rows, uint32_t topk, uint32_t vpr)
{
    const uint32_t i = blockIdx.y;
    const uint64_t total = static_cast<uint64_t>(rows) * vpr;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const char *s = static_cast<const char *>(src.p[i]);
    char *o = static_cast<char *>(dst.p[i]);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 512 + u * 256 + threadIdx.x;
        if (g >= total) continue;
        const uint32_t e = static_cast<uint32_t>(g / vpr);
        const uint32_t v = static_cast<uint32_t>(g - static_cast<uint64_t>(e) * vpr);
        const uint32_t p = pm[e];
        if (PACK) {
            if (p == kDropped) continue;
            st16(o + (static_cast<uint64_t>(p) * vpr + v) * 16, ld16(s + (static_cast<uint64_t>(e / topk) * vpr + v) * 16));
        } else {
            u32x4 x = {0, 0, 0, 0};
            if (p != kDropped) x = ld16(s + (static_cast<uint64_t>(p) * vpr + v) * 16);
            st16(o + (static_cast<uint64_t>(e) * vpr + v) * 16, x);
        }
    }
}

// out[t] = sum over j of packed[perm[t * topk + j]], j ascending, starting from the first entry that was
// not dropped; accumulated in the compute type (fp32 for 16-bit floats), narrowed once.
template <int DT>
__global__ void __launch_bounds__(256)
k_moe_combine(MoeConstPtrs packed, MoeConstPtrs perm, MoePtrs out, uint32_t tokens, uint32_t topk, uint32_t vpr)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    const uint32_t i = blockIdx.y;
    const uint64_t total = static_cast<uint64_t>(tokens) * vpr;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const char *s = static_cast<const char *>(packed.p[i]);
    char *o = static_cast<char *>(out.p[i]);
    const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= total) return;
    const uint32_t t = static_cast<uint32_t>(g / vpr);
    const uint32_t v = static_cast<uint32_t>(g - static_cast<uint64_t>(t) * vpr);
    C acc[NE];
    bool have = false;
#pragma unroll
    for (int e = 0; e < NE; ++e) acc[e] = C(0);
    for (uint32_t j = 0; j < topk; ++j) {
        const uint32_t p = pm[static_cast<uint64_t>(t) * topk + j];
        if (p == kDropped) continue;
        C x[NE];
        V::unpack(ld16(s + (static_cast<uint64_t>(p) * vpr + v) * 16), x);
        if (!have) {
#pragma unroll
            for (int e = 0; e < NE; ++e) acc[e] = x[e];
            have = true;
        } else {
#pragma unroll
            for (int e = 0; e < NE; ++e) acc[e] = V::template combine<HCCL_REDUCE_SUM>(x[e], acc[e]);
        }
    }
    st16(o + (static_cast<uint64_t>(t) * vpr + v) * 16, V::pack(acc));
}

// Where rank i's rows for destination j land: packed row p of rank i sits at landing(...) + p rows, i.e. at the
// first row of the block from i in recv[j] minus the first row of the group for j in i's packed order.  The
// tables are a few hundred bytes and stay in the caches.
__device__ __forceinline__ char *landing(const MoePtrs &recv, uint32_t i, uint32_t j, uint32_t n, uint32_t esz,
                                         const uint64_t *sdispls, const uint64_t *rdispls)
{
    const int64_t elems = static_cast<int64_t>(rdispls[j * n + i]) - static_cast<int64_t>(sdispls[i * n + j]);
    return static_cast<char *>(recv.p[j]) + elems * static_cast<int64_t>(esz);
}

// Dispatch in one pass (what the pack kernel followed by the AlltoAllV kernel does in two):
// recv[dest[e]] row (landing + perm[e]) = tokens[e / topk].
__global__ void __launch_bounds__(256)
k_moe_dispatch(MoeConstPtrs tokens, MoeConstPtrs dest, MoeConstPtrs perm, MoePtrs recv, uint32_t n, uint32_t entries,
               uint32_t topk, uint32_t vpr, uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    const uint32_t i = blockIdx.y;
    const uint64_t total = static_cast<uint64_t>(entries) * vpr;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const int32_t *dt = static_cast<const int32_t *>(dest.p[i]);
    const char *s = static_cast<const char *>(tokens.p[i]);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 512 + u * 256 + threadIdx.x;
        if (g >= total) continue;
        const uint32_t e = static_cast<uint32_t>(g / vpr);
        const uint32_t v = static_cast<uint32_t>(g - static_cast<uint64_t>(e) * vpr);
        const uint32_t p = pm[e];
        const uint32_t j = static_cast<uint32_t>(dt[e]);
        if (p == kDropped || j >= n) continue;   // perm marks entries with a destination outside 0 .. n-1 as dropped
        char *o = landing(recv, i, j, n, esz, sdispls, rdispls);
        st16(o + (static_cast<uint64_t>(p) * vpr + v) * 16, ld16(s + (static_cast<uint64_t>(e / topk) * vpr + v) * 16));
    }
}

// The way back in one pass (what the AlltoAllV kernel followed by the combine kernel does in two):
// out[t] = sum over j < topk of the row of entry t * topk + j where dispatch put it, in the buffers `expert`.
// DT = int8 moves bytes (topk == 1: nothing is added).
template <int DT>
__global__ void __launch_bounds__(256)
k_moe_gather_combine(MoeConstPtrs expert, MoeConstPtrs dest, MoeConstPtrs perm, MoePtrs out, uint32_t n, uint32_t tokens,
                     uint32_t topk, uint32_t vpr, uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    const uint32_t i = blockIdx.y;
    const uint64_t total = static_cast<uint64_t>(tokens) * vpr;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const int32_t *dt = static_cast<const int32_t *>(dest.p[i]);
    char *o = static_cast<char *>(out.p[i]);
    const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= total) return;
    const uint32_t t = static_cast<uint32_t>(g / vpr);
    const uint32_t v = static_cast<uint32_t>(g - static_cast<uint64_t>(t) * vpr);
    C acc[NE];
    bool have = false;
#pragma unroll
    for (int e = 0; e < NE; ++e) acc[e] = C(0);
    for (uint32_t j = 0; j < topk; ++j) {
        const uint64_t e = static_cast<uint64_t>(t) * topk + j;
        const uint32_t p = pm[e];
        const uint32_t d = static_cast<uint32_t>(dt[e]);
        if (p == kDropped || d >= n) continue;
        const char *from = landing(as_mutable_dev(expert), i, d, n, esz, sdispls, rdispls);
        C x[NE];
        V::unpack(ld16(from + (static_cast<uint64_t>(p) * vpr + v) * 16), x);
        if (!have) {
#pragma unroll
            for (int k = 0; k < NE; ++k) acc[k] = x[k];
            have = true;
        } else {
#pragma unroll
            for (int k = 0; k < NE; ++k) acc[k] = V::template combine<HCCL_REDUCE_SUM>(x[k], acc[k]);
        }
    }
    st16(o + (static_cast<uint64_t>(t) * vpr + v) * 16, V::pack(acc));
}

// ---- rows of at least kLongRow vectors ----------------------------------------------------------------------
// A workgroup moves one run of ONE row, so the entry, its destination and where it lands are the same for every
// thread: they are fetched with scalar loads, and no thread divides or looks anything up.
constexpr uint32_t kLongRow = 128;

struct RowRuns {
    uint32_t per_row;   // runs a row is cut into
    uint32_t vecs;      // vectors per run (the last one may be shorter)
};
inline RowRuns row_runs(uint32_t vpr, uint32_t most)
{
    RowRuns r;
    r.per_row = (vpr + most - 1) / most;
    r.vecs = (vpr + r.per_row - 1) / r.per_row;
    return r;
}

// Scatter one row per entry straight to where the AlltoAllV would put it in recv[dest[e]].  Runs of up to 512
// vectors, two per thread.
__global__ void __launch_bounds__(256)
k_moe_scatter_long(MoeConstPtrs tokens, MoeConstPtrs dest, MoeConstPtrs perm, MoePtrs dst, uint32_t n, uint32_t topk, uint32_t vpr,
                   RowRuns runs, uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    const uint32_t i = blockIdx.y;
    const uint32_t e = blockIdx.x / runs.per_row;
    const uint32_t c = blockIdx.x - e * runs.per_row;
    const uint32_t p = static_cast<const uint32_t *>(perm.p[i])[e];
    if (p == kDropped) return;
    const uint32_t j = static_cast<uint32_t>(static_cast<const int32_t *>(dest.p[i])[e]);
    if (j >= n) return;
    char *base = landing(dst, i, j, n, esz, sdispls, rdispls);
    const char *from = static_cast<const char *>(tokens.p[i]) + static_cast<uint64_t>(e / topk) * vpr * 16;
    char *to = base + static_cast<uint64_t>(p) * vpr * 16;
    const uint32_t lo = c * runs.vecs;
    const uint32_t hi = lo + runs.vecs < vpr ? lo + runs.vecs : vpr;
    const uint32_t v0 = lo + threadIdx.x;
    const uint32_t v1 = v0 + 256;
    u32x4 x0, x1;
    if (v0 < hi) x0 = ld16(from + static_cast<uint64_t>(v0) * 16);
    if (v1 < hi) x1 = ld16(from + static_cast<uint64_t>(v1) * 16);
    if (v0 < hi) st16(to + static_cast<uint64_t>(v0) * 16, x0);
    if (v1 < hi) st16(to + static_cast<uint64_t>(v1) * 16, x1);
}

// The same scatter with R consecutive entries per workgroup: the look-ups of all R rows (entry, destination, landing
// offset: three dependent scalar loads each) are issued together and all 2 R vectors of a thread are loaded before
// the first is stored.
template <int R>
__global__ void __launch_bounds__(256)
k_moe_scatter_rows(MoeConstPtrs tokens, MoeConstPtrs dest, MoeConstPtrs perm, MoePtrs dst, uint32_t n, uint32_t entries, uint32_t topk,
                   uint32_t vpr, RowRuns runs, uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    const uint32_t i = blockIdx.y;
    const uint32_t g = blockIdx.x / runs.per_row;
    const uint32_t c = blockIdx.x - g * runs.per_row;
    const uint32_t lo = c * runs.vecs;
    const uint32_t hi = lo + runs.vecs < vpr ? lo + runs.vecs : vpr;
    const uint32_t v0 = lo + threadIdx.x;
    const uint32_t v1 = v0 + 256;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const int32_t *dt = static_cast<const int32_t *>(dest.p[i]);
    uint32_t p[R];
    uint32_t j[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t e = g * R + r;
        const uint32_t at = e < entries ? e : entries - 1;   // a group behind the last entry repeats it and stores nothing
        p[r] = pm[at];
        j[r] = static_cast<uint32_t>(dt[at]);
        if (e >= entries) p[r] = kDropped;
    }
    const char *from[R];
    char *to[R];
    bool ok[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        ok[r] = p[r] != kDropped && j[r] < n;
        const uint32_t e = g * R + r;
        char *base = landing(dst, i, ok[r] ? j[r] : 0u, n, esz, sdispls, rdispls);
        from[r] = static_cast<const char *>(tokens.p[i]) + static_cast<uint64_t>((e < entries ? e : entries - 1) / topk) * vpr * 16;
        to[r] = base + static_cast<uint64_t>(ok[r] ? p[r] : 0u) * vpr * 16;
    }
    u32x4 x[R][2];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (ok[r] && v0 < hi) x[r][0] = ld16(from[r] + static_cast<uint64_t>(v0) * 16);
        if (ok[r] && v1 < hi) x[r][1] = ld16(from[r] + static_cast<uint64_t>(v1) * 16);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (ok[r] && v0 < hi) st16(to[r] + static_cast<uint64_t>(v0) * 16, x[r][0]);
        if (ok[r] && v1 < hi) st16(to[r] + static_cast<uint64_t>(v1) * 16, x[r][1]);
    }
}

// Gather the rows of a token's entries from where dispatch put them in expert[dest[.]] and add them.  Runs of up
// to 256 vectors, one per thread.  DT = int8 moves bytes (topk == 1).
template <int DT>
__global__ void __launch_bounds__(256)
k_moe_gather_long(MoeConstPtrs rows, MoeConstPtrs dest, MoeConstPtrs perm, MoePtrs out, uint32_t n, uint32_t topk, uint32_t vpr,
                  RowRuns runs, uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    const uint32_t i = blockIdx.y;
    const uint32_t t = blockIdx.x / runs.per_row;
    const uint32_t c = blockIdx.x - t * runs.per_row;
    const uint32_t lo = c * runs.vecs;
    const uint32_t hi = lo + runs.vecs < vpr ? lo + runs.vecs : vpr;
    const uint32_t v = lo + threadIdx.x;
    const uint32_t *pm = static_cast<const uint32_t *>(perm.p[i]);
    const int32_t *dt = static_cast<const int32_t *>(dest.p[i]);
    C acc[NE];
    bool have = false;
#pragma unroll
    for (int k = 0; k < NE; ++k) acc[k] = C(0);
    for (uint32_t j = 0; j < topk; ++j) {
        const uint64_t e = static_cast<uint64_t>(t) * topk + j;
        const uint32_t p = pm[e];
        if (p == kDropped) continue;
        const uint32_t d = static_cast<uint32_t>(dt[e]);
        if (d >= n) continue;
        const char *base = landing(as_mutable_dev(rows), i, d, n, esz, sdispls, rdispls);
        if (v < hi) {
            C x[NE];
            V::unpack(ld16(base + (static_cast<uint64_t>(p) * vpr + v) * 16), x);
            if (!have) {
#pragma unroll
                for (int k = 0; k < NE; ++k) acc[k] = x[k];
            } else {
#pragma unroll
                for (int k = 0; k < NE; ++k) acc[k] = V::template combine<HCCL_REDUCE_SUM>(x[k], acc[k]);
            }
        }
        have = true;
    }
    if (v < hi) st16(static_cast<char *>(out.p[i]) + (static_cast<uint64_t>(t) * vpr + v) * 16, V::pack(acc));
}

hipError_t launch_gather_long(int kind, dim3 grid, hipStream_t st, const MoeConstPtrs &rows, const MoeConstPtrs &dest,
                              const MoeConstPtrs &perm, const MoePtrs &out, uint32_t n, uint32_t topk, uint32_t vpr, RowRuns runs,
                              uint32_t esz, const uint64_t *sdispls, const uint64_t *rdispls)
{
    if (kind == HCCL_DATA_TYPE_FP32) {
        HCCLX_LAUNCH(k_moe_gather_long<HCCL_DATA_TYPE_FP32>, grid, dim3(256), 0, st, rows, dest, perm, out, n, topk,
                           vpr, runs, esz, sdispls, rdispls);
    } else if (kind == HCCL_DATA_TYPE_FP16) {
        HCCLX_LAUNCH(k_moe_gather_long<HCCL_DATA_TYPE_FP16>, grid, dim3(256), 0, st, rows, dest, perm, out, n, topk,
                           vpr, runs, esz, sdispls, rdispls);
    } else if (kind == HCCL_DATA_TYPE_BFP16) {
        HCCLX_LAUNCH(k_moe_gather_long<HCCL_DATA_TYPE_BFP16>, grid, dim3(256), 0, st, rows, dest, perm, out, n, topk,
                           vpr, runs, esz, sdispls, rdispls);
    } else {
        HCCLX_LAUNCH(k_moe_gather_long<HCCL_DATA_TYPE_INT8>, grid, dim3(256), 0, st, rows, dest, perm, out, n, topk,
                           vpr, runs, esz, sdispls, rdispls);
    }
    return hipGetLastError();
}

int check_ranks(uint32_t n)
{
    if (n == 0 || n > kMoeMaxRanks) return fail(HCCL_E_PARA, "rank count outside 1.." + std::to_string(kMoeMaxRanks));
    return HCCL_SUCCESS;
}

int fill(const void *const *in, uint32_t n, MoeConstPtrs *out, const char *what, bool align16)
{
    if (in == nullptr) return fail(HCCL_E_PTR, std::string(what) + " pointer array is null");
    std::memset(out, 0, sizeof(*out));
    for (uint32_t i = 0; i < n; ++i) {
        if (in[i] == nullptr) return fail(HCCL_E_PTR, std::string(what) + "[" + std::to_string(i) + "] is null");
        if (align16 && (reinterpret_cast<uint64_t>(in[i]) & 15) != 0) {
            return fail(HCCL_E_PARA, std::string(what) + "[" + std::to_string(i) + "] is not 16-byte aligned");
        }
        out->p[i] = in[i];
    }
    return HCCL_SUCCESS;
}

MoePtrs as_mutable(const MoeConstPtrs &c)
{
    MoePtrs m;
    for (uint32_t i = 0; i < kMoeMaxRanks; ++i) m.p[i] = const_cast<void *>(c.p[i]);
    return m;
}

}  // namespace

extern "C" {

uint64_t hcclx_moe_workspace_bytes(uint32_t n, uint32_t entries)
{
    return (static_cast<uint64_t>(n) * n * chunks_of(entries) + static_cast<uint64_t>(n) * n) * sizeof(uint32_t);
}

int hcclx_moe_route(const int32_t *const *dest, uint32_t n, uint32_t entries, uint64_t row_elems, uint64_t *send_counts,
                    uint64_t *sdispls, uint64_t *recv_counts, uint64_t *rdispls, uint32_t *const *perm, void *workspace,
                    void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    int rc = check_ranks(n);
    if (rc != HCCL_SUCCESS) return rc;
    if (!send_counts || !sdispls || !recv_counts || !rdispls || !workspace) return fail(HCCL_E_PTR, "output table or workspace is null");
    if (entries == 0) return fail(HCCL_E_PARA, "no entries to route");
    if (static_cast<uint64_t>(entries) >= kDropped) return fail(HCCL_E_PARA, "too many entries");
    MoeConstPtrs d, p;
    rc = fill(reinterpret_cast<const void *const *>(dest), n, &d, "dest", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(perm), n, &p, "perm", false);
    if (rc != HCCL_SUCCESS) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t chunks = chunks_of(entries);
    uint32_t *base = static_cast<uint32_t *>(workspace);
    uint32_t *row_start = base + static_cast<uint64_t>(n) * n * chunks;
    HCCLX_LAUNCH(k_moe_hist, dim3(chunks, n), dim3(kMoeChunk), 0, st, d, n, entries, chunks, base);
    if (chunks <= kFusedChunks && static_cast<uint64_t>(n) * n * chunks <= kFusedCells) {
        HCCLX_LAUNCH(k_moe_scan_perm, dim3(chunks, n), dim3(kMoeChunk), 0, st, d, as_mutable(p), n, entries, chunks,
                           row_elems, base, send_counts, sdispls, recv_counts, rdispls);
        hipError_t fe = hipGetLastError();
        if (fe != hipSuccess) return fail_hip(fe, "moe routing kernels");
        return HCCL_SUCCESS;
    }
    HCCLX_LAUNCH(k_moe_scan, dim3(n), dim3(256), 0, st, n, chunks, row_elems, base, row_start, send_counts, sdispls,
                       recv_counts);
    HCCLX_LAUNCH(k_moe_perm, dim3(chunks, n), dim3(kMoeChunk), 0, st, d, as_mutable(p), n, entries, chunks, base,
                       row_start, send_counts, rdispls);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe routing kernels");
    return HCCL_SUCCESS;
}

int hcclx_moe_pack(const void *const *tokens, const uint32_t *const *perm, uint32_t n, uint32_t entries, uint32_t topk,
                   uint64_t row_bytes, void *const *packed, void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    int rc = check_ranks(n);
    if (rc != HCCL_SUCCESS) return rc;
    if (topk == 0 || entries == 0 || entries % topk != 0) return fail(HCCL_E_PARA, "entries must be a positive multiple of topk");
    if (row_bytes == 0 || row_bytes % 16 != 0) return fail(HCCL_E_PARA, "row size must be a positive multiple of 16 bytes");
    if (row_bytes / 16 > 0xffffffffull) return fail(HCCL_E_PARA, "row too long");
    MoeConstPtrs s, p, o;
    rc = fill(tokens, n, &s, "tokens", true);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(perm), n, &p, "perm", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(packed, n, &o, "packed", true);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t vpr = static_cast<uint32_t>(row_bytes / 16);
    const uint64_t blocks = (static_cast<uint64_t>(entries) * vpr + 511) / 512;
    if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
    HCCLX_LAUNCH(k_moe_rows<true>, dim3(static_cast<uint32_t>(blocks), n), dim3(256), 0, static_cast<hipStream_t>(stream),
                       s, p, as_mutable(o), entries, topk, vpr);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe pack kernel");
    return HCCL_SUCCESS;
}

int hcclx_moe_combine(const void *const *packed, const uint32_t *const *perm, uint32_t n, uint32_t tokens, uint32_t topk,
                      uint64_t row_elems, int dtype, void *const *out, void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    int rc = check_ranks(n);
    if (rc != HCCL_SUCCESS) return rc;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (topk == 0 || tokens == 0) return fail(HCCL_E_PARA, "tokens and topk must be positive");
    const uint64_t row_bytes = row_elems * esz;
    if (row_bytes == 0 || row_bytes % 16 != 0) return fail(HCCL_E_PARA, "row size must be a positive multiple of 16 bytes");
    if (row_bytes / 16 > 0xffffffffull) return fail(HCCL_E_PARA, "row too long");
    if (topk > 1 && dtype != HCCL_DATA_TYPE_FP32 && dtype != HCCL_DATA_TYPE_FP16 && dtype != HCCL_DATA_TYPE_BFP16) {
        return fail(HCCL_E_NOT_SUPPORT, "combining several rows needs fp32, fp16 or bf16");
    }
    MoeConstPtrs s, p, o;
    rc = fill(packed, n, &s, "packed", true);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(perm), n, &p, "perm", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(out, n, &o, "out", true);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t vpr = static_cast<uint32_t>(row_bytes / 16);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (topk == 1) {
        const uint64_t blocks = (static_cast<uint64_t>(tokens) * vpr + 511) / 512;
        if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        HCCLX_LAUNCH(k_moe_rows<false>, dim3(static_cast<uint32_t>(blocks), n), dim3(256), 0, st, s, p, as_mutable(o),
                           tokens, 1u, vpr);
    } else {
        const uint64_t blocks = (static_cast<uint64_t>(tokens) * vpr + 255) / 256;
        if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        const dim3 grid(static_cast<uint32_t>(blocks), n);
        if (dtype == HCCL_DATA_TYPE_FP32) {
            HCCLX_LAUNCH(k_moe_combine<HCCL_DATA_TYPE_FP32>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        } else if (dtype == HCCL_DATA_TYPE_FP16) {
            HCCLX_LAUNCH(k_moe_combine<HCCL_DATA_TYPE_FP16>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        } else {
            HCCLX_LAUNCH(k_moe_combine<HCCL_DATA_TYPE_BFP16>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe combine kernel");
    return HCCL_SUCCESS;
}

int hcclx_moe_dispatch(const void *const *tokens, const int32_t *const *dest, const uint32_t *const *perm, uint32_t n,
                       uint32_t entries, uint32_t topk, uint64_t row_elems, int dtype, const uint64_t *sdispls,
                       const uint64_t *rdispls, void *const *recv, void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    int rc = check_ranks(n);
    if (rc != HCCL_SUCCESS) return rc;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (topk == 0 || entries == 0 || entries % topk != 0) return fail(HCCL_E_PARA, "entries must be a positive multiple of topk");
    const uint64_t row_bytes = row_elems * esz;
    if (row_bytes == 0 || row_bytes % 16 != 0) return fail(HCCL_E_PARA, "row size must be a positive multiple of 16 bytes");
    if (row_bytes / 16 > 0xffffffffull) return fail(HCCL_E_PARA, "row too long");
    if (!sdispls || !rdispls) return fail(HCCL_E_PTR, "displacement table is null");
    MoeConstPtrs s, d, p, o;
    rc = fill(tokens, n, &s, "tokens", true);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(dest), n, &d, "dest", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(perm), n, &p, "perm", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(recv, n, &o, "recv", true);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t vpr = static_cast<uint32_t>(row_bytes / 16);
    if (vpr >= kLongRow) {
        const RowRuns runs = row_runs(vpr, 512);
        const uint32_t rows = device_ctx()->moe_scatter_rows;
        if (rows == 2) {   // two entries per workgroup: 162.2 against 165.4 us for route + dispatch of 8 x 4096 x 7168 bf16 (four: 281.6)
            const uint64_t groups = (static_cast<uint64_t>(entries) + 1) / 2 * runs.per_row;
            if (groups > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
            HCCLX_LAUNCH(k_moe_scatter_rows<2>, dim3(static_cast<uint32_t>(groups), n), dim3(256), 0, static_cast<hipStream_t>(stream),
                         s, d, p, as_mutable(o), n, entries, topk, vpr, runs, static_cast<uint32_t>(esz), sdispls, rdispls);
            hipError_t re = hipGetLastError();
            if (re != hipSuccess) return fail_hip(re, "moe dispatch kernel");
            return HCCL_SUCCESS;
        }
        const uint64_t long_blocks = static_cast<uint64_t>(entries) * runs.per_row;
        if (long_blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        HCCLX_LAUNCH(k_moe_scatter_long, dim3(static_cast<uint32_t>(long_blocks), n), dim3(256), 0,
                           static_cast<hipStream_t>(stream), s, d, p, as_mutable(o), n, topk, vpr, runs, static_cast<uint32_t>(esz),
                           sdispls, rdispls);
        hipError_t le = hipGetLastError();
        if (le != hipSuccess) return fail_hip(le, "moe dispatch kernel");
        return HCCL_SUCCESS;
    }
    const uint64_t blocks = (static_cast<uint64_t>(entries) * vpr + 511) / 512;
    if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
    HCCLX_LAUNCH(k_moe_dispatch, dim3(static_cast<uint32_t>(blocks), n), dim3(256), 0, static_cast<hipStream_t>(stream), s, d,
                       p, as_mutable(o), n, entries, topk, vpr, static_cast<uint32_t>(esz), sdispls, rdispls);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe dispatch kernel");
    return HCCL_SUCCESS;
}

int hcclx_moe_gather_combine(const void *const *expert, const int32_t *const *dest, const uint32_t *const *perm, uint32_t n,
                             uint32_t tokens, uint32_t topk, uint64_t row_elems, int dtype, const uint64_t *sdispls,
                             const uint64_t *rdispls, void *const *out, void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    int rc = check_ranks(n);
    if (rc != HCCL_SUCCESS) return rc;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (topk == 0 || tokens == 0) return fail(HCCL_E_PARA, "tokens and topk must be positive");
    const uint64_t row_bytes = row_elems * esz;
    if (row_bytes == 0 || row_bytes % 16 != 0) return fail(HCCL_E_PARA, "row size must be a positive multiple of 16 bytes");
    if (row_bytes / 16 > 0xffffffffull) return fail(HCCL_E_PARA, "row too long");
    if (topk > 1 && dtype != HCCL_DATA_TYPE_FP32 && dtype != HCCL_DATA_TYPE_FP16 && dtype != HCCL_DATA_TYPE_BFP16) {
        return fail(HCCL_E_NOT_SUPPORT, "combining several rows needs fp32, fp16 or bf16");
    }
    if (!sdispls || !rdispls) return fail(HCCL_E_PTR, "displacement table is null");
    MoeConstPtrs s, d, p, o;
    rc = fill(expert, n, &s, "expert", true);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(dest), n, &d, "dest", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(reinterpret_cast<const void *const *>(perm), n, &p, "perm", false);
    if (rc != HCCL_SUCCESS) return rc;
    rc = fill(out, n, &o, "out", true);
    if (rc != HCCL_SUCCESS) return rc;
    const uint32_t vpr = static_cast<uint32_t>(row_bytes / 16);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int kind = topk == 1 ? HCCL_DATA_TYPE_INT8 : dtype;
    if (vpr >= kLongRow) {
        const RowRuns runs = row_runs(vpr, 256);
        const uint64_t long_blocks = static_cast<uint64_t>(tokens) * runs.per_row;
        if (long_blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        const hipError_t le = launch_gather_long(kind, dim3(static_cast<uint32_t>(long_blocks), n), st, s, d, p, as_mutable(o), n,
                                                       topk, vpr, runs, static_cast<uint32_t>(esz), sdispls, rdispls);
        if (le != hipSuccess) return fail_hip(le, "moe gather-combine kernel");
        return HCCL_SUCCESS;
    }
    const uint64_t blocks = (static_cast<uint64_t>(tokens) * vpr + 255) / 256;
    if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
    const dim3 grid(static_cast<uint32_t>(blocks), n);
    if (kind == HCCL_DATA_TYPE_FP32) {
        HCCLX_LAUNCH(k_moe_gather_combine<HCCL_DATA_TYPE_FP32>, grid, dim3(256), 0, st, s, d, p, as_mutable(o), n, tokens, topk,
                           vpr, static_cast<uint32_t>(esz), sdispls, rdispls);
    } else if (kind == HCCL_DATA_TYPE_FP16) {
        HCCLX_LAUNCH(k_moe_gather_combine<HCCL_DATA_TYPE_FP16>, grid, dim3(256), 0, st, s, d, p, as_mutable(o), n, tokens, topk,
                           vpr, static_cast<uint32_t>(esz), sdispls, rdispls);
    } else if (kind == HCCL_DATA_TYPE_BFP16) {
        HCCLX_LAUNCH(k_moe_gather_combine<HCCL_DATA_TYPE_BFP16>, grid, dim3(256), 0, st, s, d, p, as_mutable(o), n, tokens, topk,
                           vpr, static_cast<uint32_t>(esz), sdispls, rdispls);
    } else {
        HCCLX_LAUNCH(k_moe_gather_combine<HCCL_DATA_TYPE_INT8>, grid, dim3(256), 0, st, s, d, p, as_mutable(o), n, tokens, topk,
                           vpr, static_cast<uint32_t>(esz), sdispls, rdispls);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe gather-combine kernel");
    return HCCL_SUCCESS;
}

}  // extern "C"
