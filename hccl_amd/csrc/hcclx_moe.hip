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
// tokens x row bytes.
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

// rdispls[j][i] = what ranks 0 .. i-1 send to rank j.
__global__ void __launch_bounds__(kMoeMaxRanks)
k_moe_rdispls(uint32_t n, const uint64_t *send_counts, uint64_t *rdispls)
{
    const uint32_t j = threadIdx.x;
    if (j >= n) return;
    uint64_t run = 0;
    for (uint32_t i = 0; i < n; ++i) {
        rdispls[j * n + i] = run;
        run += send_counts[i * n + j];
    }
}

// perm[e] = first row of the destination's group + entries of earlier chunks with that destination + rank of
// e among the entries of its own chunk with that destination (index order: the grouping is stable).
__global__ void __launch_bounds__(kMoeChunk)
k_moe_perm(MoeConstPtrs dest, MoePtrs perm, uint32_t n, uint32_t entries, uint32_t chunks, const uint32_t *base,
           const uint32_t *row_start)
{
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
    hipLaunchKernelGGL(k_moe_hist, dim3(chunks, n), dim3(kMoeChunk), 0, st, d, n, entries, chunks, base);
    hipLaunchKernelGGL(k_moe_scan, dim3(n), dim3(256), 0, st, n, chunks, row_elems, base, row_start, send_counts, sdispls,
                       recv_counts);
    hipLaunchKernelGGL(k_moe_rdispls, dim3(1), dim3(kMoeMaxRanks), 0, st, n, send_counts, rdispls);
    hipLaunchKernelGGL(k_moe_perm, dim3(chunks, n), dim3(kMoeChunk), 0, st, d, as_mutable(p), n, entries, chunks, base,
                       row_start);
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
    hipLaunchKernelGGL(k_moe_rows<true>, dim3(static_cast<uint32_t>(blocks), n), dim3(256), 0, static_cast<hipStream_t>(stream),
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
        hipLaunchKernelGGL(k_moe_rows<false>, dim3(static_cast<uint32_t>(blocks), n), dim3(256), 0, st, s, p, as_mutable(o),
                           tokens, 1u, vpr);
    } else {
        const uint64_t blocks = (static_cast<uint64_t>(tokens) * vpr + 255) / 256;
        if (blocks > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        const dim3 grid(static_cast<uint32_t>(blocks), n);
        if (dtype == HCCL_DATA_TYPE_FP32) {
            hipLaunchKernelGGL(k_moe_combine<HCCL_DATA_TYPE_FP32>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        } else if (dtype == HCCL_DATA_TYPE_FP16) {
            hipLaunchKernelGGL(k_moe_combine<HCCL_DATA_TYPE_FP16>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        } else {
            hipLaunchKernelGGL(k_moe_combine<HCCL_DATA_TYPE_BFP16>, grid, dim3(256), 0, st, s, p, as_mutable(o), tokens, topk, vpr);
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "moe combine kernel");
    return HCCL_SUCCESS;
}

}  // extern "C"
