// C-ABI entry points of the V collectives (see include/hcclx.h).
#include "hcclx.h"
#include "hcclx_internal.h"
#include "kernels/elem.h"
#include "kernels/vops.h"

#include <cstring>
#include <vector>

using namespace hcclx;

namespace {

// Host tables are staged through the descriptor ring; device tables are used where they are.
int stage_tables(DeviceCtx *ctx, const uint64_t *const *tabs, int ntabs, size_t entries, int on_device,
                 hipStream_t st, const uint64_t **out)
{
    if (on_device) {
        for (int i = 0; i < ntabs; ++i) out[i] = tabs[i];
        return HCCL_SUCCESS;
    }
    const size_t one = (entries * sizeof(uint64_t) + 255) & ~static_cast<size_t>(255);
    char *h = nullptr;
    char *d = nullptr;
    int rc = ring_reserve(ctx, one * ntabs, st, &h, &d);
    if (rc != HCCL_SUCCESS) return rc;
    for (int i = 0; i < ntabs; ++i) {
        std::memcpy(h + one * i, tabs[i], entries * sizeof(uint64_t));
        out[i] = reinterpret_cast<const uint64_t *>(d + one * i);
    }
    HCCLX_HIP(hipMemcpyAsync(d, h, one * ntabs, hipMemcpyHostToDevice, st));
    return HCCL_SUCCESS;
}

int fill_ptrs(const void *const *send, void *const *recv, uint32_t n, VRankPtrs *p)
{
    if (send == nullptr || recv == nullptr) return fail(HCCL_E_PTR, "send/recv pointer array is null");
    if (n == 0 || n > kMaxVRanks) return fail(HCCL_E_PARA, "rank count outside 1.." + std::to_string(kMaxVRanks));
    std::memset(p, 0, sizeof(*p));
    for (uint32_t i = 0; i < n; ++i) {
        p->send[i] = static_cast<const char *>(send[i]);
        p->recv[i] = static_cast<char *>(recv[i]);
    }
    return HCCL_SUCCESS;
}

}  // namespace

namespace hcclx {

uint64_t list_alltoallv_blocks(const void *const *send, void *const *recv, const uint64_t *send_counts,
                               const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, uint32_t esz, int unroll,
                               std::vector<CopyBlock> *blocks)
{
    blocks->clear();
    blocks->reserve(static_cast<size_t>(n) * n);
    uint64_t tiles = 0;
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t j = 0; j < n; ++j) {
            const uint64_t bytes = send_counts[i * n + j] * esz;
            if (bytes == 0) continue;
            CopyBlock b;
            b.src = static_cast<const char *>(send[i]) + sdispls[i * n + j] * esz;
            b.dst = static_cast<char *>(recv[j]) + rdispls[j * n + i] * esz;
            b.bytes = bytes;
            tiles += v_tiles_of(bytes, reinterpret_cast<uint64_t>(b.dst), unroll);
            b.tile_end = tiles;
            blocks->push_back(b);
        }
    }
    return tiles;
}

}  // namespace hcclx

extern "C" {

int hcclx_alltoallv(const void *const *send, void *const *recv, const uint64_t *send_counts,
                    const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, int dtype,
                    int tables_on_device, void *stream)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (!send_counts || !sdispls || !rdispls) return fail(HCCL_E_PTR, "count/displacement table is null");
    VRankPtrs ptrs;
    int rc = fill_ptrs(send, recv, n, &ptrs);
    if (rc != HCCL_SUCCESS) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!tables_on_device) {
        const int unroll = ctx->a2av_direct_unroll == 1 ? 1 : ctx->a2av_direct_unroll == 4 ? 4 : 2;
        bool small = n <= kA2avDirectRanks && ctx->a2av_direct_unroll != 0;
        for (size_t k = 0; k < static_cast<size_t>(n) * n && small; ++k) {
            small = send_counts[k] <= 0xffffffffull && sdispls[k] <= 0xffffffffull && rdispls[k] <= 0xffffffffull;
        }
        if (small) {
            // small host tables and their tile prefix ride in the kernel arguments: one small tile per workgroup,
            // nothing is copied in front of the kernel
            VRankPtrs16 p16;
            A2avTablesDirect tabs;
            std::memset(&p16, 0, sizeof(p16));
            std::memset(&tabs, 0, sizeof(tabs));
            for (uint32_t i = 0; i < n; ++i) {
                p16.send[i] = ptrs.send[i];
                p16.recv[i] = ptrs.recv[i];
            }
            uint64_t tiles = 0;
            for (uint32_t i = 0; i < n; ++i) {
                for (uint32_t j = 0; j < n; ++j) {
                    const uint32_t k = i * n + j;
                    const uint64_t dst = reinterpret_cast<uint64_t>(ptrs.recv[j]) + rdispls[j * n + i] * esz;
                    tiles += v_tiles_of(send_counts[k] * esz, dst, unroll);
                    tabs.send_counts[k] = static_cast<uint32_t>(send_counts[k]);
                    tabs.sdispls[k] = static_cast<uint32_t>(sdispls[k]);
                    tabs.rdispls[k] = static_cast<uint32_t>(rdispls[j * n + i]);
                    tabs.tile_end[k] = static_cast<uint32_t>(tiles);
                }
            }
            if (tiles == 0) return HCCL_SUCCESS;
            if (tiles <= 0x7fffffffull) {
                hipError_t e = launch_alltoallv_direct(p16, tabs, n, static_cast<uint32_t>(esz), static_cast<uint32_t>(tiles),
                                                       unroll, st);
                if (e != hipSuccess) return fail_hip(e, "alltoallv kernel launch");
                return HCCL_SUCCESS;
            }
        }
        // any other host table: the non-empty blocks as a list in device memory, one small tile per workgroup
        std::vector<CopyBlock> blocks;
        const uint64_t tiles = list_alltoallv_blocks(send, recv, send_counts, sdispls, rdispls, n, static_cast<uint32_t>(esz),
                                                     unroll, &blocks);
        if (blocks.empty()) return HCCL_SUCCESS;
        if (tiles > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
        char *h = nullptr;
        char *d = nullptr;
        rc = ring_reserve(ctx, blocks.size() * sizeof(CopyBlock), st, &h, &d);
        if (rc != HCCL_SUCCESS) return rc;
        std::memcpy(h, blocks.data(), blocks.size() * sizeof(CopyBlock));
        HCCLX_HIP(hipMemcpyAsync(d, h, blocks.size() * sizeof(CopyBlock), hipMemcpyHostToDevice, st));
        hipError_t e = launch_copy_blocks(reinterpret_cast<const CopyBlock *>(d), static_cast<uint32_t>(blocks.size()),
                                          static_cast<uint32_t>(tiles), unroll, st);
        if (e != hipSuccess) return fail_hip(e, "alltoallv kernel launch");
        return HCCL_SUCCESS;
    }
    // tables on the device: the tile count is not known here, so a persistent grid derives its own tile map
    const uint64_t grid = static_cast<uint64_t>(ctx->num_cus) * ctx->v_blocks_per_cu;
    const uint64_t *tabs[3] = {send_counts, sdispls, rdispls};
    const uint64_t *dev[3];
    rc = stage_tables(ctx, tabs, 3, static_cast<size_t>(n) * n, tables_on_device, st, dev);
    if (rc != HCCL_SUCCESS) return rc;
    hipError_t e = launch_alltoallv(ptrs, dev[0], dev[1], dev[2], n, static_cast<uint32_t>(esz),
                                    static_cast<uint32_t>(grid), 1u, st);
    if (e != hipSuccess) return fail_hip(e, "alltoallv kernel launch");
    return HCCL_SUCCESS;
}

int hcclx_allgatherv(const void *const *send, void *const *recv, const uint64_t *counts,
                     const uint64_t *displs, uint32_t n, int dtype, int tables_on_device, void *stream)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (!counts || !displs) return fail(HCCL_E_PTR, "count/displacement table is null");
    VRankPtrs ptrs;
    int rc = fill_ptrs(send, recv, n, &ptrs);
    if (rc != HCCL_SUCCESS) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint64_t grid = static_cast<uint64_t>(ctx->num_cus) * ctx->v_blocks_per_cu;
    if (!tables_on_device) {
        uint64_t payload = 0;
        for (uint32_t i = 0; i < n; ++i) payload += counts[i] * esz;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
        // Large, and not being captured into a graph (the job table is uploaded at call time): the outputs of a run of
        // a source are written one after the other.
        if (n > 1 && ctx->agv_phased_from != 0 && payload >= ctx->agv_phased_from && capturing == hipStreamCaptureStatusNone) {
            std::vector<PhasedStream> streams;
            for (uint32_t i = 0; i < n; ++i) {
                if (counts[i] == 0) continue;
                PhasedStream s;
                s.src = ptrs.send[i];
                s.bytes = counts[i] * esz;
                for (uint32_t d = 0; d < n; ++d) s.dst.push_back(ptrs.recv[d] + displs[i] * esz);
                streams.push_back(std::move(s));
            }
            std::vector<PhasedLaunch> launches;
            build_phased(streams, ctx->fanout_run, &launches);
            for (const PhasedLaunch &l : launches) {
                // Among up to 16 ranks a job's places are one offset into every receive buffer, and the jobs of a
                // launch usually fit the kernel arguments: no table in memory, nothing copied in front of the kernel.
                if (n <= kPhasedInlineRanks && l.jobs.size() <= kPhasedInlineJobs && l.nd <= n) {
                    PhasedInline tab;
                    std::memset(&tab, 0, sizeof(tab));
                    for (uint32_t d = 0; d < n; ++d) tab.base[d] = ptrs.recv[d];
                    bool same_offset = true;
                    for (size_t j = 0; j < l.jobs.size() && same_offset; ++j) {
                        tab.jobs[j] = l.jobs[j];
                        const uint64_t off = reinterpret_cast<uint64_t>(l.dsts[j * l.nd]) - reinterpret_cast<uint64_t>(ptrs.recv[0]);
                        tab.jobs[j].dst0 = off;
                        for (uint32_t d = 0; d < l.jobs[j].ndst; ++d) same_offset = same_offset && l.dsts[j * l.nd + d] == ptrs.recv[d] + off;
                    }
                    if (same_offset) {
                        hipError_t e = launch_phased_copy_inline(tab, static_cast<uint32_t>(l.jobs.size()), l.slots, l.nd, st);
                        if (e != hipSuccess) return fail_hip(e, "allgatherv kernel launch");
                        continue;
                    }
                }
                char *h = nullptr;
                char *d = nullptr;
                rc = ring_reserve(ctx, l.bytes(), st, &h, &d);
                if (rc != HCCL_SUCCESS) return rc;
                l.fill(h);
                HCCLX_HIP(hipMemcpyAsync(d, h, l.bytes(), hipMemcpyHostToDevice, st));
                hipError_t e = launch_phased_copy(reinterpret_cast<const PhasedJob *>(d),
                                                  reinterpret_cast<char *const *>(d + l.jobs_bytes()),
                                                  static_cast<uint32_t>(l.jobs.size()), l.slots, l.nd, st);
                if (e != hipSuccess) return fail_hip(e, "allgatherv kernel launch");
            }
            return HCCL_SUCCESS;
        }
        uint64_t total = 0;
        for (uint32_t i = 0; i < n; ++i) {
            total += v_tiles_of(counts[i] * esz, reinterpret_cast<uint64_t>(ptrs.recv[0]) + displs[i] * esz, kAgvUnroll);
        }
        if (total == 0) return HCCL_SUCCESS;
        grid = (total + ctx->v_tiles_per_block - 1) / ctx->v_tiles_per_block;
        if (grid > 0x7fffffffull) grid = 0x7fffffffull;
        AgvTablesInline tabs;   // host tables of up to 64 ranks always fit the kernel arguments
        std::memset(&tabs, 0, sizeof(tabs));
        for (uint32_t i = 0; i < n; ++i) {
            tabs.counts[i] = counts[i];
            tabs.displs[i] = displs[i];
        }
        hipError_t e = launch_allgatherv_inline(ptrs, tabs, n, static_cast<uint32_t>(esz), static_cast<uint32_t>(grid),
                                                ctx->v_tiles_per_block, st);
        if (e != hipSuccess) return fail_hip(e, "allgatherv kernel launch");
        return HCCL_SUCCESS;
    }
    const uint64_t *dev[2] = {counts, displs};
    hipError_t e = launch_allgatherv(ptrs, dev[0], dev[1], n, static_cast<uint32_t>(esz), static_cast<uint32_t>(grid), tables_on_device ? 1u : ctx->v_tiles_per_block, st);
    if (e != hipSuccess) return fail_hip(e, "allgatherv kernel launch");
    return HCCL_SUCCESS;
}

int hcclx_displs_from_counts(const uint64_t *counts, uint32_t rows, uint32_t n, uint64_t *displs, uint64_t *totals,
                             void *stream)
{
    if (!device_ctx()) return HCCL_E_RUNTIME;
    if (!counts || !displs) return fail(HCCL_E_PTR, "counts or displs is null");
    if (n == 0 || n > kMaxVRanks) return fail(HCCL_E_PARA, "rank count outside 1.." + std::to_string(kMaxVRanks));
    if (rows == 0) return HCCL_SUCCESS;
    if (rows > 0x7fffffffu) return fail(HCCL_E_PARA, "too many rows");
    hipError_t e = launch_displs_from_counts(counts, rows, n, displs, totals, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(e, "displacement kernel launch");
    return HCCL_SUCCESS;
}

}  // extern "C"
