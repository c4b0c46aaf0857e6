// Launch interface of the V-collective kernels (vops.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "launch.h"

namespace hcclx {

constexpr uint32_t kMaxVRanks = 64;

// Tile geometry of the V kernels: 256 threads x `unroll` vectors of 16 bytes per tile.
// 16-byte vectors each thread moves per tile.  AlltoAllV stages and scans an n x n table per workgroup, so its
// tiles are large (32 KiB); AllGatherV's set-up is n entries, and small tiles (4 KiB: every workgroup sweeps
// a compact range and retires quickly) measured faster for its write-heavy traffic.
#ifndef HCCLX_A2AV_UNROLL
#define HCCLX_A2AV_UNROLL 8
#endif
#ifndef HCCLX_AGV_UNROLL
#define HCCLX_AGV_UNROLL 1
#endif
constexpr int kA2avUnroll = HCCLX_A2AV_UNROLL;
constexpr int kAgvUnroll = HCCLX_AGV_UNROLL;
// The copies that write one output at a time (large AllGatherV, fan-out of a fold's result): 8 KiB tiles.
#ifndef HCCLX_PHASED_UNROLL
#define HCCLX_PHASED_UNROLL 2
#endif
constexpr int kPhasedUnroll = HCCLX_PHASED_UNROLL;

// Tiles of a block of `bytes` bytes whose first destination byte sits at address `dst`.  Stores are
// aligned: the bytes before the first 16-byte boundary of dst (head) and after the last whole vector
// (tail) are moved one byte per thread by the block's last tile.  Used by the kernels and, when the
// tables are on the host, by the launcher to size the grid exactly.
// The tile grid of a block is shifted by v_shift_of() vectors so that every wavefront's 64 x 16 bytes start
// on a 1 KiB boundary of dst: whole cache lines are stored.  The first tile is then partial.
__host__ __device__ inline uint64_t v_head_of(uint64_t bytes, uint64_t dst)
{
    const uint64_t head = (16 - (dst & 15)) & 15;
    return head > bytes ? bytes : head;
}
__host__ __device__ inline uint32_t v_shift_of(uint64_t head, uint64_t dst)
{
    return static_cast<uint32_t>(((dst + head) & 1023) / 16);
}
__host__ __device__ inline uint64_t v_tiles_of(uint64_t bytes, uint64_t dst, int unroll)
{
    const uint64_t kTileVecs = 256ull * unroll;
    if (bytes == 0) return 0;
    const uint64_t head = v_head_of(bytes, dst);
    return ((bytes - head) / 16 + v_shift_of(head, dst)) / kTileVecs + 1;
}

// Base pointers of every virtual rank's send and receive buffer, passed by value as a kernel argument.
struct VRankPtrs {
    const char *send[kMaxVRanks];
    char *recv[kMaxVRanks];
};

// Count / displacement tables as the kernels read them.  Host tables of up to 15 ranks travel inside the kernel
// arguments (no host-to-device copy is queued in front of the kernel); larger host tables become a list of
// blocks in device memory; tables that already live on the device are read through pointers.
struct A2avTablesPtr {
    const uint64_t *send_counts;
    const uint64_t *sdispls;
    const uint64_t *rdispls;
    __device__ uint64_t count(uint32_t p) const { return send_counts[p]; }
    __device__ uint64_t sdispl(uint32_t p) const { return sdispls[p]; }
    __device__ uint64_t rdispl(uint32_t p) const { return rdispls[p]; }
};
// Host tables of up to 15 ranks with the tile prefix worked out by the host: a workgroup finds its block
// with a binary search over kernel arguments (scalar loads), with no LDS table and no barrier, which is
// what makes 4 KiB tiles affordable.  15 x 15 x 4 tables of uint32 = 3600 bytes of kernel arguments.
constexpr uint32_t kA2avDirectRanks = 15;
struct A2avTablesDirect {
    uint32_t send_counts[kA2avDirectRanks * kA2avDirectRanks];
    uint32_t sdispls[kA2avDirectRanks * kA2avDirectRanks];
    uint32_t rdispls[kA2avDirectRanks * kA2avDirectRanks];   // indexed like send_counts: block (i, j) at i * n + j
    uint32_t tile_end[kA2avDirectRanks * kA2avDirectRanks];  // inclusive prefix of tiles per block
};
// Base pointers for the launch with tables in the kernel arguments.
struct VRankPtrs16 {
    const char *send[16];
    char *recv[16];
};
// One contiguous block to move, for host tables of any size: the host lists the non-empty blocks with the
// inclusive prefix of their tiles; a workgroup finds its block with a binary search over that list (scalar loads).
struct CopyBlock {
    const char *src;
    char *dst;
    uint64_t bytes;
    uint64_t tile_end;
};
struct AgvTablesPtr {
    const uint64_t *counts;
    const uint64_t *displs;
    __device__ uint64_t count(uint32_t i) const { return counts[i]; }
    __device__ uint64_t displ(uint32_t i) const { return displs[i]; }
};
// One job of the copy kernel that writes one output at a time: `bytes` bytes from src to ndst places (the
// launch's pointer array holds them at [job * nd, job * nd + ndst)), cut into `tiles` tiles laid out for the
// alignment of the first place, whose address is dst0.
struct PhasedJob {
    const char *src;
    uint64_t bytes;
    uint64_t dst0;
    uint32_t ndst;
    uint32_t tiles;
};
// The same for an AllGather(V) among up to 16 ranks whose jobs fit the kernel arguments: every place a job goes to
// is the same offset (the job's dst0) into the ranks' receive buffers, so the launch needs no table in memory.
constexpr uint32_t kPhasedInlineJobs = 100;
constexpr uint32_t kPhasedInlineRanks = 16;
struct PhasedInline {
    char *base[kPhasedInlineRanks];
    PhasedJob jobs[kPhasedInlineJobs];
};
struct AgvTablesInline {
    uint64_t counts[kMaxVRanks];
    uint64_t displs[kMaxVRanks];
    __device__ uint64_t count(uint32_t i) const { return counts[i]; }
    __device__ uint64_t displ(uint32_t i) const { return displs[i]; }
};

// blocks: device array of nblocks entries; unroll: 1, 2 or 4; grid = total number of tiles
hipError_t launch_copy_blocks(const CopyBlock *blocks, uint32_t nblocks, uint32_t grid, int unroll, hipStream_t stream);
// jobs, dsts: device arrays of njobs and njobs * nd entries; slots: tiles of the longest job; slots * nd < 2^31,
// njobs < 65536
hipError_t launch_phased_copy(const PhasedJob *jobs, char *const *dsts, uint32_t njobs, uint32_t slots, uint32_t nd,
                              hipStream_t stream);
hipError_t launch_phased_copy_inline(const PhasedInline &tab, uint32_t njobs, uint32_t slots, uint32_t nd, hipStream_t stream);
// unroll: 1, 2 or 4 vectors per thread and tile; grid = total number of tiles
hipError_t launch_alltoallv_direct(const VRankPtrs16 &ptrs, const A2avTablesDirect &tabs, uint32_t n, uint32_t esz,
                                   uint32_t grid, int unroll, hipStream_t stream);
hipError_t launch_allgatherv_inline(const VRankPtrs &ptrs, const AgvTablesInline &tabs, uint32_t n, uint32_t esz,
                                    uint32_t grid, uint32_t tiles_per_block, hipStream_t stream);

// send_counts / sdispls / rdispls: device pointers, uint64 elements, row-major n x n.
hipError_t launch_alltoallv(const VRankPtrs &ptrs, const uint64_t *send_counts, const uint64_t *sdispls,
                            const uint64_t *rdispls, uint32_t n, uint32_t esz, uint32_t grid, uint32_t tiles_per_block,
                            hipStream_t stream);

// counts / displs: device pointers, uint64 elements, n entries.
hipError_t launch_displs_from_counts(const uint64_t *counts, uint32_t rows, uint32_t n, uint64_t *displs, uint64_t *totals,
                                     hipStream_t stream);
hipError_t launch_allgatherv(const VRankPtrs &ptrs, const uint64_t *counts, const uint64_t *displs, uint32_t n,
                             uint32_t esz, uint32_t grid, uint32_t tiles_per_block, hipStream_t stream);
}  // namespace hcclx
