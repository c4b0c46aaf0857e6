// Launch interface of the V-collective kernels (vops.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hcclx {

constexpr uint32_t kMaxVRanks = 64;

// Tile geometry of the V kernels: 256 threads x 8 vectors of 16 bytes = 32 KiB per tile.
constexpr int kCopyUnroll = 8;
constexpr uint32_t kTileVecs = 256 * kCopyUnroll;

// Tiles of a block of `bytes` bytes whose first destination byte sits at address `dst`.  Stores are
// aligned: the bytes before the first 16-byte boundary of dst (head) and after the last whole vector
// (tail) are moved one byte per thread by the block's last tile.  Used by the kernels and, when the
// tables are on the host, by the launcher to size the grid exactly.
__host__ __device__ inline uint64_t v_tiles_of(uint64_t bytes, uint64_t dst)
{
    if (bytes == 0) return 0;
    uint64_t head = (16 - (dst & 15)) & 15;
    if (head > bytes) head = bytes;
    return (bytes - head) / 16 / kTileVecs + 1;
}

// Base pointers of every virtual rank's send and receive buffer, passed by value as a kernel argument.
struct VRankPtrs {
    const char *send[kMaxVRanks];
    char *recv[kMaxVRanks];
};

// send_counts / sdispls / rdispls: device pointers, uint64 elements, row-major n x n.
hipError_t launch_alltoallv(const VRankPtrs &ptrs, const uint64_t *send_counts, const uint64_t *sdispls,
                            const uint64_t *rdispls, uint32_t n, uint32_t esz, uint32_t grid, hipStream_t stream);

// counts / displs: device pointers, uint64 elements, n entries.
hipError_t launch_allgatherv(const VRankPtrs &ptrs, const uint64_t *counts, const uint64_t *displs, uint32_t n,
                             uint32_t esz, uint32_t grid, hipStream_t stream);

}  // namespace hcclx
