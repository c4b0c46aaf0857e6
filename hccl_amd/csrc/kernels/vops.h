// Launch interface of the V-collective kernels (vops.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hcclx {

constexpr uint32_t kMaxVRanks = 64;

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
