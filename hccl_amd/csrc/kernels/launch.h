// Every kernel launch of the library goes through HCCLX_LAUNCH, which counts it for the calling host thread
// (hcclx_kernels_launched): the host runtime reports how many kernels a collective took from that count.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hcclx {
inline uint64_t &kernels_launched()
{
    static thread_local uint64_t n = 0;
    return n;
}
}  // namespace hcclx

#define HCCLX_LAUNCH(...)                    \
    do {                                     \
        ++::hcclx::kernels_launched();       \
        hipLaunchKernelGGL(__VA_ARGS__);     \
    } while (0)
