// HcclAllReduce among N virtual ranks of one GPU, from C++, the way an application of the reference calls it
// (include/hccl.h:65-66 of the reference: the same signature), with one host thread driving all ranks.
//
//   make -C hccl_amd/csrc            (builds the library and hccl_amd/lib/allreduce_virtual_ranks)
//   hccl_amd/lib/allreduce_virtual_ranks [ranks] [MiB per rank]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "hccl.h"
#include "hccl_comm.h"

#define CHECK_HIP(x)                                                                   \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));               \
            return 1;                                                                  \
        }                                                                              \
    } while (0)
#define CHECK_HCCL(x)                                                                  \
    do {                                                                               \
        HcclResult r_ = (x);                                                           \
        if (r_ != HCCL_SUCCESS) {                                                      \
            std::fprintf(stderr, "%s: HcclResult %d\n", #x, static_cast<int>(r_));     \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

int main(int argc, char **argv)
{
    const uint32_t n = argc > 1 ? static_cast<uint32_t>(std::atoi(argv[1])) : 8;
    const size_t mib = argc > 2 ? static_cast<size_t>(std::atoi(argv[2])) : 16;
    const uint64_t count = mib * 1024 * 1024 / sizeof(float);
    if (n == 0 || n > 64 || count == 0) {
        std::fprintf(stderr, "usage: %s [ranks 1..64] [MiB per rank]\n", argv[0]);
        return 2;
    }

    std::vector<HcclComm> comm(n);
    CHECK_HCCL(HcclCommInitAll(n, nullptr, comm.data()));
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));

    // rank r holds r + 1 everywhere, so every element of the result is n (n + 1) / 2
    std::vector<float *> send(n), recv(n);
    std::vector<float> host(count);
    for (uint32_t r = 0; r < n; ++r) {
        CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&send[r]), count * sizeof(float)));
        CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&recv[r]), count * sizeof(float)));
        for (uint64_t i = 0; i < count; ++i) host[i] = static_cast<float>(r + 1);
        CHECK_HIP(hipMemcpy(send[r], host.data(), count * sizeof(float), hipMemcpyHostToDevice));
    }

    auto all_ranks = [&]() -> int {
        for (uint32_t r = 0; r < n; ++r) {   // queued per rank; the last rank's call launches the collective
            CHECK_HCCL(HcclAllReduce(send[r], recv[r], count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm[r], stream));
        }
        return 0;
    };
    if (all_ranks()) return 1;   // the first call plans the launch and keeps the plan
    CHECK_HIP(hipStreamSynchronize(stream));

    hipEvent_t t0, t1;
    CHECK_HIP(hipEventCreate(&t0));
    CHECK_HIP(hipEventCreate(&t1));
    const int reps = 20;
    CHECK_HIP(hipEventRecord(t0, stream));
    for (int k = 0; k < reps; ++k) {
        if (all_ranks()) return 1;
    }
    CHECK_HIP(hipEventRecord(t1, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, t0, t1));

    hcclxLastOpInfo info;
    CHECK_HCCL(hcclxCommGetLastOpInfo(comm[0], &info));
    const float want = static_cast<float>(n) * static_cast<float>(n + 1) / 2;
    bool ok = true;
    for (uint32_t r = 0; r < n; ++r) {
        CHECK_HIP(hipMemcpy(host.data(), recv[r], count * sizeof(float), hipMemcpyDeviceToHost));
        for (uint64_t i = 0; i < count && ok; ++i) ok = host[i] == want;
    }
    const double bytes = 2.0 * n * count * sizeof(float);   // every input read once, every output written once
    std::printf("%s: %u ranks x %zu MiB, %s, %u launch(es), %.1f us per collective, %.0f GB/s -- %s\n", info.algName, n, mib,
                info.fused ? "one pass" : "step by step", info.launches, ms * 1e3 / reps, bytes / (ms * 1e-3 / reps) / 1e9,
                ok ? "OK" : "WRONG RESULT");

    for (uint32_t r = 0; r < n; ++r) {
        CHECK_HCCL(HcclCommDestroy(comm[r]));
        (void)hipFree(send[r]);
        (void)hipFree(recv[r]);
    }
    return ok ? 0 : 1;
}
