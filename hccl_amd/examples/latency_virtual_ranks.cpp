// Time per warm HcclAllReduce for small messages, from C++: one host thread issues every rank's call, no HIP graph.
// Cases: 8 ranks fp32 SUM with the selector's choice and through the ring template, 4 KiB ... 4 MiB per rank (the
// largest is the 8 x 1,048,576-element AllReduce), and 12 ranks int32 MAX / fp32 PROD through the NHR,
// halving-doubling and CPU-reduce NHR templates, 4 KiB ... 1 MiB per rank.
// Prints one JSON object: per (case, bytes per rank) the microseconds per collective on the GPU timeline
// ("us": events around `reps` collectives, i.e. the sustained rate) and the host time spent issuing one collective
// ("host_us": all ranks' calls, nothing waited for).
//
//   make -C hccl_amd/csrc            (builds hccl_amd/lib/latency_virtual_ranks)
//   hccl_amd/lib/latency_virtual_ranks [reps]
#include <hip/hip_runtime.h>

#include <chrono>
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
    const int reps = argc > 1 ? std::atoi(argv[1]) : 200;
    if (reps <= 0) {
        std::fprintf(stderr, "usage: %s [reps > 0]\n", argv[0]);
        return 2;
    }
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    hipEvent_t t0, t1;
    CHECK_HIP(hipEventCreate(&t0));
    CHECK_HIP(hipEventCreate(&t1));
    struct Case {
        const char *name;
        uint32_t ranks;
        HcclDataType dtype;
        HcclReduceOp op;
        const char *alg;   // nullptr: the selector decides
        size_t max_bytes;
    };
    const Case cases[] = {
        {"fp32_sum_default", 8, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, nullptr, 4u << 20},
        {"fp32_sum_ring", 8, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, "InsAllReduceRing", 4u << 20},
        {"fp32_sum_default", 12, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, nullptr, 1u << 20},
        {"int32_max_nhr", 12, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_MAX, "InsAllReduceNHR", 1u << 20},
        {"int32_max_rhd", 12, HCCL_DATA_TYPE_INT32, HCCL_REDUCE_MAX, "InsAllReduceRHD", 1u << 20},
        {"fp32_prod_aicpu_nhr", 12, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_PROD, "InsAllReduceAicpuReduceNHR", 1u << 20},
        {"fp32_prod_rhd", 12, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_PROD, "InsAllReduceRHD", 1u << 20},
    };
    std::printf("{\"reps\": %d, \"op\": \"HcclAllReduce\", \"rows\": [", reps);
    bool first = true;
    for (const Case &c : cases) {
        const uint32_t n = c.ranks;
        const size_t max_bytes = c.max_bytes;
        std::vector<HcclComm> comm(n);
        CHECK_HCCL(HcclCommInitAll(n, nullptr, comm.data()));
        if (c.alg) CHECK_HCCL(hcclxCommSetAlgorithm(comm[0], HCCLX_CMD_ALLREDUCE, c.alg));
        std::vector<float *> send(n), recv(n);
        for (uint32_t r = 0; r < n; ++r) {
            CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&send[r]), max_bytes));
            CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&recv[r]), max_bytes));
            CHECK_HIP(hipMemset(send[r], 0, max_bytes));
        }
        for (size_t bytes = 4096; bytes <= max_bytes; bytes *= 4) {
            const uint64_t count = bytes / sizeof(float);
            auto all_ranks = [&]() -> int {
                for (uint32_t r = 0; r < n; ++r) {
                    CHECK_HCCL(HcclAllReduce(send[r], recv[r], count, c.dtype, c.op, comm[r], stream));
                }
                return 0;
            };
            for (int k = 0; k < 3; ++k) {
                if (all_ranks()) return 1;   // the first call plans the launch
            }
            CHECK_HIP(hipStreamSynchronize(stream));
            if (bytes >= (1u << 20)) {
                // sizes whose kernel outweighs the launch: 20 ms of the same collective first, so that the figure is
                // that of a busy GPU and not of the clock transient after an idle period
                const auto r0 = std::chrono::steady_clock::now();
                while (std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - r0).count() < 20.0) {
                    for (int k = 0; k < 20; ++k) {
                        if (all_ranks()) return 1;
                    }
                    CHECK_HIP(hipStreamSynchronize(stream));
                }
            }
            CHECK_HIP(hipEventRecord(t0, stream));
            const auto h0 = std::chrono::steady_clock::now();
            for (int k = 0; k < reps; ++k) {
                if (all_ranks()) return 1;
            }
            const auto h1 = std::chrono::steady_clock::now();
            CHECK_HIP(hipEventRecord(t1, stream));
            CHECK_HIP(hipStreamSynchronize(stream));
            float ms = 0;
            CHECK_HIP(hipEventElapsedTime(&ms, t0, t1));
            const double host_us = std::chrono::duration<double, std::micro>(h1 - h0).count() / reps;
            hcclxLastOpInfo info;
            CHECK_HCCL(hcclxCommGetLastOpInfo(comm[0], &info));
            std::printf("%s{\"case\": \"%s\", \"ranks\": %u, \"bytes_per_rank\": %zu, \"us\": %.2f, \"host_us\": %.2f, "
                        "\"algorithm\": \"%s\", \"plan_cache_hit\": %s}",
                        first ? "" : ", ", c.name, n, bytes, ms * 1e3 / reps, host_us, info.algName,
                        info.planCacheHit ? "true" : "false");
            first = false;
        }
        for (uint32_t r = 0; r < n; ++r) {
            CHECK_HCCL(HcclCommDestroy(comm[r]));
            (void)hipFree(send[r]);
            (void)hipFree(recv[r]);
        }
    }
    std::printf("]}\n");
    return 0;
}
