// What a collective costs the host the first time, on other buffers, and from then on, from C++: one host thread
// issues every rank's call.  For every AllReduce and ReduceScatter template among 8, 16, 32 and 64 ranks
// (1 Mi fp32 per rank for AllReduce, 1 Mi per rank received for ReduceScatter):
//   first_ms   the first call of the shape: templates run, steps ordered and traced (or the template's closed form
//              taken), tables built and uploaded; the world has run one small collective of another shape before
//   moved_us   the same call on buffers somewhere else: the first plan moved there, tables through the ring
//   again_us   those buffers a second time: device tables of their own are made
//   replay_us  and a third time: the plan found by its addresses and launched
// Each figure is host time from the first rank's call to the return of the last rank's, nothing waited for; the
// stream is drained between the calls.  Prints one JSON object.
//
//   make -C hccl_amd/csrc            (builds hccl_amd/lib/first_call_virtual_ranks)
//   hccl_amd/lib/first_call_virtual_ranks [max_ranks]
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
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
    const uint32_t max_ranks = argc > 1 ? static_cast<uint32_t>(std::atoi(argv[1])) : 64;
    const uint64_t count = 1u << 20;
    struct Case {
        bool scatter;
        const char *alg;
    };
    const Case cases[] = {
        {false, "InsAllReduceMesh1DOneShot"},  {false, "InsAllReduceMesh1DTwoShot"},
        {false, "InsAllReduceMesh1DTwoShotMeshChunk"}, {false, "InsAllReduceNHR"},
        {false, "InsAllReduceRHD"},            {false, "InsAllReduceRing"},
        {false, "InsAllReduceAicpuReduceNHR"}, {true, "InsReduceScatterMesh1D"},
        {true, "InsReduceScatterMesh1DMeshChunk"}, {true, "InsReduceScatterNHR"},
        {true, "InsReduceScatterAicpuReduceNHR"},
    };
    hipStream_t stream;
    CHECK_HIP(hipStreamCreate(&stream));
    std::printf("{\"elements_per_rank\": %llu, \"dtype\": \"fp32\", \"op\": \"sum\", \"rows\": [",
                static_cast<unsigned long long>(count));
    bool first = true;
    for (uint32_t n : {8u, 16u, 32u, 64u}) {
        if (n > max_ranks) break;
        // two sets of buffers per rank; a ReduceScatter sends n * count / n = count elements too (count / n received)
        std::vector<float *> send[2], recv[2];
        for (int set = 0; set < 2; ++set) {
            send[set].resize(n);
            recv[set].resize(n);
            for (uint32_t r = 0; r < n; ++r) {
                CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&send[set][r]), count * sizeof(float)));
                CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&recv[set][r]), count * sizeof(float)));
                CHECK_HIP(hipMemset(send[set][r], 0, count * sizeof(float)));
            }
        }
        for (const Case &c : cases) {
            std::vector<HcclComm> comm(n);
            CHECK_HCCL(HcclCommInitAll(n, nullptr, comm.data()));
            CHECK_HCCL(hcclxCommSetAlgorithm(comm[0], c.scatter ? HCCLX_CMD_REDUCE_SCATTER : HCCLX_CMD_ALLREDUCE, c.alg));
            // one small collective of another shape first: the process' first launch of a kernel and the world's first
            // table allocation are paid there, not in the figures below
            for (uint32_t r = 0; r < n; ++r) {
                if (c.scatter) {
                    CHECK_HCCL(HcclReduceScatter(send[0][r], recv[0][r], 3, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm[r],
                                                 stream));
                } else {
                    CHECK_HCCL(HcclAllReduce(send[0][r], recv[0][r], 3 * n + 1, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM, comm[r],
                                             stream));
                }
            }
            CHECK_HIP(hipStreamSynchronize(stream));
            double us[4] = {0, 0, 0, 0};
            int hit[4] = {0, 0, 0, 0};
            hcclxLastOpInfo info;
            std::memset(&info, 0, sizeof(info));
            for (int call = 0; call < 4; ++call) {
                const int set = call == 0 ? 0 : 1;
                const auto h0 = std::chrono::steady_clock::now();
                for (uint32_t r = 0; r < n; ++r) {
                    if (c.scatter) {
                        CHECK_HCCL(HcclReduceScatter(send[set][r], recv[set][r], count / n, HCCL_DATA_TYPE_FP32,
                                                     HCCL_REDUCE_SUM, comm[r], stream));
                    } else {
                        CHECK_HCCL(HcclAllReduce(send[set][r], recv[set][r], count, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM,
                                                 comm[r], stream));
                    }
                }
                const auto h1 = std::chrono::steady_clock::now();
                CHECK_HIP(hipStreamSynchronize(stream));
                us[call] = std::chrono::duration<double, std::micro>(h1 - h0).count();
                CHECK_HCCL(hcclxCommGetLastOpInfo(comm[0], &info));
                hit[call] = info.planCacheHit;
            }
            std::printf("%s\n{\"ranks\": %u, \"algorithm\": \"%s\", \"first_ms\": %.3f, \"moved_us\": %.1f, \"again_us\": %.1f, "
                        "\"replay_us\": %.1f, \"cache\": [%d, %d, %d, %d], \"fused\": %d, \"launches\": %u, \"segments\": %u}",
                        first ? "" : ",", n, c.alg, us[0] / 1e3, us[1], us[2], us[3], hit[0], hit[1], hit[2], hit[3],
                        info.fused, info.launches, info.fusedSegments);
            std::fflush(stdout);
            first = false;
            for (uint32_t r = 0; r < n; ++r) CHECK_HCCL(HcclCommDestroy(comm[r]));
        }
        for (int set = 0; set < 2; ++set) {
            for (uint32_t r = 0; r < n; ++r) {
                (void)hipFree(send[set][r]);
                (void)hipFree(recv[set][r]);
            }
        }
    }
    std::printf("\n]}\n");
    return 0;
}
