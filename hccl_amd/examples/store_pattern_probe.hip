// What bounds a fold whose N results go to N places: a stand-alone measurement, no part of the library.
//
// The N orders of a one-shot AllReduce (ins_temp_all_reduce_mesh_1D_one_shot.cc:182-197) and of the CPU-reduce NHR
// AllReduce (ins_temp_all_reduce_aicpu_reduce_nhr.cc:212-236) read N buffers and write N buffers of the same size:
// half the traffic is stores, to N streams at once.  This program measures, on N = 12 streams of the size given,
//   - the ceilings: reading the 12 streams; filling them with every workgroup writing all 12 (12 stores per
//     wavefront in a row), and with one wavefront per stream (1, 4 or 12 stores per wavefront, one stream each);
//   - the fold held in registers (the pattern of k_fold<..., self-first>) as it is and in four variants of its tile
//     order and store order;
//   - the fold with one wavefront per source and destination and the pieces staged in LDS (the pattern of
//     k_fold_waves), 1 and 4 pieces per workgroup;
// and prints time, GB/s and the fraction of 8 TB/s for each.  Every variant is a kernel of its own name, so a
// profiler's per-kernel counters tell them apart.
//
//   hccl_amd/lib/store_pattern_probe [MiB per stream, default 64] [launches timed per variant, default 10]
// (a variant that draws more power than the others only shows it over many launches in a row: try 100)
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef const u32x4 __attribute__((address_space(1))) *global_cvec;
typedef u32x4 __attribute__((address_space(1))) *global_vec;

#define CHECK(x)                                                              \
    do {                                                                      \
        hipError_t e_ = (x);                                                  \
        if (e_ != hipSuccess) {                                               \
            std::printf("%s: %s\n", #x, hipGetErrorString(e_));               \
            std::exit(1);                                                     \
        }                                                                     \
    } while (0)

constexpr int N = 12;          // streams
constexpr int kThreads = 256;  // the register kernels' workgroup
struct Streams {
    const char *src[N];
    char *dst[N];
};

__device__ __forceinline__ u32x4 ld16(const char *p) { return __builtin_nontemporal_load((global_cvec)p); }
__device__ __forceinline__ void st16(char *p, u32x4 v) { __builtin_nontemporal_store(v, (global_vec)p); }
__device__ __forceinline__ float4 as_f4(u32x4 v) { return *reinterpret_cast<float4 *>(&v); }
__device__ __forceinline__ u32x4 as_u4(float4 v) { return *reinterpret_cast<u32x4 *>(&v); }
__device__ __forceinline__ float4 mul(float4 x, float4 acc) { return make_float4(x.x * acc.x, x.y * acc.y, x.z * acc.z, x.w * acc.w); }

__global__ void __launch_bounds__(kThreads) probe_read(Streams s, char *sink)
{
    const uint64_t off = (static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x) * 16;
    u32x4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < N; ++k) acc ^= ld16(s.src[k] + off);
    if (acc.x == 0x12345678u && acc.y == 77u) *reinterpret_cast<u32x4 *>(sink) = acc;   // never true: keeps the loads
}

// every workgroup writes its 4 KiB tile of all N streams: N stores per wavefront, one after the other
__global__ void __launch_bounds__(kThreads) probe_fill_every_workgroup_all_streams(Streams s)
{
    const uint64_t off = (static_cast<uint64_t>(blockIdx.x) * kThreads + threadIdx.x) * 16;
    const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
#pragma unroll
    for (int j = 0; j < N; ++j) st16(s.dst[j] + off, v);
}

// a workgroup of N wavefronts, wavefront j writes M pieces of 1 KiB of stream j only
template <int M>
__global__ void __launch_bounds__(N * 64) probe_fill_wavefront_per_stream(Streams s)
{
    const int j = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const u32x4 v = {threadIdx.x, blockIdx.x, 3u, 4u};
    char *dst = s.dst[j] + static_cast<uint64_t>(blockIdx.x) * M * 1024 + lane * 16;
#pragma unroll
    for (int m = 0; m < M; ++m) st16(dst + m * 1024, v);
}

__device__ __forceinline__ uint64_t xcd_contiguous(uint64_t t, uint64_t total)
{
    // workgroups go to the eight XCDs in turn: give each XCD a contiguous eighth of the tiles
    const uint64_t q = total / 8, r = total % 8, xcd = t % 8;
    return xcd * q + (xcd < r ? xcd : r) + t / 8;
}

// The fold in registers: every thread loads U vectors of each of the N sources and stores the N results.
//   U        vectors per thread (tile = U x 4 KiB per stream)
//   RUN      consecutive tiles a workgroup takes
//   XCD      tiles in XCD-contiguous order
//   BY_DEST  all of a thread's vectors go to one destination before the next (else: vector by vector)
template <int U, int RUN, bool XCD, bool BY_DEST>
__global__ void __launch_bounds__(kThreads) probe_fold_registers(Streams s, uint64_t tiles)
{
    const uint64_t chunks = (tiles + RUN - 1) / RUN;
    const uint64_t c = XCD ? xcd_contiguous(blockIdx.x, chunks) : blockIdx.x;
    for (int i = 0; i < RUN; ++i) {
        const uint64_t t = c * RUN + i;
        if (t >= tiles) break;
        const uint64_t off = (t * (kThreads * U) + threadIdx.x) * 16;
        float4 val[U][N];
#pragma unroll
        for (int k = 0; k < N; ++k) {
#pragma unroll
            for (int u = 0; u < U; ++u) val[u][k] = as_f4(ld16(s.src[k] + off + static_cast<uint64_t>(u) * kThreads * 16));
        }
        auto result = [&](int u, int j) {
            float4 acc = val[u][j];   // output j starts from source j, then the others ascending
#pragma unroll
            for (int k = 0; k < N; ++k) {
                if (k != j) acc = mul(val[u][k], acc);
            }
            return as_u4(acc);
        };
        if (BY_DEST) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
#pragma unroll
                for (int u = 0; u < U; ++u) st16(s.dst[j] + off + static_cast<uint64_t>(u) * kThreads * 16, result(u, j));
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int j = 0; j < N; ++j) st16(s.dst[j] + off + static_cast<uint64_t>(u) * kThreads * 16, result(u, j));
            }
        }
    }
}

// The fold with one wavefront per source / destination: wavefront w loads a 1 KiB piece of source w into LDS; after
// the barrier it reads all N pieces, folds them in the order of output w and stores the piece of destination w: one
// load and one store per wavefront and piece.  P pieces per workgroup, the next piece's load issued before the fold.
template <int P>
__global__ void __launch_bounds__(N * 64) probe_fold_wavefronts(Streams s, uint64_t pieces)
{
    __shared__ float4 buf[2][N][64];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const char *src = s.src[w];
    char *dst = s.dst[w];
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * P;
    u32x4 next = ld16(src + (first * 64 + lane) * 16);
#pragma unroll 1
    for (int i = 0; i < P; ++i) {
        const uint64_t piece = first + i;
        if (piece >= pieces) break;
        buf[i & 1][w][lane] = as_f4(next);
        if (i + 1 < P && piece + 1 < pieces) next = ld16(src + ((piece + 1) * 64 + lane) * 16);
        __syncthreads();
        float4 acc = buf[i & 1][w][lane];
#pragma unroll
        for (int base = 0; base < N; base += 4) {
            float4 x[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) x[k] = buf[i & 1][base + k][lane];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float4 r = mul(x[k], acc);
                const bool take = (base + k) != w;
                acc = make_float4(take ? r.x : acc.x, take ? r.y : acc.y, take ? r.z : acc.z, take ? r.w : acc.w);
            }
        }
        st16(dst + (piece * 64 + lane) * 16, as_u4(acc));
    }
}

__global__ void probe_init(float *p, uint64_t n, float v)
{
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull) p[i] = v + (i % 97) * 1e-4f;
}

__global__ void probe_count_differences(const uint32_t *a, const uint32_t *b, uint64_t n, unsigned long long *bad)
{
    for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += gridDim.x * 256ull) {
        if (a[i] != b[i]) atomicAdd(bad, 1ull);
    }
}

int g_reps = 10;   // launches timed per variant

template <typename F>
float time_us(F launch)
{
    const int reps = g_reps;
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    for (int i = 0; i < 2; ++i) launch();
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(a));
    for (int i = 0; i < reps; ++i) launch();
    CHECK(hipEventRecord(b));
    CHECK(hipEventSynchronize(b));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, a, b));
    CHECK(hipEventDestroy(a));
    CHECK(hipEventDestroy(b));
    return ms * 1000 / reps;
}

int main(int argc, char **argv)
{
    const uint64_t mib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 64;
    if (argc > 2) g_reps = std::atoi(argv[2]);
    if (mib == 0 || mib > 2048 || g_reps < 1 || g_reps > 10000) {
        std::printf("usage: store_pattern_probe [MiB per stream, 1..2048] [launches timed per variant, 1..10000]\n");
        return 2;
    }
    const uint64_t bytes = mib << 20;   // a multiple of every tile size used below
    Streams a{}, b{};                   // the same sources, two sets of destinations (to compare two kernels' results)
    for (int k = 0; k < N; ++k) {
        char *src, *d0, *d1;
        CHECK(hipMalloc(&src, bytes));
        CHECK(hipMalloc(&d0, bytes));
        CHECK(hipMalloc(&d1, bytes));
        a.src[k] = b.src[k] = src;
        a.dst[k] = d0;
        b.dst[k] = d1;
        hipLaunchKernelGGL(probe_init, dim3(4096), dim3(256), 0, 0, reinterpret_cast<float *>(src), bytes / 4, 0.95f + 0.01f * k);
    }
    char *sink;
    unsigned long long *bad;
    CHECK(hipMalloc(&sink, 64));
    CHECK(hipMalloc(&bad, 8));
    CHECK(hipMemset(bad, 0, 8));
    CHECK(hipDeviceSynchronize());

    const uint64_t tiles = bytes / 4096;   // 4 KiB tiles per stream
    const uint64_t pieces = bytes / 1024;  // 1 KiB pieces per stream
    std::printf("%d streams of %llu MiB, %d launches timed per variant; fractions are of 8000 GB/s\n", N,
                static_cast<unsigned long long>(mib), g_reps);
    auto report = [&](const char *name, float us, int streams_moved) {
        const double gbs = static_cast<double>(streams_moved) * bytes / us / 1e3;
        std::printf("%-64s %9.1f us %7.0f GB/s  %.3f\n", name, us, gbs, gbs / 8000);
        std::fflush(stdout);
    };
    report("read 12 streams", time_us([&] { hipLaunchKernelGGL(probe_read, dim3(tiles), dim3(kThreads), 0, 0, a, sink); }), N);
    report("fill: every workgroup all 12 streams (12 stores per wavefront)",
           time_us([&] { hipLaunchKernelGGL(probe_fill_every_workgroup_all_streams, dim3(tiles), dim3(kThreads), 0, 0, a); }), N);
    report("fill: a wavefront per stream, 1 store per wavefront",
           time_us([&] { hipLaunchKernelGGL(probe_fill_wavefront_per_stream<1>, dim3(pieces), dim3(N * 64), 0, 0, a); }), N);
    report("fill: a wavefront per stream, 4 stores per wavefront",
           time_us([&] { hipLaunchKernelGGL(probe_fill_wavefront_per_stream<4>, dim3(pieces / 4), dim3(N * 64), 0, 0, a); }), N);
    report("fill: a wavefront per stream, 12 stores per wavefront",
           time_us([&] { hipLaunchKernelGGL(probe_fill_wavefront_per_stream<12>, dim3(pieces / 12), dim3(N * 64), 0, 0, a); }), N);

#define FOLD_REGISTERS(U, RUN, XCD, BY_DEST, NAME)                                                                   \
    report(NAME, time_us([&] {                                                                                       \
               hipLaunchKernelGGL((probe_fold_registers<U, RUN, XCD, BY_DEST>), dim3((tiles / U + RUN - 1) / RUN),   \
                                  dim3(kThreads), 0, 0, b, tiles / U);                                               \
           }), 2 * N)
    FOLD_REGISTERS(1, 1, false, false, "fold in registers: one vector per thread, tiles in launch order");
    FOLD_REGISTERS(1, 1, true, false, "fold in registers: XCD-contiguous tile order");
    FOLD_REGISTERS(1, 4, false, false, "fold in registers: 4 consecutive tiles per workgroup");
    FOLD_REGISTERS(1, 4, true, false, "fold in registers: 4 consecutive tiles, XCD-contiguous");
    FOLD_REGISTERS(2, 1, false, false, "fold in registers: two vectors per thread");
    FOLD_REGISTERS(2, 1, false, true, "fold in registers: two vectors, both to a destination before the next");
    FOLD_REGISTERS(1, 1, false, false, "fold in registers: one vector per thread, again");
    report("fold by wavefronts through LDS: 1 piece per workgroup",
           time_us([&] { hipLaunchKernelGGL(probe_fold_wavefronts<1>, dim3(pieces), dim3(N * 64), 0, 0, a, pieces); }), 2 * N);
    report("fold by wavefronts through LDS: 4 pieces per workgroup",
           time_us([&] { hipLaunchKernelGGL(probe_fold_wavefronts<4>, dim3(pieces / 4), dim3(N * 64), 0, 0, a, pieces); }), 2 * N);

    for (int k = 0; k < N; ++k) {
        hipLaunchKernelGGL(probe_count_differences, dim3(4096), dim3(256), 0, 0, reinterpret_cast<const uint32_t *>(a.dst[k]),
                           reinterpret_cast<const uint32_t *>(b.dst[k]), bytes / 4, bad);
    }
    unsigned long long differ = 0;
    CHECK(hipMemcpy(&differ, bad, 8, hipMemcpyDeviceToHost));
    std::printf("32-bit words in which the two folds differ: %llu\n", differ);
    return differ == 0 ? 0 : 1;
}
