// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>
#include <vector>
#include "hccl_types.h"
#include "kernels/launch.h"

namespace hcclx {

// Thread-local text of the last failure; returned by hcclx_last_error().
void set_error(const std::string &msg);
int fail(int code, const std::string &msg);  // records msg, returns code
int fail_hip(hipError_t e, const char *what);

#define HCCLX_HIP(expr)                                          \
    do {                                                         \
        hipError_t e_ = (expr);                                  \
        if (e_ != hipSuccess) return ::hcclx::fail_hip(e_, #expr); \
    } while (0)

// Per-device launch resources.
struct DeviceCtx {
    int device = -1;
    int num_cus = 0;
    // Fold launches use one workgroup per tile (measured faster than a persistent grid on MI355X: the
    // hardware staggers workgroups, a grid-stride loop runs them in lock step).  A non-zero value caps
    // the grid at blocks_per_cu x CUs instead.
    uint32_t blocks_per_cu = 0;
    // Chain folds whose largest fan-in reaches this go to the wide chain kernel (HCCLX_WIDE_CHAIN_FROM); with 9 to
    // 16 sources it measured 2 to 8 % faster than the kernel that holds all sources in registers, with 8 the same.
    uint32_t wide_chain_from = 9;
    // The same for chains with a single destination (HCCLX_WIDE_CHAIN_FROM_ONE_DST): there the wide kernel moves
    // four vectors per thread, and an 8-source ReduceScatter measured 5 % faster on it.
    uint32_t wide_chain_from_one_dst = 5;
    // Wide launches whose segments have this many destinations give each XCD a contiguous eighth of the tiles
    // (HCCLX_WIDE_XCD_REMAP_FROM).
    uint32_t wide_xcd_remap_from = 16;
    // A single-destination chain launch that would have fewer four-vector tiles than this takes two vectors per
    // thread instead, to spread a small job over more CUs (HCCLX_WIDE_MIN_TILES; set from the CU count).
    uint32_t wide_min_tiles = 0;
    uint32_t a2av_direct_unroll = 2;   // HCCLX_A2AV_DIRECT: 0 = off, 1 / 2 / 4 = vectors per thread and tile
    // V kernels whose tables live on the device cannot know their tile count on the host and run as a
    // persistent grid of this many workgroups per CU.
    uint32_t v_blocks_per_cu = 2;
    // With host tables the V kernels launch one workgroup per run of this many consecutive tiles.
    uint32_t v_tiles_per_block = 1;
    // Writing n outputs at once runs HBM a third slower than writing them one after the other (the banks see n
    // streams of row misses).  A fold whose result goes to several places therefore stores it once and a second
    // launch copies it to the other places, one place at a time in runs of fanout_run bytes (HCCLX_FANOUT_RUN)
    // whose re-reads the L2 serves: 8 x 64 MiB fp32 AllReduce 204 -> 175 us.  It pays from about 560 MiB read
    // and written by such folds in one launch (HCCLX_FANOUT_FROM, 0 = never): below that the Infinity Cache
    // (256 MiB) absorbs enough of the writes for the single pass to win (8 x 32 MiB: 84 against 90 us).
    uint64_t fanout_from = 560ull << 20;
    uint64_t fanout_run = 8ull << 20;
    // AllGather(V) with host tables: from this many bytes of payload on (HCCLX_AGV_PHASED_FROM, 0 = never) the outputs
    // of a run of a source are written one after the other, each workgroup writing one output.
    uint64_t agv_phased_from = 4ull << 20;
    // The n orders of a self-first fold among up to waves_max_fan ranks (HCCLX_WAVES_MAX_FAN) take the kernel with one
    // store per wavefront when the launch writes waves_from bytes or more (HCCLX_WAVES_FROM, 0 = never); waves_chains
    // (HCCLX_WAVES_CHAINS): also chains whose value goes to several places; waves_pieces (HCCLX_WAVES_PIECES): 1 KiB
    // pieces per source and workgroup, 0 = chosen per launch (2, 4 or 8).
    uint64_t waves_from = 1;
    uint32_t waves_max_fan = 16;
    bool waves_chains = false;
    uint32_t waves_pieces = 0;
    uint32_t moe_scatter_rows = 2;          // MoE dispatch of long rows: entries per workgroup, 1 or 2 (HCCLX_MOE_SCATTER_ROWS)
    uint64_t store_through_upto = 320ull << 20;   // fold launches with several destinations that write no more than this store through the L2 (HCCLX_STORE_THROUGH_UPTO)
    // Descriptor ring: tables of one-shot launches are written to pinned host memory and copied to the
    // device ring on the launch stream just before the kernel.
    char *h_ring = nullptr;
    char *d_ring = nullptr;
    size_t ring_bytes = 0;
    // Device address, on this GPU, of the library's fixed launch-table array (hcclx_fold_static): looked up once
    // when the context is made.
    char *static_table = nullptr;
};

// Returns the context of the current device, creating it on first use (nullptr + error set on failure).
DeviceCtx *device_ctx();

// Reserves `bytes` (multiple of 256) in the descriptor ring.  Blocks the host only when the ring wraps
// onto a slice whose earlier launches have not finished.
int ring_reserve(DeviceCtx *ctx, size_t bytes, hipStream_t stream, char **h, char **d);

uint32_t grid_for(const DeviceCtx *ctx, uint64_t total_tiles);

struct CopyBlock;
struct PhasedJob;

// One launch of the copy kernel that writes one output at a time.
struct PhasedLaunch {
    std::vector<PhasedJob> jobs;
    std::vector<char *> dsts;   // jobs.size() * nd pointers, job j's at [j * nd, j * nd + ndst)
    uint32_t slots = 0;         // tiles of the longest job
    uint32_t nd = 0;            // destinations of the widest job
    size_t jobs_bytes() const;  // size of the job array, rounded up to 256
    size_t bytes() const;       // job array + pointer array as they lie in the launch table
    void fill(char *h) const;
};
// A contiguous source that goes to several places whole.
struct PhasedStream {
    const char *src;
    uint64_t bytes;
    std::vector<char *> dst;
};
// Turns streams into launches: streams that continue each other (source and every destination) are joined, each
// is cut into runs of at most run_bytes of equal length, and runs of similar length share a launch (a launch's
// grid is sized for its longest run; shorter ones leave workgroups that exit at once).
void build_phased(std::vector<PhasedStream> &streams, uint64_t run_bytes, std::vector<PhasedLaunch> *out);
// The non-empty blocks of an AlltoAllV with host tables (row-major n x n, elements of esz bytes), with the
// inclusive prefix of their tiles of `unroll` vectors per thread; returns the number of tiles.
uint64_t list_alltoallv_blocks(const void *const *send, void *const *recv, const uint64_t *send_counts,
                               const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, uint32_t esz, int unroll,
                               std::vector<CopyBlock> *blocks);

}  // namespace hcclx
