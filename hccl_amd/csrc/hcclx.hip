// C-ABI launcher of the fold kernels (see include/hcclx.h): table building, descriptor ring, plans.
#include "hcclx.h"
#include "hcclx_internal.h"
#include "kernels/fold.h"
#include "kernels/vops.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

// The launch table of hcclx_fold_static: a fixed array in every GPU's memory that the library runs on, so that the
// entry point has nothing to allocate.  In host code this name is only a handle for hipGetSymbolAddress (done once
// per device in init_slot below); everything else uses the device address kept in DeviceCtx::static_table.
static __device__ __align__(256) unsigned char scratch[HCCLX_STATIC_TABLE_BYTES];

namespace hcclx {

// One piece of a launch table, carried in the kernel arguments and stored to `dst`: how hcclx_fold_static gets its
// table into device memory without a staging buffer or a copy engine.
constexpr uint32_t kPutBytes = 3584;   // kernel arguments hold up to 4 KiB
struct TablePiece {
    u32x4 v[kPutBytes / 16];
};
__global__ void __launch_bounds__(256) k_put_table(TablePiece piece, char *dst, uint32_t bytes)
{
    const uint32_t i = threadIdx.x;
    if (i * 16 < bytes) *reinterpret_cast<u32x4 *>(dst + i * 16) = piece.v[i];
}

static thread_local std::string g_err;

void set_error(const std::string &msg) { g_err = msg; }
int fail(int code, const std::string &msg)
{
    g_err = msg;
    return code;
}
int fail_hip(hipError_t e, const char *what)
{
    g_err = std::string(what) + ": " + hipGetErrorString(e);
    return (e == hipErrorOutOfMemory) ? HCCL_E_MEMORY : HCCL_E_RUNTIME;
}

// ---------------------------------------------------------------------------------------------------
// device context + descriptor ring
// ---------------------------------------------------------------------------------------------------
namespace {

constexpr int kMaxDevices = 32;
constexpr size_t kSliceBytes = 1u << 20;
constexpr int kSlices = 8;

struct Ring {
    std::mutex mu;
    int cur = 0;
    size_t off = 0;
    struct Pending {
        hipStream_t stream;
        hipEvent_t event;
    };
    std::vector<hipStream_t> used[kSlices];   // streams that launched from the slice since it was opened
    std::vector<Pending> pending[kSlices];    // events recorded when the slice was closed
    std::vector<hipEvent_t> pool;
};

// Pinned host memory that a plan's table is assembled in before it is copied to the device on a stream of its own
// and waited for.
constexpr size_t kPlanStageBytes = 4u << 20;   // to begin with; a larger table makes it grow
struct PlanStage {
    std::mutex mu;
    char *host = nullptr;
    size_t bytes = 0;
    hipStream_t stream = nullptr;   // the copies run on a stream of their own: they order with nothing else
};

// Who used the fixed launch table of hcclx_fold_static last.  Calls on one stream follow each other by stream order;
// a call on another stream first waits for the event recorded behind the previous call's fold kernel, so that the
// table is never rewritten under a kernel that still reads it.  The event is made once per device: nothing is
// allocated per call.
struct StaticTableUse {
    std::mutex mu;                  // one host thread at a time issues "upload the table, launch the fold"
    hipEvent_t done = nullptr;      // recorded behind the last fold that read the table
    hipStream_t last = nullptr;
    bool recorded = false;
};

struct DeviceSlot {
    std::once_flag once;
    bool ok = false;
    std::string err;
    DeviceCtx ctx;
    Ring ring;
    PlanStage stage;
    StaticTableUse static_use;
};

DeviceSlot g_slots[kMaxDevices];

void init_slot(DeviceSlot *s, int dev)
{
    DeviceCtx &c = s->ctx;
    c.device = dev;
    hipError_t e = hipDeviceGetAttribute(&c.num_cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || c.num_cus <= 0) {
        s->err = std::string("hipDeviceGetAttribute(MultiprocessorCount): ") + hipGetErrorString(e);
        return;
    }
    if (const char *v = std::getenv("HCCLX_BLOCKS_PER_CU")) {
        c.blocks_per_cu = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    }
    if (const char *v = std::getenv("HCCLX_A2AV_DIRECT")) c.a2av_direct_unroll = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    if (const char *v = std::getenv("HCCLX_WIDE_CHAIN_FROM")) c.wide_chain_from = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    if (const char *v = std::getenv("HCCLX_WIDE_XCD_REMAP_FROM")) c.wide_xcd_remap_from = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    c.wide_min_tiles = 2u * static_cast<uint32_t>(c.num_cus);
    if (const char *v = std::getenv("HCCLX_WIDE_MIN_TILES")) c.wide_min_tiles = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    if (const char *v = std::getenv("HCCLX_WIDE_CHAIN_FROM_ONE_DST")) {
        c.wide_chain_from_one_dst = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    }
    if (const char *v = std::getenv("HCCLX_V_BLOCKS_PER_CU")) {
        const uint32_t b = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
        if (b != 0) c.v_blocks_per_cu = b;
    }
    if (const char *v = std::getenv("HCCLX_V_TILES_PER_BLOCK")) {
        const uint32_t b = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
        if (b != 0) c.v_tiles_per_block = b;
    }
    if (const char *v = std::getenv("HCCLX_FANOUT_FROM")) c.fanout_from = std::strtoull(v, nullptr, 10);
    if (const char *v = std::getenv("HCCLX_FANOUT_RUN")) {
        // between 64 KiB and 1 GiB: a run is one job of a launch, and its tile count has to stay within the length
        // classes the launches are grouped by
        const uint64_t b = std::min<uint64_t>(std::strtoull(v, nullptr, 10), 1ull << 30);
        if (b >= 65536) c.fanout_run = b & ~static_cast<uint64_t>(4095);
    }
    if (const char *v = std::getenv("HCCLX_WAVES_FROM")) c.waves_from = std::strtoull(v, nullptr, 10);
    if (const char *v = std::getenv("HCCLX_WAVES_MAX_FAN")) {
        const unsigned long b = std::strtoul(v, nullptr, 10);
        c.waves_max_fan = b > HCCLX_MAX_FAN ? static_cast<uint32_t>(HCCLX_MAX_FAN) : static_cast<uint32_t>(b);
    }
    if (const char *v = std::getenv("HCCLX_WAVES_CHAINS")) c.waves_chains = std::strtoul(v, nullptr, 10) != 0;
    if (const char *v = std::getenv("HCCLX_WAVES_PIECES")) {
        const unsigned long b = std::strtoul(v, nullptr, 10);
        c.waves_pieces = b > kWavePieces ? static_cast<uint32_t>(kWavePieces) : static_cast<uint32_t>(b);
    }
    if (const char *v = std::getenv("HCCLX_AGV_PHASED_FROM")) c.agv_phased_from = std::strtoull(v, nullptr, 10);
    if (const char *v = std::getenv("HCCLX_MOE_SCATTER_ROWS")) c.moe_scatter_rows = static_cast<uint32_t>(std::strtoul(v, nullptr, 10));
    if (const char *v = std::getenv("HCCLX_STORE_THROUGH_UPTO")) c.store_through_upto = std::strtoull(v, nullptr, 10);
    c.ring_bytes = kSliceBytes * kSlices;
    e = hipHostMalloc(reinterpret_cast<void **>(&c.h_ring), c.ring_bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        s->err = std::string("hipHostMalloc(descriptor ring): ") + hipGetErrorString(e);
        return;
    }
    e = hipMalloc(reinterpret_cast<void **>(&c.d_ring), c.ring_bytes);
    if (e != hipSuccess) {
        s->err = std::string("hipMalloc(descriptor ring): ") + hipGetErrorString(e);
        return;
    }
    // The runtime sets up its path for host-to-device copies above 16 KiB when the first one is made (6-10 ms):
    // make it here, so that it does not land in the first collective whose table is that large.
    e = hipStreamCreateWithFlags(&s->stage.stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void **>(&s->stage.host), kPlanStageBytes, hipHostMallocDefault);
    if (e == hipSuccess) s->stage.bytes = kPlanStageBytes;
    if (e == hipSuccess) e = hipMemcpyAsync(c.d_ring, c.h_ring, 64 * 1024, hipMemcpyHostToDevice, s->stage.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(s->stage.stream);
    if (e != hipSuccess) {
        s->err = std::string("first table upload: ") + hipGetErrorString(e);
        return;
    }
    // init_slot runs with `dev` current (device_ctx() asks for the current device): this is that device's copy
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&c.static_table), HIP_SYMBOL(scratch));
    if (e != hipSuccess || c.static_table == nullptr) {
        s->err = std::string("hipGetSymbolAddress(launch table): ") + hipGetErrorString(e);
        return;
    }
    e = hipEventCreateWithFlags(&s->static_use.done, hipEventDisableTiming);
    if (e != hipSuccess) {
        s->err = std::string("hipEventCreate(launch table): ") + hipGetErrorString(e);
        return;
    }
    s->ok = true;
}

}  // namespace

DeviceCtx *device_ctx()
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        fail_hip(e, "hipGetDevice");
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        fail(HCCL_E_PARA, "device index out of range");
        return nullptr;
    }
    DeviceSlot *s = &g_slots[dev];
    std::call_once(s->once, init_slot, s, dev);
    if (!s->ok) {
        set_error(s->err);
        return nullptr;
    }
    return &s->ctx;
}

int ring_reserve(DeviceCtx *ctx, size_t bytes, hipStream_t stream, char **h, char **d)
{
    bytes = (bytes + 255) & ~static_cast<size_t>(255);
    if (bytes > kSliceBytes) {
        return fail(HCCL_E_PARA, "descriptor table larger than one ring slice");
    }
    // A captured copy would read its ring slot again at every replay, long after the slot has been reused.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
        (void)hipGetLastError();
    } else if (capturing != hipStreamCaptureStatusNone) {
        return fail(HCCL_E_NOT_SUPPORT,
                    "this launch uploads its tables at call time and cannot be captured into a HIP graph: create a plan "
                    "outside the capture and capture hcclx_plan_launch");
    }
    Ring &r = g_slots[ctx->device].ring;
    std::lock_guard<std::mutex> lock(r.mu);
    if (r.off + bytes > kSliceBytes) {
        // close the current slice: one event per stream that read from it
        for (hipStream_t s : r.used[r.cur]) {
            hipEvent_t ev;
            if (!r.pool.empty()) {
                ev = r.pool.back();
                r.pool.pop_back();
            } else {
                HCCLX_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
            }
            HCCLX_HIP(hipEventRecord(ev, s));
            r.pending[r.cur].push_back({s, ev});
        }
        r.used[r.cur].clear();
        r.cur = (r.cur + 1) % kSlices;
        r.off = 0;
        // open the next one: everything that still reads it must have finished
        for (auto &p : r.pending[r.cur]) {
            HCCLX_HIP(hipEventSynchronize(p.event));
            r.pool.push_back(p.event);
        }
        r.pending[r.cur].clear();
    }
    bool seen = false;
    for (hipStream_t s : r.used[r.cur]) seen = seen || (s == stream);
    if (!seen) r.used[r.cur].push_back(stream);
    const size_t at = static_cast<size_t>(r.cur) * kSliceBytes + r.off;
    r.off += bytes;
    *h = ctx->h_ring + at;
    *d = ctx->d_ring + at;
    return HCCL_SUCCESS;
}

uint32_t grid_for(const DeviceCtx *ctx, uint64_t total_tiles)
{
    uint64_t cap = static_cast<uint64_t>(ctx->num_cus) * ctx->blocks_per_cu;
    if (ctx->blocks_per_cu == 0 || total_tiles < cap) cap = total_tiles;
    if (cap > 0x7fffffffu) cap = 0x7fffffffu;
    return static_cast<uint32_t>(cap);
}

// ---------------------------------------------------------------------------------------------------
// copies that write one output at a time
// ---------------------------------------------------------------------------------------------------
size_t PhasedLaunch::jobs_bytes() const { return (jobs.size() * sizeof(PhasedJob) + 255) & ~static_cast<size_t>(255); }
size_t PhasedLaunch::bytes() const { return jobs_bytes() + dsts.size() * sizeof(char *); }
void PhasedLaunch::fill(char *h) const
{
    std::memcpy(h, jobs.data(), jobs.size() * sizeof(PhasedJob));
    std::memcpy(h + jobs_bytes(), dsts.data(), dsts.size() * sizeof(char *));
}

void build_phased(std::vector<PhasedStream> &streams, uint64_t run_bytes, std::vector<PhasedLaunch> *out)
{
    // join streams that continue each other: the slices of a two-shot AllReduce lie back to back in every buffer
    std::vector<PhasedStream> joined;
    for (PhasedStream &st : streams) {
        if (st.bytes == 0 || st.dst.empty()) continue;
        bool cont = !joined.empty() && joined.back().dst.size() == st.dst.size() &&
                    joined.back().src + joined.back().bytes == st.src;
        for (size_t d = 0; cont && d < st.dst.size(); ++d) cont = joined.back().dst[d] + joined.back().bytes == st.dst[d];
        if (cont) {
            joined.back().bytes += st.bytes;
        } else {
            joined.push_back(std::move(st));
        }
    }
    struct Run {
        const PhasedStream *st;
        uint64_t at, len;
        uint32_t tiles;
    };
    // runs of equal length per stream, a multiple of the tile size; then launches by length class (powers of four)
    constexpr uint64_t kTile = 256ull * 16 * kPhasedUnroll;
    run_bytes = std::min<uint64_t>(std::max<uint64_t>(run_bytes, kTile), 1ull << 30);   // every run falls into a class below
    std::vector<Run> runs;
    for (const PhasedStream &st : joined) {
        const uint64_t n = (st.bytes + run_bytes - 1) / run_bytes;
        const uint64_t len = ((st.bytes + n - 1) / n + kTile - 1) / kTile * kTile;
        for (uint64_t at = 0; at < st.bytes; at += len) {
            Run r{&st, at, st.bytes - at < len ? st.bytes - at : len, 0};
            r.tiles = static_cast<uint32_t>(v_tiles_of(r.len, reinterpret_cast<uint64_t>(st.dst[0]) + at, kPhasedUnroll));
            runs.push_back(r);
        }
    }
    constexpr size_t kMaxJobs = 4096;   // per launch: the table stays well inside one slice of the descriptor ring
    for (int cls = 15; cls >= 0; --cls) {
        PhasedLaunch cur;
        auto flush = [&]() {
            if (cur.jobs.empty()) return;
            // Workgroups go to the eight XCDs in turn, each with an L2 of its own: with a multiple of eight slots per
            // destination a tile is copied to all its destinations by the same XCD, whose L2 then serves the re-reads.
            cur.slots = (cur.slots + 7) & ~7u;
            // the pointer array is laid out once the widest job is known
            std::vector<char *> flat(cur.jobs.size() * cur.nd, nullptr);
            size_t at = 0;
            for (size_t j = 0; j < cur.jobs.size(); ++j) {
                for (uint32_t d = 0; d < cur.jobs[j].ndst; ++d) flat[j * cur.nd + d] = cur.dsts[at++];
            }
            cur.dsts = std::move(flat);
            out->push_back(std::move(cur));
            cur = PhasedLaunch();
        };
        for (const Run &r : runs) {
            int c = 0;
            for (uint32_t t = r.tiles; t > 1; t = (t + 3) / 4) ++c;
            if (std::min(c, 15) != cls) continue;
            const uint32_t nd = static_cast<uint32_t>(r.st->dst.size());
            const uint64_t grid_x = (static_cast<uint64_t>(std::max(cur.slots, r.tiles)) + 7) * std::max(cur.nd, nd);
            if (cur.jobs.size() == kMaxJobs || grid_x > 0x7fffffffull ||
                (cur.jobs.size() + 1) * (sizeof(PhasedJob) + 8ull * std::max(cur.nd, nd)) > (1u << 19)) {
                flush();
            }
            PhasedJob j;
            j.src = r.st->src + r.at;
            j.bytes = r.len;
            j.dst0 = reinterpret_cast<uint64_t>(r.st->dst[0]) + r.at;
            j.ndst = nd;
            j.tiles = r.tiles;
            cur.jobs.push_back(j);
            for (char *p : r.st->dst) cur.dsts.push_back(p + r.at);   // packed for now, see flush()
            cur.slots = std::max(cur.slots, r.tiles);
            cur.nd = std::max(cur.nd, nd);
        }
        flush();
    }
}

// ---------------------------------------------------------------------------------------------------
// fold tables
// ---------------------------------------------------------------------------------------------------
namespace {

bool is_reduce_dtype(int dt)
{
    switch (dt) {
        case HCCL_DATA_TYPE_INT8:
        case HCCL_DATA_TYPE_INT16:
        case HCCL_DATA_TYPE_INT32:
        case HCCL_DATA_TYPE_INT64:
        case HCCL_DATA_TYPE_UINT64:
        case HCCL_DATA_TYPE_FP16:
        case HCCL_DATA_TYPE_FP32:
        case HCCL_DATA_TYPE_FP64:
        case HCCL_DATA_TYPE_BFP16:
            return true;
        default:
            return false;
    }
}

bool is_float_dtype(int dt)
{
    return dt == HCCL_DATA_TYPE_FP16 || dt == HCCL_DATA_TYPE_FP32 || dt == HCCL_DATA_TYPE_FP64 ||
           dt == HCCL_DATA_TYPE_BFP16;
}

// What one kernel launch needs, before it is placed in device memory.
struct Batch {
    bool copy = false;
    int dtype = 0;
    int op = 0;
    int mode = 0;
    int maxn = 1;
    uint64_t total_tiles = 0;
    std::vector<uint64_t> tile_end;
    std::vector<SegDev> segs;
    std::vector<SegWide> wide;   // instead of segs when maxn == kMaxWideFan
    int wide_unroll = 1;         // vectors per thread of the wide kernel
    uint32_t xcd_remap = 0;      // wide kernels: contiguous tile ranges per XCD (pays with 16 or more destinations)
    std::vector<CopyBlock> blocks;   // instead of everything above: a list of blocks for the block copy kernel
    int block_unroll = 2;
    PhasedLaunch phased;         // instead of everything above: jobs of the copy kernel that writes one output at a time
    uint32_t store_policy = kStoreStream;   // how the fold kernels store (fold.h)
    uint32_t waves = 0;          // non-zero: the one-store-per-wavefront kernel, this many wavefronts per workgroup
    uint32_t pieces = 1;         // and this many 1 KiB pieces per source and workgroup
    uint32_t waves_fixed = 0;    // and, when every segment has the same number of sources, that number
    size_t nseg() const { return segs.size() + wide.size(); }
    size_t bytes() const
    {
        if (!phased.jobs.empty()) return phased.bytes();
        if (!blocks.empty()) return blocks.size() * sizeof(CopyBlock);
        return align256(tile_end.size() * 8) + segs.size() * sizeof(SegDev) + wide.size() * sizeof(SegWide);
    }
    static size_t align256(size_t x) { return (x + 255) & ~static_cast<size_t>(255); }
};

struct Built {
    std::vector<Batch> batches;
    uint64_t algo_bytes = 0;
};

// Embeds the (dst, src) step program of a tree over nsrc registers into a complete binary tree with `slots`
// leaf slots: code[i] of inner heap node i (0 = nothing below, 1 = take the dst child, 2 = combine) and, per
// leaf slot, the register whose source sits there (-1 = empty).  Returns false when the tree is deeper than
// log2(slots).
// code and slot_reg hold `slots` <= kMaxWideFan entries; nothing is allocated.
bool embed_tree(uint32_t nsrc, const uint8_t *prog, uint32_t slots, uint8_t *code, int *slot_reg)
{
    struct N {
        int dst = -1, src = -1, leaf = -1;
    };
    N nodes[2 * kMaxWideFan];
    int holder[kMaxWideFan];  // node currently held by each register
    uint32_t nnodes = nsrc;
    for (uint32_t k = 0; k < nsrc; ++k) {
        nodes[k].leaf = static_cast<int>(k);
        holder[k] = static_cast<int>(k);
    }
    for (uint32_t t = 0; t + 1 < nsrc; ++t) {
        N n;
        n.dst = holder[prog[2 * t]];
        n.src = holder[prog[2 * t + 1]];
        nodes[nnodes] = n;
        holder[prog[2 * t]] = static_cast<int>(nnodes++);
    }
    for (uint32_t k = 0; k < slots; ++k) {
        code[k] = 0;
        slot_reg[k] = -1;
    }
    // place(node, heap index): inner nodes combine their two children; a leaf above the bottom level is
    // passed up from the left-most slot below it
    struct Todo {
        int id;
        uint32_t at;
    };
    Todo stack[2 * kMaxWideFan];
    uint32_t top = 0;
    stack[top++] = {holder[0], 1u};
    while (top != 0) {
        const int id = stack[top - 1].id;
        uint32_t at = stack[top - 1].at;
        --top;
        const N &n = nodes[id];
        if (n.leaf >= 0) {
            while (at < slots) {
                code[at] = 1;
                at *= 2;
            }
            slot_reg[at - slots] = n.leaf;
        } else {
            if (at >= slots) return false;
            code[at] = 2;
            stack[top++] = {n.dst, 2 * at};
            stack[top++] = {n.src, 2 * at + 1};
        }
    }
    return true;
}

bool embed_tree(const hcclx_seg_t &s, uint32_t slots, SegDev *sd)
{
    uint8_t code[kMaxWideFan];
    int slot_reg[kMaxWideFan];
    if (!embed_tree(s.nsrc, s.prog, slots, code, slot_reg)) return false;
    sd->tree_codes = 0;
    sd->leaf_mask = 0;
    for (uint32_t k = 0; k < kMaxFan; ++k) sd->src[k] = nullptr;
    for (uint32_t i = 1; i < slots; ++i) sd->tree_codes |= static_cast<uint32_t>(code[i]) << (2 * i);
    for (uint32_t k = 0; k < slots; ++k) {
        if (slot_reg[k] < 0) continue;
        sd->src[k] = static_cast<const char *>(s.src[slot_reg[k]]);
        sd->leaf_mask |= 1u << k;
    }
    return true;
}

// Checks a tree program: nsrc - 1 steps, every register but 0 consumed exactly once, register 0 never, no
// step on a consumed register.  Returns the number of levels of the tree, or -1 when it is malformed.
int tree_levels(uint32_t nsrc, const uint8_t *prog)
{
    bool dead[kMaxWideFan] = {};
    uint32_t depth[kMaxWideFan] = {};
    for (uint32_t t = 0; t + 1 < nsrc; ++t) {
        const uint32_t rd = prog[2 * t];
        const uint32_t rs = prog[2 * t + 1];
        if (rd >= nsrc || rs >= nsrc || rd == rs || rs == 0 || dead[rd] || dead[rs]) return -1;
        dead[rs] = true;
        depth[rd] = (depth[rd] > depth[rs] ? depth[rd] : depth[rs]) + 1;
    }
    return static_cast<int>(depth[0]);
}

int build_wide_batches_impl(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode,
                            Built *out);

// What the segments of one launch of the register-resident kernels have in common.
struct SegProto {
    bool copy = false;   // no segment combines anything: the byte copy kernel
    int mode = 0;        // the kernel's mode (integers take the chain kernel whatever order is asked for)
    int maxn = 1;        // source slots of the kernel instance
    int esz = 1;
    uint32_t waves = 0;  // non-zero: tiles are those of the one-store-per-wavefront kernel (pieces x 64 vectors)
    uint32_t pieces = 1;
};

// Checks the segments of a call and works out the kernel instance they need.  Allocates nothing unless it fails.
int check_segs(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, SegProto *sp)
{
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (mode != HCCLX_FOLD_CHAIN && mode != HCCLX_FOLD_SELF_FIRST && mode != HCCLX_FOLD_TREE) {
        return fail(HCCL_E_PARA, "unknown fold mode");
    }
    uint32_t max_src = 0;
    uint32_t max_depth = 0;  // tree mode: levels of the deepest tree
    for (uint32_t i = 0; i < nseg; ++i) {
        const hcclx_seg_t &s = segs[i];
        if (s.nsrc == 0 || s.nsrc > HCCLX_MAX_FAN || s.ndst == 0 || s.ndst > HCCLX_MAX_FAN) {
            return fail(HCCL_E_PARA, "segment " + std::to_string(i) + ": nsrc/ndst outside 1.." +
                                         std::to_string(HCCLX_MAX_FAN));
        }
        if (mode == HCCLX_FOLD_SELF_FIRST && s.nsrc != s.ndst) {
            return fail(HCCL_E_PARA, "self-first fold needs nsrc == ndst");
        }
        if (s.count != 0) {
            for (uint32_t k = 0; k < s.nsrc; ++k) {
                if (s.src[k] == nullptr) return fail(HCCL_E_PTR, "segment " + std::to_string(i) + ": null source");
            }
            for (uint32_t k = 0; k < s.ndst; ++k) {
                if (s.dst[k] == nullptr) return fail(HCCL_E_PTR, "segment " + std::to_string(i) + ": null destination");
            }
        }
        if (mode == HCCLX_FOLD_TREE) {
            const int levels = tree_levels(s.nsrc, s.prog);
            if (levels < 0) return fail(HCCL_E_PARA, "segment " + std::to_string(i) + ": malformed tree program");
            if (is_float_dtype(dtype) && (1u << levels) > HCCLX_MAX_FAN) {
                return fail(HCCL_E_NOT_SUPPORT, "segment " + std::to_string(i) + ": tree has " + std::to_string(levels) +
                                                    " levels, the kernel holds 4");
            }
            if (static_cast<uint32_t>(levels) > max_depth) max_depth = static_cast<uint32_t>(levels);
        }
        if (s.nsrc > max_src) max_src = s.nsrc;
    }
    sp->copy = (max_src <= 1);
    sp->mode = mode;
    sp->esz = esz;
    if (!sp->copy) {
        if (!is_reduce_dtype(dtype)) return fail(HCCL_E_NOT_SUPPORT, "data type cannot be reduced");
        if (op < HCCL_REDUCE_SUM || op > HCCL_REDUCE_MIN) return fail(HCCL_E_NOT_SUPPORT, "unknown reduce op");
        sp->maxn = max_src <= 2 ? 2 : max_src <= 4 ? 4 : max_src <= 8 ? 8 : 16;
        // a tree needs one leaf slot per position of the complete tree of its depth
        if (mode == HCCLX_FOLD_TREE && is_float_dtype(dtype) && (1 << max_depth) > sp->maxn) sp->maxn = 1 << max_depth;
        // Integer folds are association-free: the self-first order and every tree give the bits of the plain
        // chain.  The kernels for those orders exist only for floating types, so integers take the chain kernel.
        if (mode != HCCLX_FOLD_CHAIN && !is_float_dtype(dtype)) sp->mode = HCCLX_FOLD_CHAIN;
    } else {
        sp->maxn = 1;
        sp->mode = HCCLX_FOLD_CHAIN;
    }
    return HCCL_SUCCESS;
}

// The device descriptor of one segment and its number of tiles; false when a tree does not fit the kernel instance.
bool make_segdev(const hcclx_seg_t &s, const SegProto &sp, int mode, SegDev *out, uint64_t *tiles)
{
    SegDev sd;
    std::memset(&sd, 0, sizeof(sd));
    sd.count = sp.copy ? s.count * sp.esz : s.count;  // the copy kernel counts bytes
    sd.nsrc = s.nsrc;
    sd.ndst = s.ndst;
    for (uint32_t k = 0; k < s.nsrc; ++k) sd.src[k] = static_cast<const char *>(s.src[k]);
    for (uint32_t k = 0; k < s.ndst; ++k) sd.dst[k] = static_cast<char *>(s.dst[k]);
    if (mode == HCCLX_FOLD_CHAIN) {
        for (uint32_t k = 1; k < s.nsrc; ++k) sd.tree_codes |= (s.prog[k] ? 1u : 0u) << k;   // acc (+) src[k] steps
    }
    if (sp.mode == HCCLX_FOLD_TREE && !embed_tree(s, static_cast<uint32_t>(sp.maxn), &sd)) return false;
    const int ne = sp.copy ? 16 : 16 / sp.esz;
    const uint64_t tile_vecs = sp.waves != 0 ? waves_tile_vecs(static_cast<int>(sp.pieces)) : fold_tile_vecs(sp.maxn, sp.mode);
    sd.head = fold_head_of(sd.count, sp.copy ? 1 : sp.esz, sd.dst[0]);
    sd.shift = fold_shift_of(sd.head, sp.copy ? 1 : sp.esz, tile_vecs, sd.dst[0]);
    *tiles = fold_tiles_of(sd.count, ne, tile_vecs, sd.head, sd.shift);
    *out = sd;
    return true;
}

// Results that go to several places, from fanout_from bytes of them on: the fold stores each result once (to
// dst[0]) and a second launch copies it to the other places, one place at a time in runs whose re-reads the L2
// serves; segments that only copy go to that second launch whole (their source is the run).
// Fills `one` (the segments of the first launch, one destination each) and `fan` (what the second launch copies)
// and returns true; returns false when the launch stays as it is.  max_fan: the segment type's array size.
template <typename SEG>
bool split_fanout(const DeviceCtx *ctx, const SEG *segs, uint32_t nseg, int esz, int mode, uint32_t max_fan,
                  std::vector<SEG> *one, std::vector<PhasedStream> *fan)
{
    if (ctx == nullptr || mode == HCCLX_FOLD_SELF_FIRST || esz == 0) return false;
    uint64_t fold_traffic = 0;   // bytes read and written by the folds whose result goes to several places
    uint64_t copy_payload = 0;   // bytes of the sources that are only copied to several places
    for (uint32_t i = 0; i < nseg; ++i) {
        const SEG &g = segs[i];
        if (g.nsrc == 0 || g.nsrc > max_fan || g.ndst == 0 || g.ndst > max_fan) return false;   // rejected later
        if (g.count == 0 || g.ndst < 2) continue;
        for (uint32_t d = 0; d < g.ndst; ++d) {
            if (g.dst[d] == nullptr) return false;
        }
        if (g.src[0] == nullptr) return false;
        const uint64_t bytes = g.count * static_cast<uint64_t>(esz);
        if (g.nsrc == 1) {
            copy_payload += bytes;
        } else {
            fold_traffic += bytes * (g.nsrc + g.ndst);
        }
    }
    const bool split_folds = ctx->fanout_from != 0 && fold_traffic >= ctx->fanout_from;
    const bool split_copies = ctx->agv_phased_from != 0 && copy_payload >= ctx->agv_phased_from;
    if (!split_folds && !split_copies) return false;
    one->clear();
    fan->clear();
    for (uint32_t i = 0; i < nseg; ++i) {
        const SEG &g = segs[i];
        if (g.count == 0 || g.ndst < 2 || !(g.nsrc == 1 ? split_copies : split_folds)) {
            one->push_back(g);
            continue;
        }
        const bool copy = g.nsrc == 1;
        PhasedStream st;
        st.src = copy ? static_cast<const char *>(g.src[0]) : static_cast<const char *>(g.dst[0]);
        st.bytes = g.count * static_cast<uint64_t>(esz);
        for (uint32_t d = copy ? 0 : 1; d < g.ndst; ++d) st.dst.push_back(static_cast<char *>(g.dst[d]));
        fan->push_back(std::move(st));
        if (!copy) {
            SEG f = g;
            f.ndst = 1;
            one->push_back(f);
        }
    }
    return true;
}

// Appends the second launch (or launches) of a split fold.
void append_fanout(const DeviceCtx *ctx, std::vector<PhasedStream> &fan, Built *out)
{
    std::vector<PhasedLaunch> launches;
    build_phased(fan, ctx->fanout_run, &launches);
    for (PhasedLaunch &l : launches) {
        Batch b;
        b.copy = true;
        b.phased = std::move(l);
        out->batches.push_back(std::move(b));
    }
}

// How a fold launch stores its results (fold.h): written through the L2 when every segment has one destination, and
// for launches with several destinations up to the size from which they are split into fold + fan-out anyway
// (8 ranks x 32 MiB AllReduce in one pass: 83.8 us against 96.3 streamed; no difference left at 8 x 39 MiB);
// larger ones, which only the orders that cannot be split reach, are streamed.
template <typename SEG>
uint32_t store_policy_for(const DeviceCtx *ctx, const SEG *segs, uint32_t nseg, int esz)
{
    const uint64_t upto = ctx ? ctx->store_through_upto : (320ull << 20);
    uint64_t written = 0;
    uint32_t most_dst = 0;
    for (uint32_t i = 0; i < nseg; ++i) {
        written += segs[i].count * static_cast<uint64_t>(esz) * segs[i].ndst;
        most_dst = segs[i].ndst > most_dst ? segs[i].ndst : most_dst;
    }
    return (most_dst <= 1 || written <= upto) ? kStoreThrough : kStoreStream;
}

int build_batches_impl(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, Built *out);

int build_batches(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, Built *out)
{
    if (nseg != 0 && segs == nullptr) return fail(HCCL_E_PTR, "segs is null");
    std::vector<hcclx_seg_t> one;
    std::vector<PhasedStream> fan;
    const DeviceCtx *fctx = device_ctx();
    if (!split_fanout(fctx, segs, nseg, dtype_size(dtype), mode, HCCLX_MAX_FAN, &one, &fan)) {
        return build_batches_impl(segs, nseg, dtype, op, mode, out);
    }
    const uint64_t algo_before = out->algo_bytes;
    const int rc = build_batches_impl(one.data(), static_cast<uint32_t>(one.size()), dtype, op, mode, out);
    if (rc != HCCL_SUCCESS) return rc;
    // the algorithmic bytes are those of the segments as the caller gave them, however the work is split
    out->algo_bytes = algo_before;
    for (uint32_t i = 0; i < nseg; ++i) {
        out->algo_bytes += static_cast<uint64_t>(segs[i].nsrc + segs[i].ndst) * segs[i].count * dtype_size(dtype);
    }
    append_fanout(fctx, fan, out);
    return HCCL_SUCCESS;
}

// The n orders of a self-first fold take the kernel in which every wavefront issues one store (fold.h) when all
// segments have the same number of ranks, at most waves_max_fan, and the launch writes waves_from bytes or more.
// Measured against the register kernel on fp32 PROD (us, register : wavefronts): 4 ranks x 64 MiB 97.7 : 77.4,
// 8 x 64 MiB 210 : 175, 12 x 64 MiB 281 : 270, 12 x 256 MiB 1183 : 1056, 16 x 256 MiB 1582 : 1445, and at
// 256 KiB per rank and below 4.6-5.6 : 3.2-3.5 among 8 to 12 ranks (at 4 KiB per rank: 4 ranks 3.9 : 3.1, 16 ranks
// 5.3 : 3.9; the register kernel's threads each walk all the sources, here the wavefronts share them).  Where the register kernel measured
// better it stays: two ranks below 32 MiB per rank (no difference), seven and eight ranks between 3 and 12 MiB per
// rank (8 x 4 MiB: 10.6 : 12.1).  Pieces per workgroup: two for small launches and up to four ranks; five to eight
// ranks four below 32 MiB per rank (8 x 16 MiB: 47.9 / 43.0 us with 2 / 4) and two from there on (8 x 64 MiB:
// 168.8 / 182.6); nine and more eight below 12 MiB per rank (12 x 8 MiB: 35.6 / 36.4 / 32.3 us with 2 / 4 / 8) and
// four from there on (12 x 64 MiB: 268.7 / 260.6 / 281.7).  Launches
// whose segments differ in their number of ranks run on the instance that reads the count per segment, which only
// wins up to eight ranks.  Chains whose value goes to several places (integer one-shot AllReduce, two-shot, NHR of
// integers) take this kernel up to 256 KiB per place, where its prologue is the shorter one (12 ranks: 3.4-3.6
// against 3.9-4.3 us for one segment, 5.0-6.2 against 5.9-6.8 for twelve slices; from 1 MiB per place on the register
// kernels win: 4.9 against 5.5), and beyond only when asked for (waves_chains; as one pass the 8 x 64 MiB AllReduce
// measured 189 to 245 us against 172 for fold + fan-out).
// Returns the number of wavefronts per workgroup (the widest segment's sources or destinations), 0 = the register
// kernels.
uint32_t waves_for(const DeviceCtx *ctx, const hcclx_seg_t *segs, uint32_t nseg, int dtype, int mode, uint32_t *pieces)
{
    if (ctx == nullptr || ctx->waves_from == 0 || nseg == 0) return 0;
    if (mode != HCCLX_FOLD_SELF_FIRST && mode != HCCLX_FOLD_CHAIN) return 0;
    const uint64_t esz = static_cast<uint64_t>(dtype_size(dtype));
    uint32_t most_src = 0;
    uint32_t most_dst = 0;
    uint32_t least_src = ~0u;
    uint64_t written = 0;
    uint64_t tiles = 0;
    for (uint32_t i = 0; i < nseg; ++i) {
        if (segs[i].nsrc == 0 || segs[i].nsrc > HCCLX_MAX_FAN || segs[i].ndst == 0 || segs[i].ndst > HCCLX_MAX_FAN) return 0;
        if (segs[i].count == 0) continue;
        most_src = segs[i].nsrc > most_src ? segs[i].nsrc : most_src;
        least_src = segs[i].nsrc < least_src ? segs[i].nsrc : least_src;
        most_dst = segs[i].ndst > most_dst ? segs[i].ndst : most_dst;
        written += segs[i].count * esz * segs[i].ndst;
        tiles += segs[i].count * esz / 1024 + 2;
    }
    const uint32_t widest = most_src > most_dst ? most_src : most_dst;
    if (most_src < 2 || most_dst < 2 || widest > ctx->waves_max_fan || written < ctx->waves_from || esz == 0) return 0;
    const bool same = least_src == most_src;
    const uint64_t per_place = written / most_dst;
    if (mode == HCCLX_FOLD_SELF_FIRST) {
        if (!same && widest > 8) return 0;
    } else if (!ctx->waves_chains && per_place > (256ull << 10)) {
        return 0;   // chains to several places: only the small ones by default (see above)
    }
    uint32_t p = ctx->waves_pieces;
    if (p == 0) {   // the shipped policy; a forced piece count takes every launch that passed the tests above
        if (mode == HCCLX_FOLD_SELF_FIRST) {
            if (widest == 2 && per_place < (32ull << 20)) return 0;
            if ((widest == 7 || widest == 8) && per_place >= (3ull << 20) && per_place < (12ull << 20)) return 0;
        }
        if (per_place < (2ull << 20) || widest <= 4) {
            p = 2;
        } else if (widest <= 8) {
            p = per_place < (32ull << 20) ? 4u : 2u;
        } else {
            p = per_place < (12ull << 20) ? 8u : 4u;
        }
    }
    if (tiles / p > 0x7fffffffull) return 0;   // one workgroup per tile: the grid has to hold them
    *pieces = p;
    return widest;
}

int build_batches_impl(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, Built *out)
{
    if (nseg != 0 && segs == nullptr) return fail(HCCL_E_PTR, "segs is null");
    // the order a launch is asked for, and the one its kernel runs: integer folds are association-free
    const int kernel_mode = (mode != HCCLX_FOLD_CHAIN && !is_float_dtype(dtype)) ? HCCLX_FOLD_CHAIN : mode;
    uint32_t wave_pieces = 1;
    const uint32_t waves = waves_for(device_ctx(), segs, nseg, dtype, kernel_mode, &wave_pieces);
    // Chains over many sources run faster on the wide chain kernel (sources in groups of eight, two vectors per
    // thread) than on the kernel that holds every source in registers.
    if (mode == HCCLX_FOLD_CHAIN && nseg != 0 && waves == 0) {
        const DeviceCtx *ctx = device_ctx();
        uint32_t most = 0;
        uint32_t most_dst = 0;
        bool plain = true;
        for (uint32_t i = 0; i < nseg; ++i) {
            plain = plain && segs[i].nsrc <= HCCLX_MAX_FAN && segs[i].ndst <= HCCLX_MAX_FAN;
            most = segs[i].nsrc > most ? segs[i].nsrc : most;
            most_dst = segs[i].ndst > most_dst ? segs[i].ndst : most_dst;
        }
        if (ctx && plain && most >= (most_dst <= 1 ? ctx->wide_chain_from_one_dst : ctx->wide_chain_from)) {
            std::vector<hcclx_wide_seg_t> wide(nseg);
            for (uint32_t i = 0; i < nseg; ++i) {
                std::memset(&wide[i], 0, sizeof(wide[i]));
                wide[i].count = segs[i].count;
                wide[i].nsrc = segs[i].nsrc;
                wide[i].ndst = segs[i].ndst;
                for (uint32_t k = 0; k < segs[i].nsrc; ++k) wide[i].src[k] = segs[i].src[k];
                for (uint32_t k = 0; k < segs[i].ndst; ++k) wide[i].dst[k] = segs[i].dst[k];
                for (uint32_t k = 1; k < segs[i].nsrc; ++k) wide[i].prog[k] = segs[i].prog[k];   // operand order per step
            }
            return build_wide_batches_impl(wide.data(), nseg, dtype, op, HCCLX_FOLD_CHAIN, out);
        }
    }
    SegProto sp;
    const int rc = check_segs(segs, nseg, dtype, op, mode, &sp);
    if (rc != HCCL_SUCCESS) return rc;
    if (waves != 0 && !sp.copy && (sp.mode == HCCLX_FOLD_CHAIN || sp.mode == HCCLX_FOLD_SELF_FIRST)) {
        sp.waves = waves;
        sp.pieces = wave_pieces;
    }
    Batch proto;
    proto.copy = sp.copy;
    proto.dtype = dtype;
    proto.op = op;
    proto.mode = sp.mode;
    proto.maxn = sp.maxn;
    proto.waves = sp.waves;
    proto.pieces = sp.pieces;
    if (sp.waves != 0) {
        // the kernel instance compiled for one source count takes launches whose segments all have it
        uint32_t common = 0;
        bool same = true;
        for (uint32_t i = 0; i < nseg; ++i) {
            if (segs[i].count == 0) continue;
            if (common == 0) common = segs[i].nsrc;
            same = same && segs[i].nsrc == common;
        }
        proto.waves_fixed = same ? common : 0;
    }
    proto.store_policy = store_policy_for(device_ctx(), segs, nseg, sp.copy ? 1 : dtype_size(dtype));
    Batch cur = proto;
    for (uint32_t i = 0; i < nseg; ++i) {
        const hcclx_seg_t &s = segs[i];
        if (s.count == 0) continue;
        SegDev sd;
        uint64_t tiles = 0;
        if (!make_segdev(s, sp, mode, &sd, &tiles)) {
            return fail(HCCL_E_NOT_SUPPORT, "segment " + std::to_string(i) + ": tree deeper than log2(" +
                                                std::to_string(sp.maxn) + ") levels");
        }
        if (static_cast<int>(cur.segs.size()) == kMaxSegsPerLaunch) {
            out->batches.push_back(std::move(cur));
            cur = proto;
        }
        cur.total_tiles += tiles;
        cur.tile_end.push_back(cur.total_tiles);
        cur.segs.push_back(sd);
        out->algo_bytes += static_cast<uint64_t>(s.nsrc + s.ndst) * s.count * sp.esz;
    }
    if (!cur.segs.empty()) out->batches.push_back(std::move(cur));
    return HCCL_SUCCESS;
}

int build_wide_batches(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, Built *out)
{
    if (nseg != 0 && segs == nullptr) return fail(HCCL_E_PTR, "segs is null");
    std::vector<hcclx_wide_seg_t> one;
    std::vector<PhasedStream> fan;
    const DeviceCtx *fctx = device_ctx();
    if (!split_fanout(fctx, segs, nseg, dtype_size(dtype), mode, HCCLX_MAX_WIDE_FAN, &one, &fan)) {
        return build_wide_batches_impl(segs, nseg, dtype, op, mode, out);
    }
    const uint64_t algo_before = out->algo_bytes;
    const int rc = build_wide_batches_impl(one.data(), static_cast<uint32_t>(one.size()), dtype, op, mode, out);
    if (rc != HCCL_SUCCESS) return rc;
    out->algo_bytes = algo_before;
    for (uint32_t i = 0; i < nseg; ++i) {
        out->algo_bytes += static_cast<uint64_t>(segs[i].nsrc + segs[i].ndst) * segs[i].count * dtype_size(dtype);
    }
    append_fanout(fctx, fan, out);
    return HCCL_SUCCESS;
}

// Wide segments: chain order, up to kMaxWideFan sources and destinations, one kernel for every fan-in.
int build_wide_batches_impl(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode,
                            Built *out)
{
    if (nseg != 0 && segs == nullptr) return fail(HCCL_E_PTR, "segs is null");
    if (mode != HCCLX_FOLD_CHAIN && mode != HCCLX_FOLD_SELF_FIRST && mode != HCCLX_FOLD_TREE) {
        return fail(HCCL_E_PARA, "unknown fold mode");
    }
    int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    uint32_t max_src = 0;
    for (uint32_t i = 0; i < nseg; ++i) {
        const hcclx_wide_seg_t &s = segs[i];
        if (s.nsrc == 0 || s.nsrc > HCCLX_MAX_WIDE_FAN || s.ndst == 0 || s.ndst > HCCLX_MAX_WIDE_FAN) {
            return fail(HCCL_E_PARA, "segment " + std::to_string(i) + ": nsrc/ndst outside 1.." +
                                         std::to_string(HCCLX_MAX_WIDE_FAN));
        }
        if (s.count != 0) {
            for (uint32_t k = 0; k < s.nsrc; ++k) {
                if (s.src[k] == nullptr) return fail(HCCL_E_PTR, "segment " + std::to_string(i) + ": null source");
            }
            for (uint32_t k = 0; k < s.ndst; ++k) {
                if (s.dst[k] == nullptr) return fail(HCCL_E_PTR, "segment " + std::to_string(i) + ": null destination");
            }
        }
        if (mode == HCCLX_FOLD_SELF_FIRST) {
            if (s.nsrc != s.ndst) return fail(HCCL_E_PARA, "self-first fold needs nsrc == ndst");
            // the outputs are computed sixteen at a time by different workgroups: none may overwrite a source
            // (integers have one value whatever the order and take the chain kernel: exempt)
            const uint64_t bytes = is_float_dtype(dtype) ? s.count * static_cast<uint64_t>(esz) : 0;
            for (uint32_t d = 0; d < s.ndst && bytes != 0; ++d) {
                const uint64_t lo = reinterpret_cast<uint64_t>(s.dst[d]);
                for (uint32_t k = 0; k < s.nsrc; ++k) {
                    const uint64_t a = reinterpret_cast<uint64_t>(s.src[k]);
                    if (lo < a + bytes && a < lo + bytes) {
                        return fail(HCCL_E_PARA, "segment " + std::to_string(i) + ": a destination of a wide self-first fold overlaps a source");
                    }
                }
            }
        }
        if (mode == HCCLX_FOLD_TREE) {
            const int levels = tree_levels(s.nsrc, s.prog);
            if (levels < 0) return fail(HCCL_E_PARA, "segment " + std::to_string(i) + ": malformed tree program");
            if (is_float_dtype(dtype) && (1u << levels) > HCCLX_MAX_WIDE_FAN) {
                return fail(HCCL_E_NOT_SUPPORT, "segment " + std::to_string(i) + ": tree has " + std::to_string(levels) +
                                                    " levels, the kernel holds 6");
            }
        }
        if (s.nsrc > max_src) max_src = s.nsrc;
    }
    Batch proto;
    proto.dtype = dtype;
    proto.op = op;
    proto.store_policy = store_policy_for(device_ctx(), segs, nseg, dtype_size(dtype));
    // a tree over integers equals the chain of its leaves, and so does every self-first order
    proto.mode = (mode != HCCLX_FOLD_CHAIN && is_float_dtype(dtype) && max_src > 1) ? mode : HCCLX_FOLD_CHAIN;
    proto.maxn = kMaxWideFan;
    uint32_t max_dst = 0;
    for (uint32_t i = 0; i < nseg; ++i) max_dst = segs[i].ndst > max_dst ? segs[i].ndst : max_dst;
    proto.wide_unroll = proto.mode != HCCLX_FOLD_CHAIN ? 1 : max_dst <= 1 ? kWideUnrollOne : kWideUnrollMany;
    const DeviceCtx *dctx = device_ctx();
    if (proto.wide_unroll == kWideUnrollOne && dctx) {
        uint64_t bytes = 0;
        for (uint32_t i = 0; i < nseg; ++i) bytes += segs[i].count * static_cast<uint64_t>(esz);
        if (bytes / (16 * wide_tile_vecs(kWideUnrollOne)) < dctx->wide_min_tiles) proto.wide_unroll = kWideUnrollMany;
    }
    proto.xcd_remap = (dctx && max_dst >= dctx->wide_xcd_remap_from) ? 1u : 0u;
    const uint64_t tile_vecs = wide_tile_vecs(proto.wide_unroll);
    uint64_t scale = 1;
    if (max_src <= 1) {
        // nothing is combined: any type is moved as bytes
        proto.dtype = HCCL_DATA_TYPE_INT8;
        proto.op = HCCL_REDUCE_SUM;
        scale = static_cast<uint64_t>(esz);
        esz = 1;
    } else {
        if (!is_reduce_dtype(dtype)) return fail(HCCL_E_NOT_SUPPORT, "data type cannot be reduced");
        if (op < HCCL_REDUCE_SUM || op > HCCL_REDUCE_MIN) return fail(HCCL_E_NOT_SUPPORT, "unknown reduce op");
    }
    const int ne = 16 / esz;
    Batch cur = proto;
    cur.wide.reserve(nseg < static_cast<uint32_t>(kMaxWideSegsPerLaunch) ? nseg : kMaxWideSegsPerLaunch);
    cur.tile_end.reserve(cur.wide.capacity());
    for (uint32_t i = 0; i < nseg; ++i) {
        const hcclx_wide_seg_t &s = segs[i];
        if (s.count == 0) continue;
        SegWide sd;
        std::memset(&sd, 0, sizeof(sd));
        sd.count = s.count * scale;
        sd.nsrc = s.nsrc;
        sd.ndst = s.ndst;
        for (uint32_t k = 0; k < s.nsrc; ++k) sd.src[k] = static_cast<const char *>(s.src[k]);
        for (uint32_t k = 0; k < s.ndst; ++k) sd.dst[k] = static_cast<char *>(s.dst[k]);
        if (mode == HCCLX_FOLD_CHAIN) {
            for (uint32_t k = 1; k < s.nsrc; ++k) sd.leaf_mask |= static_cast<uint64_t>(s.prog[k] ? 1 : 0) << k;
        }
        if (proto.mode == HCCLX_FOLD_TREE) {
            uint8_t code[kMaxWideFan];
            int slot_reg[kMaxWideFan];
            if (!embed_tree(s.nsrc, s.prog, kMaxWideFan, code, slot_reg)) {
                return fail(HCCL_E_NOT_SUPPORT, "segment " + std::to_string(i) + ": tree deeper than 6 levels");
            }
            for (uint32_t node = 1; node < static_cast<uint32_t>(kMaxWideFan); ++node) {
                sd.tree_codes[node / 16] |= static_cast<uint32_t>(code[node]) << (2 * (node % 16));
            }
            for (uint32_t k = 0; k < static_cast<uint32_t>(kMaxWideFan); ++k) {
                sd.src[k] = slot_reg[k] < 0 ? nullptr : static_cast<const char *>(s.src[slot_reg[k]]);
                if (slot_reg[k] >= 0) sd.leaf_mask |= 1ull << k;
            }
        }
        // a self-first segment is entered once per group of kMaxFan outputs; its tiles follow that group's first
        // destination
        const uint32_t entries = proto.mode == HCCLX_FOLD_SELF_FIRST ? (s.nsrc + kMaxFan - 1) / kMaxFan : 1;
        for (uint32_t g = 0; g < entries; ++g) {
            sd.first_dst = g * kMaxFan;
            char *lead = sd.dst[sd.first_dst];
            sd.head = fold_head_of(sd.count, esz, lead);
            sd.shift = fold_shift_of(sd.head, esz, tile_vecs, lead);
            const uint64_t tiles = fold_tiles_of(sd.count, ne, tile_vecs, sd.head, sd.shift);
            if (static_cast<int>(cur.wide.size()) == kMaxWideSegsPerLaunch) {
                out->batches.push_back(std::move(cur));
                cur = proto;
                cur.wide.reserve(kMaxWideSegsPerLaunch);
                cur.tile_end.reserve(kMaxWideSegsPerLaunch);
            }
            cur.total_tiles += tiles;
            cur.tile_end.push_back(cur.total_tiles);
            cur.wide.push_back(sd);
        }
        out->algo_bytes += static_cast<uint64_t>(s.nsrc + s.ndst) * sd.count * esz;
    }
    if (!cur.wide.empty()) out->batches.push_back(std::move(cur));
    return HCCL_SUCCESS;
}

void fill_table(const Batch &b, char *h)
{
    if (!b.phased.jobs.empty()) {
        b.phased.fill(h);
        return;
    }
    if (!b.blocks.empty()) {
        std::memcpy(h, b.blocks.data(), b.blocks.size() * sizeof(CopyBlock));
        return;
    }
    std::memcpy(h, b.tile_end.data(), b.tile_end.size() * 8);
    char *at = h + Batch::align256(b.tile_end.size() * 8);
    if (!b.segs.empty()) std::memcpy(at, b.segs.data(), b.segs.size() * sizeof(SegDev));
    if (!b.wide.empty()) std::memcpy(at, b.wide.data(), b.wide.size() * sizeof(SegWide));
}

// The common tile count of the segments of a launch, or 0 when they differ (or it does not fit 32 bits).
uint32_t uniform_tiles_of(const uint64_t *tile_end, size_t nseg)
{
    if (nseg < 2 || tile_end[0] == 0 || tile_end[0] > 0xffffffffull) return 0;
    for (size_t i = 1; i < nseg; ++i) {
        if (tile_end[i] != tile_end[0] * (i + 1)) return 0;
    }
    return static_cast<uint32_t>(tile_end[0]);
}

hipError_t dispatch_fold(int dtype, int op, int maxn, int mode, const FoldLaunch &l)
{
    switch (dtype) {
        case HCCL_DATA_TYPE_INT8: return fold_dispatch_i8(op, maxn, mode, l);
        case HCCL_DATA_TYPE_INT16: return fold_dispatch_i16(op, maxn, mode, l);
        case HCCL_DATA_TYPE_INT32: return fold_dispatch_i32(op, maxn, mode, l);
        case HCCL_DATA_TYPE_INT64: return fold_dispatch_i64(op, maxn, mode, l);
        case HCCL_DATA_TYPE_UINT64: return fold_dispatch_u64(op, maxn, mode, l);
        case HCCL_DATA_TYPE_FP16: return fold_dispatch_f16(op, maxn, mode, l);
        case HCCL_DATA_TYPE_FP32: return fold_dispatch_f32(op, maxn, mode, l);
        case HCCL_DATA_TYPE_FP64: return fold_dispatch_f64(op, maxn, mode, l);
        case HCCL_DATA_TYPE_BFP16: return fold_dispatch_bf16(op, maxn, mode, l);
        default: return hipErrorInvalidValue;
    }
}

int launch_batch(const DeviceCtx *ctx, const Batch &b, const char *d_table, hipStream_t stream)
{
    if (!b.phased.jobs.empty()) {
        const hipError_t pe = launch_phased_copy(reinterpret_cast<const PhasedJob *>(d_table),
                                                 reinterpret_cast<char *const *>(d_table + b.phased.jobs_bytes()),
                                                 static_cast<uint32_t>(b.phased.jobs.size()), b.phased.slots, b.phased.nd, stream);
        if (pe != hipSuccess) return fail_hip(pe, "phased copy kernel launch");
        return HCCL_SUCCESS;
    }
    if (!b.blocks.empty()) {
        const hipError_t be = launch_copy_blocks(reinterpret_cast<const CopyBlock *>(d_table), static_cast<uint32_t>(b.blocks.size()),
                                                 static_cast<uint32_t>(b.total_tiles), b.block_unroll, stream);
        if (be != hipSuccess) return fail_hip(be, "block copy kernel launch");
        return HCCL_SUCCESS;
    }
    FoldLaunch l;
    l.tile_end = reinterpret_cast<const uint64_t *>(d_table);
    l.segs = d_table + Batch::align256(b.tile_end.size() * 8);
    l.nseg = static_cast<uint32_t>(b.nseg());
    l.total_tiles = b.total_tiles;
    l.grid = grid_for(ctx, b.total_tiles);
    l.wide_unroll = b.wide_unroll;
    l.xcd_remap = b.xcd_remap;
    l.store_policy = b.store_policy;
    l.uniform_tiles = uniform_tiles_of(b.tile_end.data(), b.tile_end.size());
    l.waves = b.waves;
    l.pieces = b.pieces;
    l.waves_fixed = b.waves_fixed;
    l.stream = stream;
    const hipError_t e = b.copy ? fold_dispatch_copy(l) : dispatch_fold(b.dtype, b.op, b.maxn, b.mode, l);
    if (e != hipSuccess) return fail_hip(e, "fold kernel launch");
    return HCCL_SUCCESS;
}

}  // namespace
}  // namespace hcclx

using namespace hcclx;

struct hcclx_plan {
    int device = -1;
    char *d_table = nullptr;
    uint64_t table_bytes = 0;
    uint64_t algo_bytes = 0;
    std::vector<Batch> batches;
    std::vector<size_t> offsets;
};

extern "C" {

int hcclx_init(void) { return device_ctx() ? HCCL_SUCCESS : HCCL_E_RUNTIME; }

const char *hcclx_last_error(void) { return g_err.c_str(); }

uint64_t hcclx_kernels_launched(void) { return hcclx::kernels_launched(); }

int hcclx_tune(const char *name, uint64_t value)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    if (name == nullptr) return fail(HCCL_E_PTR, "name is null");
    const std::string key(name);
    if (key == "waves_from") {
        ctx->waves_from = value;
    } else if (key == "waves_max_fan") {
        if (value < 2 || value > HCCLX_MAX_FAN) return fail(HCCL_E_PARA, "waves_max_fan outside 2..16");
        ctx->waves_max_fan = static_cast<uint32_t>(value);
    } else if (key == "waves_chains") {
        ctx->waves_chains = value != 0;
    } else if (key == "waves_pieces") {
        if (value > static_cast<uint64_t>(kWavePieces)) return fail(HCCL_E_PARA, "waves_pieces beyond " + std::to_string(kWavePieces));
        ctx->waves_pieces = static_cast<uint32_t>(value);
    } else if (key == "fanout_from") {
        ctx->fanout_from = value;
    } else if (key == "moe_scatter_rows") {
        if (value != 1 && value != 2) return fail(HCCL_E_PARA, "moe_scatter_rows is 1 or 2");
        ctx->moe_scatter_rows = static_cast<uint32_t>(value);
    } else if (key == "store_through_upto") {
        ctx->store_through_upto = value;
    } else {
        return fail(HCCL_E_PARA, "unknown knob: " + key);
    }
    return HCCL_SUCCESS;
}

uint32_t hcclx_dtype_size(int dtype) { return static_cast<uint32_t>(dtype_size(dtype)); }

static int launch_built(DeviceCtx *ctx, const Built &built, hipStream_t st)
{
    for (const Batch &b : built.batches) {
        char *h = nullptr;
        char *d = nullptr;
        int rc = ring_reserve(ctx, b.bytes(), st, &h, &d);
        if (rc != HCCL_SUCCESS) return rc;
        fill_table(b, h);
        HCCLX_HIP(hipMemcpyAsync(d, h, b.bytes(), hipMemcpyHostToDevice, st));
        rc = launch_batch(ctx, b, d, st);
        if (rc != HCCL_SUCCESS) return rc;
    }
    return HCCL_SUCCESS;
}

static int plan_from(DeviceCtx *ctx, Built &built, hcclx_plan_t **plan)
{
    hcclx_plan *p = new hcclx_plan;
    p->device = ctx->device;
    p->algo_bytes = built.algo_bytes;
    p->batches = std::move(built.batches);
    size_t total = 0;
    for (const Batch &b : p->batches) {
        p->offsets.push_back(total);
        total += b.bytes();
    }
    p->table_bytes = total;
    if (total != 0) {
        PlanStage &stage = g_slots[ctx->device].stage;
        std::lock_guard<std::mutex> lock(stage.mu);
        hipError_t e = hipSuccess;
        if (stage.bytes < total) {
            if (stage.host) (void)hipHostFree(stage.host);
            stage.host = nullptr;
            stage.bytes = 0;
            const size_t want = total + total / 2;
            e = hipHostMalloc(reinterpret_cast<void **>(&stage.host), want, hipHostMallocDefault);
            if (e == hipSuccess) stage.bytes = want;
        }
        if (e == hipSuccess) {
            for (size_t i = 0; i < p->batches.size(); ++i) fill_table(p->batches[i], stage.host + p->offsets[i]);
            e = hipMalloc(reinterpret_cast<void **>(&p->d_table), total);
        }
        if (e == hipSuccess) e = hipMemcpyAsync(p->d_table, stage.host, total, hipMemcpyHostToDevice, stage.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(stage.stream);
        if (e != hipSuccess) {
            if (p->d_table) (void)hipFree(p->d_table);
            delete p;
            return fail_hip(e, "plan table upload");
        }
    }
    *plan = p;
    return HCCL_SUCCESS;
}

int hcclx_fold(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    Built built;
    int rc = build_batches(segs, nseg, dtype, op, mode, &built);
    if (rc != HCCL_SUCCESS) return rc;
    return launch_built(ctx, built, static_cast<hipStream_t>(stream));
}

int hcclx_fold_static(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    if (nseg != 0 && segs == nullptr) return fail(HCCL_E_PTR, "segs is null");
    if (nseg > HCCLX_STATIC_MAX_SEGS) {
        return fail(HCCL_E_PARA, "hcclx_fold_static takes at most " + std::to_string(HCCLX_STATIC_MAX_SEGS) +
                                     " segments per call (its launch table is a fixed array); got " + std::to_string(nseg));
    }
    SegProto sp;
    int rc = check_segs(segs, nseg, dtype, op, mode, &sp);
    if (rc != HCCL_SUCCESS) return rc;
    // the table as the kernels read it: tile_end[] (rounded up to 256 bytes), then the segment descriptors
    alignas(16) char table[HCCLX_STATIC_TABLE_BYTES];
    uint64_t *tile_end = reinterpret_cast<uint64_t *>(table);
    uint32_t live = 0;
    for (uint32_t i = 0; i < nseg; ++i) live += segs[i].count != 0 ? 1 : 0;
    if (live == 0) return HCCL_SUCCESS;
    const size_t seg_off = (static_cast<size_t>(live) * 8 + 255) & ~static_cast<size_t>(255);
    const size_t bytes = seg_off + static_cast<size_t>(live) * sizeof(SegDev);
    static_assert(((HCCLX_STATIC_MAX_SEGS * 8 + 255) & ~255) + HCCLX_STATIC_MAX_SEGS * sizeof(SegDev) <= HCCLX_STATIC_TABLE_BYTES,
                  "the fixed launch table holds HCCLX_STATIC_MAX_SEGS segments");
    std::memset(table, 0, seg_off);
    SegDev *descs = reinterpret_cast<SegDev *>(table + seg_off);
    uint64_t total = 0;
    uint32_t at = 0;
    for (uint32_t i = 0; i < nseg; ++i) {
        if (segs[i].count == 0) continue;
        uint64_t tiles = 0;
        if (!make_segdev(segs[i], sp, mode, &descs[at], &tiles)) {
            return fail(HCCL_E_NOT_SUPPORT, "segment " + std::to_string(i) + ": tree deeper than the kernel holds");
        }
        total += tiles;
        tile_end[at++] = total;
    }
    if (total > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // One table per GPU: the upload and the fold of a call are issued as a unit, and a call on another stream than
    // the previous one waits for that one's fold.  While `st` is being captured into a graph neither the wait nor
    // the record is issued (an event recorded in a capture would draw every later waiter into that capture): the
    // replays of a captured call are the caller's to order against other users of the table.
    StaticTableUse &use = g_slots[ctx->device].static_use;
    std::lock_guard<std::mutex> use_lock(use.mu);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusNone;
    }
    const bool ordered = capturing == hipStreamCaptureStatusNone;
    if (ordered && use.recorded && use.last != st) {
        const hipError_t we = hipStreamWaitEvent(st, use.done, 0);
        if (we != hipSuccess) return fail_hip(we, "hipStreamWaitEvent(launch table)");
    }
    // the table travels in kernel arguments, piece by piece; the fold kernel follows on the same stream
    for (size_t off = 0; off < bytes; off += kPutBytes) {
        TablePiece piece;
        const uint32_t n = static_cast<uint32_t>(bytes - off < kPutBytes ? bytes - off : kPutBytes);
        std::memcpy(&piece, table + off, n);
        HCCLX_LAUNCH(k_put_table, dim3(1), dim3(256), 0, st, piece, ctx->static_table + off, n);
        const hipError_t pe = hipGetLastError();
        if (pe != hipSuccess) return fail_hip(pe, "launch table upload");
    }
    FoldLaunch l;
    l.tile_end = reinterpret_cast<const uint64_t *>(ctx->static_table);
    l.segs = ctx->static_table + seg_off;
    l.nseg = live;
    l.total_tiles = total;
    l.grid = grid_for(ctx, total);
    l.wide_unroll = 1;
    l.xcd_remap = 0;
    l.store_policy = store_policy_for(ctx, segs, nseg, sp.copy ? 1 : dtype_size(dtype));
    l.uniform_tiles = uniform_tiles_of(tile_end, live);
    l.stream = st;
    hipError_t e;
    if (sp.copy) {
        e = fold_dispatch_copy(l);
    } else {
        e = dispatch_fold(dtype, op, sp.maxn, sp.mode, l);
    }
    if (e != hipSuccess) return fail_hip(e, "fold kernel launch");
    if (ordered) {
        e = hipEventRecord(use.done, st);
        if (e != hipSuccess) return fail_hip(e, "hipEventRecord(launch table)");
        use.last = st;
        use.recorded = true;
    }
    return HCCL_SUCCESS;
}

int hcclx_fold_wide(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream)
{
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    Built built;
    int rc = build_wide_batches(segs, nseg, dtype, op, mode, &built);
    if (rc != HCCL_SUCCESS) return rc;
    return launch_built(ctx, built, static_cast<hipStream_t>(stream));
}

int hcclx_plan_create(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, hcclx_plan_t **plan)
{
    if (plan == nullptr) return fail(HCCL_E_PTR, "plan is null");
    *plan = nullptr;
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    Built built;
    int rc = build_batches(segs, nseg, dtype, op, mode, &built);
    if (rc != HCCL_SUCCESS) return rc;
    return plan_from(ctx, built, plan);
}

int hcclx_plan_create_wide(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode,
                           hcclx_plan_t **plan)
{
    if (plan == nullptr) return fail(HCCL_E_PTR, "plan is null");
    *plan = nullptr;
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    Built built;
    int rc = build_wide_batches(segs, nseg, dtype, op, mode, &built);
    if (rc != HCCL_SUCCESS) return rc;
    return plan_from(ctx, built, plan);
}

int hcclx_alltoallv_plan_create(const void *const *send, void *const *recv, const uint64_t *send_counts,
                                const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, int dtype, hcclx_plan_t **plan)
{
    if (plan == nullptr) return fail(HCCL_E_PTR, "plan is null");
    *plan = nullptr;
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    const int esz = dtype_size(dtype);
    if (esz == 0) return fail(HCCL_E_NOT_SUPPORT, "unknown data type " + std::to_string(dtype));
    if (!send || !recv) return fail(HCCL_E_PTR, "send/recv pointer array is null");
    if (!send_counts || !sdispls || !rdispls) return fail(HCCL_E_PTR, "count/displacement table is null");
    if (n == 0 || n > kMaxVRanks) return fail(HCCL_E_PARA, "rank count outside 1.." + std::to_string(kMaxVRanks));
    Built built;
    Batch b;
    b.copy = true;
    b.block_unroll = ctx->a2av_direct_unroll == 1 ? 1 : ctx->a2av_direct_unroll == 4 ? 4 : 2;
    b.total_tiles = list_alltoallv_blocks(send, recv, send_counts, sdispls, rdispls, n, static_cast<uint32_t>(esz), b.block_unroll,
                                          &b.blocks);
    if (b.total_tiles > 0x7fffffffull) return fail(HCCL_E_PARA, "too much data for one launch");
    for (const CopyBlock &c : b.blocks) built.algo_bytes += 2 * c.bytes;
    if (!b.blocks.empty()) built.batches.push_back(std::move(b));
    return plan_from(ctx, built, plan);
}

int hcclx_plan_launch(const hcclx_plan_t *plan, void *stream)
{
    if (plan == nullptr) return fail(HCCL_E_PTR, "plan is null");
    DeviceCtx *ctx = device_ctx();
    if (!ctx) return HCCL_E_RUNTIME;
    if (ctx->device != plan->device) return fail(HCCL_E_PARA, "plan belongs to another device");
    for (size_t i = 0; i < plan->batches.size(); ++i) {
        int rc = launch_batch(ctx, plan->batches[i], plan->d_table + plan->offsets[i], static_cast<hipStream_t>(stream));
        if (rc != HCCL_SUCCESS) return rc;
    }
    return HCCL_SUCCESS;
}

int hcclx_plan_destroy(hcclx_plan_t *plan)
{
    if (plan == nullptr) return HCCL_SUCCESS;
    if (plan->d_table) (void)hipFree(plan->d_table);
    delete plan;
    return HCCL_SUCCESS;
}

uint64_t hcclx_plan_bytes(const hcclx_plan_t *plan) { return plan ? plan->algo_bytes : 0; }

uint64_t hcclx_plan_table_bytes(const hcclx_plan_t *plan) { return plan ? plan->table_bytes : 0; }

}  // extern "C"
