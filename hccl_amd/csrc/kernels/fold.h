// The fused fold kernel: every segment reads each of its sources once and writes each of its
// destinations once, in a single pass over HBM.
//
// It replaces the reference's per-step primitives HcommLocalCopyOnThread / HcommLocalReduceOnThread /
// Hcomm{Write,Read}[Reduce]OnThread (ABI visible in test/st/algorithm/utils/src/hccl_proxy/hccl_stub.cc:467,
// :633, :664, :705) and, when a whole template is fused, the chains of them that the templates emit, e.g.
// PostLocalReduce of the one-shot AllReduce (src/ops/all_reduce/template/aicpu/
// ins_temp_all_reduce_mesh_1D_one_shot.cc:182-197) and PostCopy of the mesh ReduceScatter
// (src/ops/reduce_scatter/template/aicpu/ins_temp_reduce_scatter_mesh_1D.cc:147-154).
//
// Bound: HBM bandwidth.  Algorithmic bytes per element: (nsrc + ndst) * sizeof(element).
#pragma once
#include "elem.h"
#include "segtab.h"
#include "launch.h"

namespace hcclx {

// 16-byte vectors each thread keeps in flight per source.  More sources -> fewer vectors per source, so
// the loads outstanding per thread stay near 16 and the register file still holds several wavefronts.  A plain
// copy does best with small tiles (two vectors per thread: 6.0 TB/s on 1 GiB against 5.55 with eight).
#ifndef HCCLX_FOLD_UNROLLS
#define HCCLX_FOLD_UNROLLS 2, 4, 4, 2, 1   // for up to 1, 2, 4, 8, 16 sources
#endif
#ifndef HCCLX_FOLD_THREADS
#define HCCLX_FOLD_THREADS 256
#endif
constexpr int kFoldThreads = HCCLX_FOLD_THREADS;
// The wide chain kernel loads eight sources at a time for U vectors per thread.  U = 2 measured 24 % faster on a
// 32-rank AllReduce than one vector with sixteen sources (the same loads outstanding, twice the contiguous run per
// source); with a single destination (the ReduceScatter shape) U = 4 measured another 3 to 5 % faster, while it
// costs 5 % where every result is written to many places.
constexpr int kWideGroup = 8;
constexpr int kWideUnrollMany = 2;   // several destinations
constexpr int kWideUnrollOne = 4;    // one destination
constexpr uint32_t kFoldDirectSegs = 64;   // up to this many segments the tile prefix is searched in place
#ifndef HCCLX_TREE16_UNROLL
#define HCCLX_TREE16_UNROLL 1   // vectors per thread of the tree over up to 16 leaf slots
#endif
static_assert(kFoldTree == 2, "fold_unroll names the tree mode by its number");
// mode: a FoldMode (segtab.h)
__host__ __device__ constexpr int fold_unroll(int maxn, int mode)
{
    constexpr int u[5] = {HCCLX_FOLD_UNROLLS};
    if (mode == 2 /* kFoldTree */ && maxn > 8) return HCCLX_TREE16_UNROLL;
    return maxn <= 1 ? u[0] : maxn <= 2 ? u[1] : maxn <= 4 ? u[2] : maxn <= 8 ? u[3] : u[4];
}
__host__ __device__ constexpr uint64_t fold_tile_vecs(int maxn, int mode)
{
    return static_cast<uint64_t>(kFoldThreads) * fold_unroll(maxn, mode);
}
// Tiles of the wide kernels: `unroll` vectors per thread (the chain: kWideUnrollMany or kWideUnrollOne; the
// self-first and tree orders: 1).
__host__ __device__ constexpr uint64_t wide_tile_vecs(int unroll)
{
    return static_cast<uint64_t>(kFoldThreads) * unroll;
}

#ifndef HCCLX_NT_LOAD
#define HCCLX_NT_LOAD 1
#endif
// Every data pointer of the library is a device pointer into HBM.  A pointer that a kernel fetched from a table has
// no address space the compiler can see, and a load through it becomes a FLAT instruction, which counts as an LDS
// operation too (every wait for LDS then also waits for the loads in flight).  These casts say what the pointers
// are, and the loads and stores become GLOBAL instructions.
typedef const u32x4_u __attribute__((address_space(1))) *global_cvec_ptr;
typedef u32x4_u __attribute__((address_space(1))) *global_vec_ptr;
__device__ __forceinline__ global_cvec_ptr as_global(const char *p) { return (global_cvec_ptr)(p); }
__device__ __forceinline__ global_vec_ptr as_global(char *p) { return (global_vec_ptr)(p); }

__device__ __forceinline__ u32x4 ld16(const char *p)
{
#if HCCLX_NT_LOAD
    return __builtin_nontemporal_load(as_global(p));
#else
    return *as_global(p);
#endif
}
// an ordinary (cached) load: the next reader of the same bytes finds them in the L2
__device__ __forceinline__ u32x4 ld16_cached(const char *p) { return *as_global(p); }
// How results leave the CU.  Two ways to store, measured on MI355X against each other and against ordinary stores:
//   stream   nontemporal: the line is marked for early eviction.  Best where many large output streams are
//            written at once (the self-first orders) and for the copy kernels (AlltoAllV 154 us against 162).
//   through  agent scope ("sc1"): written through the L2 instead of sitting there as a dirty line that has to be
//            evicted later.  Best for a single output stream (8 sources of 64 MiB folded into one output: 97.2 us
//            against 99.5 streamed and 96.8 ordinary; also when a second launch fans that output out: 174.6 us
//            against 179.8 with ordinary stores for the 8 x 64 MiB AllReduce) and for every launch that writes
//            several streams at once below the size where it is split into fold + fan-out (8 x 32 MiB AllReduce
//            in one pass: 83.8 us against 96.3).
constexpr uint32_t kStoreStream = 0;
constexpr uint32_t kStoreThrough = 1;
__device__ __forceinline__ void st16(char *p, u32x4 v)
{
    __builtin_nontemporal_store(v, as_global(p));
}
__device__ __forceinline__ void st16x(char *p, u32x4 v, uint32_t policy)
{
    if (policy == kStoreThrough) {
        // global_store_dwordx4 takes any byte address, like the compiler's own store of an unaligned vector.  The
        // compiler does not look inside an asm statement, so the one hazard of this instruction is handled here: a
        // VALU instruction that overwrites the data registers of a store of more than 8 bytes must come at least two
        // wait states after it (the compiler keeps that distance for its own stores); hence the s_nop.  Address and
        // data are VGPRs whose producers the compiler has already waited for, and no scalar operand is read.
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
    } else {
        st16(p, v);
    }
}
__device__ __forceinline__ uint64_t uniform64(uint64_t x)
{
    uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(x));
    uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(x >> 32));
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Evaluates an embedded (sub)tree bottom-up.  leaf[k] are the SLOTS leaf slots below heap node ROOT; the node
// at width w, position i of that subtree is heap node ROOT * w + i, and code(node) gives its 2-bit code.  Every
// index below is a compile time constant and every condition is wave-uniform, so the values stay in named
// registers.  The value of node ROOT ends up in leaf[0].
template <int DT, int OP, int SLOTS, int ROOT, typename C, int NE, typename CODE>
__device__ __forceinline__ void tree_eval_at(C (&leaf)[SLOTS][NE], CODE code)
{
    // level by level in place: after the pass for width w, leaf[0 .. w) hold the nodes ROOT*w .. ROOT*w + w-1
#pragma unroll
    for (int w = SLOTS / 2; w >= 1; w /= 2) {
#pragma unroll
        for (int i = 0; i < w; ++i) {
            const uint32_t c = code(ROOT * w + i);
            if (c == 2u) {
#pragma unroll
                for (int e = 0; e < NE; ++e) leaf[i][e] = Vec16<DT>::template combine<OP>(leaf[2 * i + 1][e], leaf[2 * i][e]);
            } else if (c == 1u && i != 0) {
                // pass the dst child up (for i == 0 it already sits in place)
#pragma unroll
                for (int e = 0; e < NE; ++e) leaf[i][e] = leaf[2 * i][e];
            }
        }
    }
}

template <int DT, int OP, int MAXN, typename C, int NE>
__device__ __forceinline__ void tree_eval(C (&leaf)[MAXN][NE], uint32_t codes)
{
    tree_eval_at<DT, OP, MAXN, 1, C, NE>(leaf, [codes](int node) { return (codes >> (2 * node)) & 3u; });
}

template <int DT, int OP, int MAXN, int MODE, bool CHECK>
__device__ __forceinline__ void fold_tile(const SegDev &sd, uint32_t nsrc, uint32_t ndst, uint64_t v0, uint64_t nvec,
                                          uint32_t head_bytes, uint32_t policy)
{
    constexpr int UNROLL = fold_unroll(MAXN, MODE);
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    u32x4 raw[UNROLL][MAXN];
    const uint32_t present = (MODE == kFoldTree) ? sd.leaf_mask : ((nsrc >= 32u) ? ~0u : ((1u << nsrc) - 1u));
#pragma unroll
    for (int k = 0; k < MAXN; ++k) {
        if ((present >> k) & 1u) {
            const char *p = sd.src[k] + head_bytes;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                // A lane outside the segment loads the segment's first vector and stores nothing: the loads
                // stay unconditional, so all of them are in flight at once as in the unchecked tile.
                const uint64_t vi = v0 + static_cast<uint64_t>(u) * kFoldThreads;
                raw[u][k] = ld16(p + ((!CHECK || vi < nvec) ? vi : 0) * 16);
            }
        }
    }

#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t vi = v0 + static_cast<uint64_t>(u) * kFoldThreads;
        if (CHECK && vi >= nvec) {
            continue;
        }
        if constexpr (MODE == kFoldChain) {
            C acc[NE];
            V::unpack(raw[u][0], acc);
            const uint32_t flips = sd.tree_codes;
#pragma unroll
            for (int k = 1; k < MAXN; ++k) {
                if (k < static_cast<int>(nsrc)) {
                    C x[NE];
                    V::unpack(raw[u][k], x);
                    if (OperandOrderMatters<DT, OP>::value && ((flips >> k) & 1u)) {
#pragma unroll
                        for (int e = 0; e < NE; ++e) acc[e] = V::template combine<OP>(acc[e], x[e]);
                    } else {
#pragma unroll
                        for (int e = 0; e < NE; ++e) acc[e] = V::template combine<OP>(x[e], acc[e]);
                    }
                }
            }
            const u32x4 out = V::pack(acc);
            // a constant trip count with a uniform guard: the destination pointers are then fetched in one
            // batch of scalar loads instead of one dependent load per iteration
#pragma unroll
            for (int d = 0; d < kMaxFan; ++d) {
                if (d < static_cast<int>(ndst)) st16x(sd.dst[d] + head_bytes + vi * 16, out, policy);
            }
        } else if constexpr (MODE == kFoldTree) {
            C val[MAXN][NE];
#pragma unroll
            for (int k = 0; k < MAXN; ++k) {
                if ((present >> k) & 1u) V::unpack(raw[u][k], val[k]);
            }
            tree_eval<DT, OP, MAXN, C, NE>(val, sd.tree_codes);
            const u32x4 out = V::pack(val[0]);
            // a constant trip count with a uniform guard: the destination pointers are then fetched in one
            // batch of scalar loads instead of one dependent load per iteration
#pragma unroll
            for (int d = 0; d < kMaxFan; ++d) {
                if (d < static_cast<int>(ndst)) st16x(sd.dst[d] + head_bytes + vi * 16, out, policy);
            }
        } else {
            C val[MAXN][NE];
#pragma unroll
            for (int k = 0; k < MAXN; ++k) {
                if (k < static_cast<int>(nsrc)) V::unpack(raw[u][k], val[k]);
            }
#pragma unroll
            for (int j = 0; j < MAXN; ++j) {
                if (j < static_cast<int>(nsrc)) {
                    C acc[NE];
#pragma unroll
                    for (int e = 0; e < NE; ++e) acc[e] = val[j][e];
#pragma unroll
                    for (int k = 0; k < MAXN; ++k) {
                        if (k != j && k < static_cast<int>(nsrc)) {
#pragma unroll
                            for (int e = 0; e < NE; ++e) acc[e] = V::template combine<OP>(val[k][e], acc[e]);
                        }
                    }
                    st16(sd.dst[j] + head_bytes + vi * 16, V::pack(acc));   // N output streams at once: streamed
                }
            }
        }
    }
}

// Chain mode: bit k set = step k takes the accumulated value as its source operand.
__device__ __forceinline__ uint64_t chain_flips(const SegDev &sd) { return sd.tree_codes; }
__device__ __forceinline__ uint64_t chain_flips(const SegWide &sd) { return sd.leaf_mask; }

// The last (count % NE) elements of a segment, one per thread.
template <int DT, int OP, int MAXN, int MODE, typename SEG>
__device__ __forceinline__ void fold_tail(const SEG &sd, uint32_t nsrc, uint32_t ndst, uint64_t idx)
{
    using D = DTypeOf<DT>;
    using S = typename D::S;
    using C = typename D::C;
    using Op = Combine<DT, OP>;
    if constexpr (MODE == kFoldChain) {
        C acc = D::widen(reinterpret_cast<const S *>(sd.src[0])[idx]);
        const uint64_t flips = chain_flips(sd);
        for (uint32_t k = 1; k < nsrc; ++k) {
            const C x = D::widen(reinterpret_cast<const S *>(sd.src[k])[idx]);
            acc = (OperandOrderMatters<DT, OP>::value && ((flips >> k) & 1u)) ? Op::run(acc, x) : Op::run(x, acc);
        }
        const S out = D::narrow(acc);
        for (uint32_t d = 0; d < ndst; ++d) reinterpret_cast<S *>(sd.dst[d])[idx] = out;
    } else if constexpr (MODE == kFoldTree) {
        C val[MAXN][1];
#pragma unroll
        for (int k = 0; k < MAXN; ++k) {
            if ((sd.leaf_mask >> k) & 1u) val[k][0] = D::widen(reinterpret_cast<const S *>(sd.src[k])[idx]);
        }
        if constexpr (MAXN > kMaxFan) {
            tree_eval_at<DT, OP, MAXN, 1, C, 1>(val, [&sd](int node) { return (sd.tree_codes[node / 16] >> (2 * (node % 16))) & 3u; });
        } else {
            tree_eval<DT, OP, MAXN, C, 1>(val, sd.tree_codes);
        }
        const S out = D::narrow(val[0][0]);
        for (uint32_t d = 0; d < ndst; ++d) reinterpret_cast<S *>(sd.dst[d])[idx] = out;
    } else if constexpr (MAXN > kMaxFan) {
        // The wide self-first order: the outputs of this entry's group, each from the sources as they lie in
        // memory (no destination overlaps a source in this mode).
        const uint32_t first = sd.first_dst;
        for (uint32_t j = first; j < first + kMaxFan && j < nsrc; ++j) {
            C acc = D::widen(reinterpret_cast<const S *>(sd.src[j])[idx]);
            for (uint32_t k = 0; k < nsrc; ++k) {
                if (k != j) acc = Op::run(D::widen(reinterpret_cast<const S *>(sd.src[k])[idx]), acc);
            }
            reinterpret_cast<S *>(sd.dst[j])[idx] = D::narrow(acc);
        }
    } else {
        // Every source is read before the first destination is written: a destination may alias a source.
        C val[kMaxFan];
        for (uint32_t k = 0; k < nsrc; ++k) val[k] = D::widen(reinterpret_cast<const S *>(sd.src[k])[idx]);
        for (uint32_t j = 0; j < nsrc; ++j) {
            C acc = val[j];
            for (uint32_t k = 0; k < nsrc; ++k) {
                if (k != j) acc = Op::run(val[k], acc);
            }
            reinterpret_cast<S *>(sd.dst[j])[idx] = D::narrow(acc);
        }
    }
}

// Workgroups are handed to the eight XCDs round-robin; with the remap each XCD sweeps one contiguous eighth of
// the tiles instead of every eighth tile.  Measured on chains written to many places: +5 % with 16 destinations,
// +7 % with 32; with few destinations it costs (-10 % on the 8-source, 1-destination shape), so the launcher
// asks for it from 16 destinations on.
__device__ __forceinline__ uint64_t remap_tile(uint64_t t, uint64_t total)
{
    const uint64_t q = total / 8;
    const uint64_t r = total % 8;
    const uint64_t xcd = t % 8;
    return xcd * q + (xcd < r ? xcd : r) + t / 8;
}

// Maps tile number t of a launch to its segment (the first one whose inclusive tile prefix exceeds t) and
// to the tile's number inside that segment.  Every value is wave-uniform.
__device__ __forceinline__ void locate_tile(const uint64_t *__restrict__ tile_end, const uint64_t *s_end, uint32_t nseg,
                                            bool direct, uint32_t uniform_tiles, uint64_t t, uint32_t *seg,
                                            uint64_t *tile_in_seg)
{
    if (uniform_tiles != 0) {
        // every segment has this many tiles (the slices of a two-shot, ring or NHR AllReduce): no table to search.
        // A search is a chain of dependent loads, which a launch of a few hundred workgroups cannot hide.
        const uint64_t s = t / uniform_tiles;
        *seg = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(s));
        *tile_in_seg = uniform64(t - s * uniform_tiles);
        return;
    }
    uint32_t lo = 0;
    uint32_t hi = nseg - 1;
    uint64_t before = 0;   // tiles of the segments in front of the one found
    if (direct) {
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (tile_end[mid] > t) {
                hi = mid;
            } else {
                lo = mid + 1;
            }
        }
        before = lo ? tile_end[lo - 1] : 0;
    } else {
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (s_end[mid] > t) {
                hi = mid;
            } else {
                lo = mid + 1;
            }
        }
        before = lo ? s_end[lo - 1] : 0;
    }
    *seg = __builtin_amdgcn_readfirstlane(lo);
    *tile_in_seg = uniform64(t - before);
}

template <int DT, int OP, int MAXN, int MODE>
__global__ void __launch_bounds__(kFoldThreads)
k_fold(const uint64_t *__restrict__ tile_end, const SegDev *__restrict__ segs, uint32_t nseg, uint64_t total_tiles,
       uint32_t store_policy, uint32_t uniform_tiles)
{
    const uint32_t policy = store_policy;
    constexpr int NE = Vec16<DT>::kElems;   // elements per 16-byte vector
    constexpr uint64_t TV = fold_tile_vecs(MAXN, MODE);
    extern __shared__ uint64_t s_end[];  // nseg entries, sized by the launcher
    // Few segments: the prefix is searched where it lies (every index is wave-uniform, so these are scalar
    // loads that hit the constant cache after the first workgroup); staging it in LDS would cost a barrier
    // before the first data load.  Many segments: staged once per workgroup.
    const bool direct = nseg <= kFoldDirectSegs || uniform_tiles != 0;
    if (!direct) {
        for (uint32_t i = threadIdx.x; i < nseg; i += kFoldThreads) {
            s_end[i] = tile_end[i];
        }
        __syncthreads();
    }

    for (uint64_t t = blockIdx.x; t < total_tiles; t += gridDim.x) {
        uint32_t s;
        uint64_t tl;
        locate_tile(tile_end, s_end, nseg, direct, uniform_tiles, t, &s, &tl);
        const SegDev &sd = segs[s];
        const uint32_t nsrc = sd.nsrc;
        const uint32_t ndst = sd.ndst;
        const uint64_t count = sd.count;
        const uint32_t head = sd.head;                      // elements before the aligned body
        const uint64_t body = count - head;
        const uint64_t nvec = body / NE;
        const uint32_t rem = static_cast<uint32_t>(body % NE);
        const uint32_t head_bytes = head * (16 / NE);
        const uint32_t shift = sd.shift;
        // In the first tile of a shifted grid v0 wraps below zero for the vectors in front of the segment;
        // they fail the bound check of the checked path like the ones behind its end.
        const uint64_t v0 = tl * TV + threadIdx.x - shift;
        if (tl * TV >= shift && (tl + 1) * TV - shift <= nvec) {
            fold_tile<DT, OP, MAXN, MODE, false>(sd, nsrc, ndst, v0, nvec, head_bytes, policy);
        } else {
            if (nvec != 0) fold_tile<DT, OP, MAXN, MODE, true>(sd, nsrc, ndst, v0, nvec, head_bytes, policy);
            // the last tile also takes the elements in front of and behind the vector body, one per thread
            if (tl == (nvec + shift) / TV && threadIdx.x < head + rem) {
                const uint64_t idx = threadIdx.x < head ? threadIdx.x : head + nvec * NE + (threadIdx.x - head);
                fold_tail<DT, OP, MAXN, MODE>(sd, nsrc, ndst, idx);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// One store per wavefront.  A wavefront that issues several 16-byte stores per lane in a row writes HBM a fifth
// slower than wavefronts that issue one each and end (measured on MI355X with plain fills: 12 streams of 1 GiB,
// every workgroup all 12: 5.6 TB/s; one stream per wavefront: 6.6 to 7.2), and a fold whose results go to n places
// is half writes.  Here a workgroup has one wavefront per source / destination: wavefront w loads a 1 KiB piece of
// source w into LDS; after the barrier every wavefront w < ndst reads all pieces, folds them in its own order and
// stores the piece of destination w: one global load and one global store per wavefront and piece.  A workgroup
// takes `pieces` pieces in a row (the load of the next is issued before the current one is folded); the LDS holds
// two pieces per source.  Same results, bit for bit, as the register kernel: the fold order per element is the same.
// ---------------------------------------------------------------------------------------------------
constexpr int kWaveLanes = 64;
constexpr int kWavePieces = 8;   // most pieces per source and workgroup
__host__ __device__ constexpr uint64_t waves_tile_vecs(int pieces) { return static_cast<uint64_t>(kWaveLanes) * pieces; }
// LDS bytes of the pieces: two buffers of `waves` pieces
__host__ __device__ constexpr uint32_t waves_lds_bytes(int waves) { return 2u * waves * kWaveLanes * 16u; }

// The fold of one piece by one wavefront of k_fold_waves.  The LDS traffic of this kernel is what bounds it after
// HBM (every wavefront reads every source piece: n * n reads of 1 KiB per 2 n KiB moved), so only the pieces that
// exist are read: four at a time, all four before the first is combined so that the reads overlap.  Within a group
// a missing source is read from the group's first slot and dropped by a select: as a branch around each step the
// test keeps the compiler from overlapping the steps with the reads.
template <int DT, int OP, int MODE>
__device__ __forceinline__ void waves_fold(const u32x4 *buf, uint32_t nsrc, uint32_t w, uint32_t lane, uint32_t flips,
                                           typename Vec16<DT>::C (&acc)[Vec16<DT>::NE])
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    constexpr int G = 4;
    // self-first: the wavefront's own source starts the fold (its index is not a compile-time constant: one more
    // read instead of a register picked at run time); the chain starts from the first source, read with group 0
    if constexpr (MODE != kFoldChain) V::unpack(buf[w * kWaveLanes + lane], acc);
#pragma unroll
    for (int base = 0; base < kMaxFan; base += G) {
        if (base < static_cast<int>(nsrc)) {
            u32x4 raw[G];
#pragma unroll
            for (int k = 0; k < G; ++k) {
                const uint32_t slot = static_cast<uint32_t>(base + k) < nsrc ? static_cast<uint32_t>(base + k) : static_cast<uint32_t>(base);
                raw[k] = buf[slot * kWaveLanes + lane];
            }
#pragma unroll
            for (int k = 0; k < G; ++k) {
                const int at = base + k;
                C x[NE];
                V::unpack(raw[k], x);
                if (MODE == kFoldChain && at == 0) {
#pragma unroll
                    for (int e = 0; e < NE; ++e) acc[e] = x[e];
                    continue;
                }
                const bool take = at < static_cast<int>(nsrc) && (MODE == kFoldChain || at != static_cast<int>(w));
                const bool flip = MODE == kFoldChain && OperandOrderMatters<DT, OP>::value && ((flips >> at) & 1u);
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    C r = V::template combine<OP>(x[e], acc[e]);
                    if (OperandOrderMatters<DT, OP>::value && MODE == kFoldChain) {
                        const C r2 = V::template combine<OP>(acc[e], x[e]);
                        r = flip ? r2 : r;
                    }
                    acc[e] = take ? r : acc[e];
                }
            }
        }
    }
}

// The same fold for a source count the compiler knows: straight-line code, no test per source.  Measured on the
// twelve orders of a 12-rank AllReduce (64 MiB per rank): 265 us against 273 with the tests.
template <int DT, int OP, int MODE, int N>
__device__ __forceinline__ void waves_fold_fixed(const u32x4 *buf, uint32_t w, uint32_t lane, uint32_t flips,
                                                 typename Vec16<DT>::C (&acc)[Vec16<DT>::NE])
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    constexpr int G = 4;
    if constexpr (MODE != kFoldChain) V::unpack(buf[w * kWaveLanes + lane], acc);
#pragma unroll
    for (int base = 0; base < N; base += G) {
        u32x4 raw[G];
#pragma unroll
        for (int k = 0; k < G; ++k) {
            if (base + k < N) raw[k] = buf[(base + k) * kWaveLanes + lane];
        }
#pragma unroll
        for (int k = 0; k < G; ++k) {
            const int at = base + k;
            if (at >= N) continue;
            C x[NE];
            V::unpack(raw[k], x);
            if (MODE == kFoldChain && at == 0) {
#pragma unroll
                for (int e = 0; e < NE; ++e) acc[e] = x[e];
                continue;
            }
            const bool flip = MODE == kFoldChain && OperandOrderMatters<DT, OP>::value && ((flips >> at) & 1u);
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                C r = V::template combine<OP>(x[e], acc[e]);
                if (OperandOrderMatters<DT, OP>::value && MODE == kFoldChain) {
                    const C r2 = V::template combine<OP>(acc[e], x[e]);
                    r = flip ? r2 : r;
                }
                // self-first: the wavefront's own source has been taken first and is passed over here
                acc[e] = (MODE == kFoldChain || at != static_cast<int>(w)) ? r : acc[e];
            }
        }
    }
}

// The pieces of one tile.  CHECK = false: the tile lies wholly inside the segment, no vector is tested against the
// segment's end (263 against 266 us on the same twelve orders).  Every condition that leads to the barrier is the
// same for all wavefronts of the workgroup.
template <int DT, int OP, int MODE, int NFIX, bool CHECK>
__device__ __forceinline__ void waves_tile(u32x4 *s_piece, uint32_t waves, uint32_t w, uint32_t lane, const char *src, char *dst,
                                           uint32_t nsrc, uint32_t ndst, uint64_t v_first, uint64_t nvec, uint64_t tile_first,
                                           uint32_t shift, uint32_t pieces, uint32_t flips, uint32_t store_policy)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    const bool loads = w < nsrc;
    const bool stores = w < ndst;
    // vectors in front of a shifted segment wrap below zero and fail the bound check like those behind its end; a
    // lane outside the segment loads the segment's first vector and stores nothing.
    // The load of the next piece is issued before the current one is folded.
    u32x4 next = {0, 0, 0, 0};
    if (loads) next = ld16(src + ((!CHECK || v_first < nvec) ? v_first : 0) * 16);
#pragma unroll 1
    for (uint32_t i = 0; i < pieces; ++i) {
        const uint64_t v = v_first + static_cast<uint64_t>(i) * kWaveLanes;
        // the whole piece lies outside the segment (the tile grid is rounded up)
        if (CHECK && tile_first + static_cast<uint64_t>(i) * kWaveLanes >= nvec + shift) break;
        u32x4 *buf = s_piece + (i & 1u) * waves * kWaveLanes;
        if (loads) {
            buf[w * kWaveLanes + lane] = next;
            const uint64_t vn = v + kWaveLanes;
            if (i + 1 < pieces) next = ld16(src + ((!CHECK || vn < nvec) ? vn : 0) * 16);
        }
        __syncthreads();
        if (stores && (!CHECK || v < nvec)) {
            C acc[NE];
            if constexpr (NFIX != 0) {
                waves_fold_fixed<DT, OP, MODE, NFIX>(buf, w, lane, flips, acc);
            } else {
                waves_fold<DT, OP, MODE>(buf, nsrc, w, lane, flips, acc);
            }
            st16x(dst + v * 16, V::pack(acc), store_policy);
        }
    }
}

// NFIX != 0: every segment of the launch has NFIX sources (the launcher checks); 0: the count is read per segment.
template <int DT, int OP, int MODE, int NFIX>
__global__ void __launch_bounds__(kMaxFan * kWaveLanes)
k_fold_waves(const uint64_t *__restrict__ tile_end, const SegDev *__restrict__ segs, uint32_t nseg, uint32_t pieces,
             uint32_t store_policy, uint32_t uniform_tiles)
{
    static_assert(MODE == kFoldChain || MODE == kFoldSelfFirst, "trees stay on the register kernel");
    constexpr int NV = Vec16<DT>::kElems;   // elements per 16-byte vector
    extern __shared__ u32x4 s_piece[];      // [2][waves][64], then the staged tile prefix when it is searched in LDS
    const uint32_t waves = blockDim.x / kWaveLanes;
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x / kWaveLanes);
    const uint32_t lane = threadIdx.x % kWaveLanes;
    uint32_t s = 0;
    uint64_t tl = blockIdx.x;
    if (nseg != 1) {   // a single segment (the n orders of an AllReduce): the tile number is the tile in the segment
        const uint64_t *s_end = reinterpret_cast<const uint64_t *>(s_piece + 2 * waves * kWaveLanes);
        const bool direct = nseg <= kFoldDirectSegs || uniform_tiles != 0;
        if (!direct) {
            uint64_t *stage = reinterpret_cast<uint64_t *>(s_piece + 2 * waves * kWaveLanes);
            for (uint32_t i = threadIdx.x; i < nseg; i += blockDim.x) stage[i] = tile_end[i];
            __syncthreads();
        }
        locate_tile(tile_end, s_end, nseg, direct, uniform_tiles, blockIdx.x, &s, &tl);
    }
    const SegDev &sd = segs[s];
    // the pointers are fetched whether or not this wavefront has a source / destination (the arrays hold kMaxFan
    // entries and a workgroup at most as many wavefronts)
    const char *src_base = sd.src[w];
    char *dst_base = sd.dst[w];
    const uint32_t nsrc = NFIX != 0 ? static_cast<uint32_t>(NFIX) : sd.nsrc;
    const uint32_t ndst = sd.ndst;
    const uint32_t head = sd.head;
    const uint32_t shift = sd.shift;
    const uint64_t count = sd.count;
    const uint32_t flips = sd.tree_codes;
    const uint64_t body = count - head;
    const uint64_t nvec = body / NV;
    const uint32_t rem = static_cast<uint32_t>(body % NV);
    const uint32_t head_bytes = head * (16 / NV);
    const uint64_t TV = waves_tile_vecs(static_cast<int>(pieces));
    const uint64_t v_first = tl * TV + lane - shift;
    const char *src = src_base + head_bytes;
    char *dst = dst_base + head_bytes;
    if (tl * TV >= shift && (tl + 1) * TV - shift <= nvec) {
        waves_tile<DT, OP, MODE, NFIX, false>(s_piece, waves, w, lane, src, dst, nsrc, ndst, v_first, nvec, tl * TV, shift, pieces,
                                              flips, store_policy);
        return;   // a tile inside the segment holds none of the elements outside the vector body
    }
    if (nvec != 0) {
        waves_tile<DT, OP, MODE, NFIX, true>(s_piece, waves, w, lane, src, dst, nsrc, ndst, v_first, nvec, tl * TV, shift, pieces,
                                             flips, store_policy);
    }
    // the last tile (the one that holds vector nvec + shift; said without a division, which takes hundreds of cycles
    // for 64-bit operands) also takes the elements in front of and behind the vector body, one per thread
    if (tl * TV <= nvec + shift && nvec + shift < (tl + 1) * TV && threadIdx.x < head + rem) {
        const uint64_t idx = threadIdx.x < head ? threadIdx.x : head + nvec * NV + (threadIdx.x - head);
        fold_tail<DT, OP, kMaxFan, MODE>(sd, nsrc, ndst, idx);
    }
}

// More than kMaxFan sources or destinations, chain order: the sources are walked in groups of kMaxFan,
// each group loaded before it is folded in, so the loads in flight per thread stay what the 16-source kernel
// has.  One vector per thread and tile.
template <int DT, int OP, int U, bool CHECK>
__device__ __forceinline__ void fold_tile_wide(const SegWide &sd, uint32_t nsrc, uint32_t ndst, uint64_t v0, uint64_t nvec,
                                               uint32_t head_bytes, uint32_t policy)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    constexpr int G = kWideGroup;
    bool ok[U];
    uint64_t off[U];
    C acc[U][NE];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint64_t v = v0 + static_cast<uint64_t>(u) * kFoldThreads;
        // A lane outside the segment loads the segment's first vector and stores nothing: the loads stay
        // unconditional, so all of a group are in flight at once as in the unchecked tile.
        ok[u] = !CHECK || v < nvec;
        off[u] = head_bytes + (ok[u] ? v : 0) * 16;
        V::unpack(ld16(sd.src[0] + off[u]), acc[u]);
    }
    const uint64_t flips = sd.leaf_mask;
    for (uint32_t base = 1; base < nsrc; base += G) {
        u32x4 raw[U][G];
#pragma unroll
        for (int k = 0; k < G; ++k) {
            if (base + k < nsrc) {
#pragma unroll
                for (int u = 0; u < U; ++u) raw[u][k] = ld16(sd.src[base + k] + off[u]);
            }
        }
#pragma unroll
        for (int k = 0; k < G; ++k) {
            if (base + k < nsrc) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    C x[NE];
                    V::unpack(raw[u][k], x);
                    if (OperandOrderMatters<DT, OP>::value && ((flips >> (base + k)) & 1u)) {
#pragma unroll
                        for (int e = 0; e < NE; ++e) acc[u][e] = V::template combine<OP>(acc[u][e], x[e]);
                    } else {
#pragma unroll
                        for (int e = 0; e < NE; ++e) acc[u][e] = V::template combine<OP>(x[e], acc[u][e]);
                    }
                }
            }
        }
    }
    for (uint32_t base = 0; base < ndst; base += kMaxFan) {
#pragma unroll
        for (int d = 0; d < kMaxFan; ++d) {
            if (base + d < ndst) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (ok[u]) st16x(sd.dst[base + d] + off[u], V::pack(acc[u]), policy);
                }
            }
        }
    }
}

// The value of the subtree over leaf slots G * kMaxFan .. G * kMaxFan + kMaxFan - 1 (heap node
// kMaxWideFan / kMaxFan + G); nothing is loaded and `out` is left alone when no leaf of it is present.
template <int DT, int OP, int G>
__device__ __forceinline__ void wide_subtree(const SegWide &sd, uint64_t off, uint64_t mask,
                                             typename Vec16<DT>::C (&out)[Vec16<DT>::NE])
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    const uint32_t present = static_cast<uint32_t>(mask >> (G * kMaxFan)) & 0xffffu;
    if (present == 0) {
        return;
    }
    u32x4 raw[kMaxFan];
#pragma unroll
    for (int k = 0; k < kMaxFan; ++k) {
        if ((present >> k) & 1u) raw[k] = ld16(sd.src[G * kMaxFan + k] + off);
    }
    C val[kMaxFan][NE];
#pragma unroll
    for (int k = 0; k < kMaxFan; ++k) {
        if ((present >> k) & 1u) V::unpack(raw[k], val[k]);
    }
    tree_eval_at<DT, OP, kMaxFan, kMaxWideFan / kMaxFan + G, C, NE>(
        val, [&sd](int node) { return (sd.tree_codes[node / 16] >> (2 * (node % 16))) & 3u; });
#pragma unroll
    for (int e = 0; e < NE; ++e) out[e] = val[0][e];
}

// A tree over up to kMaxWideFan leaf slots: the four subtrees of kMaxFan slots below heap nodes 4 .. 7 are
// evaluated one after the other, each with its leaves loaded first as in the 16-slot kernel, and their values go
// through the two top levels.
template <int DT, int OP, bool CHECK>
__device__ __forceinline__ void fold_tile_wide_tree(const SegWide &sd, uint32_t ndst, uint64_t v, uint64_t nvec,
                                                    uint32_t head_bytes, uint32_t policy)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    constexpr int kGroups = kMaxWideFan / kMaxFan;
    if (CHECK && v >= nvec) {
        return;
    }
    const uint64_t off = head_bytes + v * 16;
    const uint64_t mask = sd.leaf_mask;
    auto code = [&sd](int node) { return (sd.tree_codes[node / 16] >> (2 * (node % 16))) & 3u; };
    C part[kGroups][NE];
    wide_subtree<DT, OP, 0>(sd, off, mask, part[0]);
    wide_subtree<DT, OP, 1>(sd, off, mask, part[1]);
    wide_subtree<DT, OP, 2>(sd, off, mask, part[2]);
    wide_subtree<DT, OP, 3>(sd, off, mask, part[3]);
    static_assert(kMaxFan == 16 && kGroups == 4, "the subtree roots above are heap nodes 4 .. 7");
    tree_eval_at<DT, OP, kGroups, 1, C, NE>(part, code);
    const u32x4 out = V::pack(part[0]);
    for (uint32_t base = 0; base < ndst; base += kMaxFan) {
#pragma unroll
        for (int d = 0; d < kMaxFan; ++d) {
            if (base + d < ndst) st16x(sd.dst[base + d] + off, out, policy);
        }
    }
}

// The self-first order among more than kMaxFan ranks: this segment entry computes the kMaxFan outputs
// first_dst .. first_dst + kMaxFan - 1 (a segment of n ranks is entered once per such group).  Output j starts
// from src[j] and takes the other sources in ascending order; the sources are loaded in groups of kMaxFan and every
// loaded vector goes into all accumulators but its own.  Destinations must not overlap sources: other workgroups
// still read what this one would overwrite.
template <int DT, int OP, bool CHECK>
__device__ __forceinline__ void fold_tile_wide_self(const SegWide &sd, uint32_t nsrc, uint64_t v, uint64_t nvec,
                                                    uint32_t head_bytes)
{
    using V = Vec16<DT>;
    using C = typename V::C;
    constexpr int NE = V::NE;
    if (CHECK && v >= nvec) {
        return;
    }
    const uint64_t off = head_bytes + v * 16;
    const uint32_t first = sd.first_dst;
    C acc[kMaxFan][NE];
    {
        u32x4 raw[kMaxFan];
#pragma unroll
        for (int j = 0; j < kMaxFan; ++j) {
            if (first + j < nsrc) raw[j] = ld16(sd.src[first + j] + off);
        }
#pragma unroll
        for (int j = 0; j < kMaxFan; ++j) {
            if (first + j < nsrc) V::unpack(raw[j], acc[j]);
        }
    }
    constexpr int G = 8;   // sources per load group: the unrolled body is G x kMaxFan updates
    for (uint32_t base = 0; base < nsrc; base += G) {
        u32x4 raw[G];
#pragma unroll
        for (int k = 0; k < G; ++k) {
            if (base + k < nsrc) raw[k] = ld16(sd.src[base + k] + off);
        }
        // only the groups at first and first + G hold the outputs' own sources: source base + k is output
        // j's own when j == k + (base - first)
        const bool own_lo = (base == first);
        const bool own_hi = (base == first + G);
#pragma unroll
        for (int k = 0; k < G; ++k) {
            if (base + k < nsrc) {
                C x[NE];
                V::unpack(raw[k], x);
#pragma unroll
                for (int j = 0; j < kMaxFan; ++j) {
                    const bool own = (own_lo && j == k) || (own_hi && j == k + G);
                    if (first + j < nsrc && !own) {
#pragma unroll
                        for (int e = 0; e < NE; ++e) acc[j][e] = V::template combine<OP>(x[e], acc[j][e]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < kMaxFan; ++j) {
        if (first + j < nsrc) st16(sd.dst[first + j] + off, V::pack(acc[j]));
    }
}

template <int DT, int OP, int MODE, int U>
__global__ void __launch_bounds__(kFoldThreads)
k_fold_wide(const uint64_t *__restrict__ tile_end, const SegWide *__restrict__ segs, uint32_t nseg, uint64_t total_tiles,
            uint32_t xcd_remap, uint32_t store_policy, uint32_t uniform_tiles)
{
    constexpr int NE = Vec16<DT>::kElems;
    const uint32_t policy = store_policy;
    static_assert(MODE == kFoldChain || U == 1, "only the chain moves several vectors per thread");
    constexpr uint64_t TV = wide_tile_vecs(U);
    extern __shared__ uint64_t s_end[];
    const bool direct = nseg <= kFoldDirectSegs || uniform_tiles != 0;
    if (!direct) {
        for (uint32_t i = threadIdx.x; i < nseg; i += kFoldThreads) {
            s_end[i] = tile_end[i];
        }
        __syncthreads();
    }
    for (uint64_t t = blockIdx.x; t < total_tiles; t += gridDim.x) {
        uint32_t s;
        uint64_t tl;
        locate_tile(tile_end, s_end, nseg, direct, uniform_tiles, xcd_remap ? remap_tile(t, total_tiles) : t, &s, &tl);
        const SegWide &sd = segs[s];
        const uint32_t nsrc = sd.nsrc;
        const uint32_t ndst = sd.ndst;
        const uint32_t head = sd.head;
        const uint64_t body = sd.count - head;
        const uint64_t nvec = body / NE;
        const uint32_t rem = static_cast<uint32_t>(body % NE);
        const uint32_t head_bytes = head * (16 / NE);
        const uint32_t shift = sd.shift;
        const uint64_t v = tl * TV + threadIdx.x - shift;   // wraps in front of a shifted segment: fails the check
        if (tl * TV >= shift && (tl + 1) * TV - shift <= nvec) {
            if constexpr (MODE == kFoldTree) {
                fold_tile_wide_tree<DT, OP, false>(sd, ndst, v, nvec, head_bytes, policy);
            } else if constexpr (MODE == kFoldSelfFirst) {
                fold_tile_wide_self<DT, OP, false>(sd, nsrc, v, nvec, head_bytes);
            } else {
                fold_tile_wide<DT, OP, U, false>(sd, nsrc, ndst, v, nvec, head_bytes, policy);
            }
        } else {
            if constexpr (MODE == kFoldTree) {
                fold_tile_wide_tree<DT, OP, true>(sd, ndst, v, nvec, head_bytes, policy);
            } else if constexpr (MODE == kFoldSelfFirst) {
                fold_tile_wide_self<DT, OP, true>(sd, nsrc, v, nvec, head_bytes);
            } else {
                if (nvec != 0) fold_tile_wide<DT, OP, U, true>(sd, nsrc, ndst, v, nvec, head_bytes, policy);
            }
            if (tl == (nvec + shift) / TV && threadIdx.x < head + rem) {
                const uint64_t idx = threadIdx.x < head ? threadIdx.x : head + nvec * NE + (threadIdx.x - head);
                fold_tail<DT, OP, kMaxWideFan, MODE>(sd, nsrc, ndst, idx);
            }
        }
    }
}

// Host-side geometry, used by the launcher to build tile_end[].
// Elements of a segment in front of the first 16-byte boundary of its first destination.
inline uint32_t fold_head_of(uint64_t count, int esz, const void *dst0)
{
    const uint64_t bytes = (16 - (reinterpret_cast<uint64_t>(dst0) & 15)) & 15;
    if (bytes % esz != 0) {
        return 0;   // the pointer is not element-aligned: no element boundary falls on a 16-byte boundary
    }
    const uint64_t head = bytes / esz;
    return static_cast<uint32_t>(head < count ? head : count);
}

// Vectors by which the tile grid is shifted so that tiles are aligned in the address space of dst0.
inline uint32_t fold_shift_of(uint32_t head, int esz, uint64_t tile_vecs, const void *dst0)
{
    const uint64_t body_addr = reinterpret_cast<uint64_t>(dst0) + static_cast<uint64_t>(head) * esz;
    if (body_addr % 16 != 0) {
        return 0;   // no aligned body (see fold_head_of)
    }
    return static_cast<uint32_t>((body_addr % (tile_vecs * 16)) / 16);
}

inline uint64_t fold_tiles_of(uint64_t count, int ne, uint64_t tile_vecs, uint32_t head, uint32_t shift)
{
    if (count == 0) {
        return 0;
    }
    const uint64_t body = count - head;
    const uint64_t nvec = body / ne;
    const uint64_t units = shift + nvec + ((head + body % ne) ? 1 : 0);
    return (units + tile_vecs - 1) / tile_vecs;
}

struct FoldLaunch {
    const uint64_t *tile_end;  // device
    const void *segs;          // device: SegDev[], or SegWide[] for the wide kernel
    uint32_t nseg;
    uint64_t total_tiles;
    uint32_t grid;
    int wide_unroll;           // the wide chain kernel: vectors per thread (kWideUnrollMany or kWideUnrollOne)
    uint32_t xcd_remap;        // the wide kernels: give each XCD a contiguous eighth of the tiles
    uint32_t store_policy;     // kStoreStream / kStoreThrough
    uint32_t uniform_tiles;    // non-zero: every segment has this many tiles, tile t belongs to segment t / uniform_tiles
    uint32_t waves = 0;        // non-zero: the one-store-per-wavefront kernel with this many wavefronts per workgroup
    uint32_t pieces = 1;       // and this many 1 KiB pieces per source and workgroup
    uint32_t waves_fixed = 0;  // non-zero: every segment of the launch has this many sources
    hipStream_t stream;
};

// One translation unit per data type defines these (fold_inst.hip).
#define HCCLX_DECLARE_FOLD(NAME) hipError_t fold_dispatch_##NAME(int op, int maxn, int mode, const FoldLaunch &l);
HCCLX_DECLARE_FOLD(i8)
HCCLX_DECLARE_FOLD(i16)
HCCLX_DECLARE_FOLD(i32)
HCCLX_DECLARE_FOLD(i64)
HCCLX_DECLARE_FOLD(u64)
HCCLX_DECLARE_FOLD(f16)
HCCLX_DECLARE_FOLD(f32)
HCCLX_DECLARE_FOLD(f64)
HCCLX_DECLARE_FOLD(bf16)
hipError_t fold_dispatch_copy(const FoldLaunch &l);

}  // namespace hcclx
