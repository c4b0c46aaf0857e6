// Device-side work tables shared by the host launcher and the kernels.
//
// A launch processes a list of segments.  A segment is one contiguous run of elements with up to
// kMaxFan sources and up to kMaxFan destinations; it is cut into tiles of 256 threads x UNROLL x 16 B
// (per source).  tile_end[] is the inclusive prefix sum of tiles per segment, staged into LDS by every
// workgroup and binary-searched to map a tile number to its segment.
#pragma once
#include <stdint.h>

namespace hcclx {

constexpr int kMaxFan = 16;        // sources fused in one pass / destinations written in one pass
constexpr int kMaxWideFan = 64;    // the same for the wide chain kernel (communicators of more than 16 ranks)
constexpr int kThreads = 256;      // workgroup size: 4 wavefronts of 64
constexpr int kMaxSegsPerLaunch = 2048;  // tile_end[] must fit the LDS staging array (16 KiB)
constexpr int kMaxWideSegsPerLaunch = 512;   // and a launch's table one slice of the descriptor ring

struct SegDev {
    uint64_t count;            // elements (bytes for the copy kernel)
    uint32_t nsrc;
    uint32_t ndst;
    const char *src[kMaxFan];  // in fold order
    char *dst[kMaxFan];
    // Tree mode: the tree is embedded in a complete binary tree with MAXN leaf slots (heap numbering: root
    // 1, children of i are 2i = the step's dst side and 2i+1 = its src side, leaf slots MAXN .. 2*MAXN-1
    // hold src[slot - MAXN]).  Two bits per inner node i at bit 2*i: 0 = nothing below, 1 = take the dst
    // child unchanged, 2 = child(2i+1) (+) child(2i).  leaf_mask has bit k set when src[k] is present.
    // Chain mode: bit k of tree_codes set = step k is  acc = acc (+) src[k]  instead of  src[k] (+) acc  (only
    // floating-point max and min tell the two apart).
    uint32_t tree_codes;
    uint32_t leaf_mask;
    // Elements in front of the first 16-byte boundary of dst[0]; they are handled one by one so that the
    // vector stores to dst[0] (and every pointer that shares its alignment) are aligned.
    uint32_t head;
    // The tile grid is shifted by this many 16-byte vectors so that tile boundaries fall on multiples of
    // the tile size in dst[0]'s address space: every wavefront then stores whole, aligned cache lines.
    // The first tile is partial when shift != 0.
    uint32_t shift;
};

// A segment of the wide kernels.  Chain: acc = src[0]; acc = src[k] (+) acc for k = 1 .. nsrc-1, or
// acc (+) src[k] where bit k of leaf_mask is set.  Tree: as in
// SegDev, embedded in a complete binary tree with kMaxWideFan leaf slots; the 2-bit code of inner node i sits at
// bit 2 * (i % 16) of tree_codes[i / 16].  In both the value goes to every dst.  Self-first: nsrc == ndst, and
// the entry computes the outputs first_dst .. first_dst + kMaxFan - 1 only (the launcher enters a segment once per
// such group).  head and shift as in SegDev, for the tile size of the mode.
struct SegWide {
    uint64_t count;
    uint32_t nsrc;
    uint32_t ndst;
    uint32_t head;
    uint32_t shift;
    uint64_t leaf_mask;
    uint32_t tree_codes[4];
    uint32_t first_dst;
    uint32_t reserved;
    const char *src[kMaxWideFan];
    char *dst[kMaxWideFan];
};

// How the sources of a segment are folded.
enum FoldMode : int {
    // acc = src[0]; for k = 1..nsrc-1: acc = src[k] (+) acc; the one value goes to every dst.
    kFoldChain = 0,
    // nsrc == ndst; dst[j] = fold starting from src[j], then src[k] for k ascending, k != j.
    kFoldSelfFirst = 1,
    // A binary tree of at most log2(MAXN) levels over the sources (see SegDev::tree_codes); the value of
    // the root goes to every dst.
    kFoldTree = 2,
};

}  // namespace hcclx
