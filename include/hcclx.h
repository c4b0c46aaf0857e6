/*
 * hcclx.h -- the thin C ABI over the HIP kernels of the virtual-rank backend.
 *
 * This is the boundary a host runtime binds (C++, cgo, JNI, ctypes ...): plain pointers and sizes, no
 * C++ or torch types.  All data pointers are device pointers in one GPU's HBM; tables (segment lists,
 * host count arrays) are host pointers unless stated otherwise.  `stream` is a hipStream_t (NULL = the
 * default stream).  Work is enqueued, not completed, when a call returns.  Every function returns an
 * HcclResult value (0 = HCCL_SUCCESS); hcclx_last_error() gives the text of the last failure on the
 * calling thread.
 *
 * What each entry point replaces in the reference (paths relative to the reference tree):
 *   hcclx_fold / hcclx_plan_*   the Hcomm data primitives the templates enqueue -- HcommLocalCopyOnThread,
 *                               HcommLocalReduceOnThread, HcommWriteOnThread, HcommReadOnThread,
 *                               HcommWriteReduceOnThread, HcommReadReduceOnThread
 *                               (test/st/algorithm/utils/src/hccl_proxy/hccl_stub.cc:467, :633, :495, :534,
 *                               :664, :705) and the CPU reduce AicpuReduce
 *                               (src/ops/op_common/template/wrapper/alg_data_trans_wrapper.cc:1165-1252);
 *   hcclx_alltoallv             pack/unpack of InsTempAlltoAllVMesh1D
 *                               (src/ops/all_to_all_v/template/aicpu/ins_temp_all_to_all_v_mesh_1D.cc:275-339,
 *                               :412-440);
 *   hcclx_allgatherv            InsTempAllGatherVMesh1D
 *                               (src/ops/all_gather_v/template/aicpu/ins_temp_all_gather_v_mesh_1D.cc:97-242).
 */
#ifndef HCCL_AMD_HCCLX_H_
#define HCCL_AMD_HCCLX_H_

#include <stdint.h>
#include "hccl_types.h"

#ifdef __cplusplus
extern "C" {
#endif

#define HCCLX_MAX_FAN 16

/* How the sources of a segment are folded; every step is  acc = src (+) acc  (operand order of
 * AicpuReduceTemplate, alg_data_trans_wrapper.cc:1226-1243). */
typedef enum {
    /* acc = src[0]; for k = 1 .. nsrc-1: acc = src[k] (+) acc; the result goes to dst[0 .. ndst-1].
     * A non-zero prog[k] turns step k into  acc = acc (+) src[k]  (a ring hands the accumulated value on as the
     * source operand); only floating-point MAX and MIN tell the two apart, for signed zeros and NaNs. */
    HCCLX_FOLD_CHAIN = 0,
    /* nsrc == ndst; dst[j] = fold that starts from src[j] and then takes src[k], k ascending, k != j:
     * the per-rank order of the one-shot AllReduce and of the CPU-reduce NHR AllReduce
     * (ins_temp_all_reduce_mesh_1D_one_shot.cc:182-197, ins_temp_all_reduce_aicpu_reduce_nhr.cc:226-233). */
    HCCLX_FOLD_SELF_FIRST = 1,
    /* A binary tree over the sources, for schedules that no chain reproduces (the NHR and recursive
     * halving-doubling reduce-scatter phases, ins_temp_all_reduce_nhr.cc:183-243).  Registers 0 .. nsrc-1
     * start as src[0 .. nsrc-1]; step t does  reg[prog[2t]] = reg[prog[2t+1]] (+) reg[prog[2t]];  there are
     * nsrc-1 steps, every register but 0 is consumed exactly once as a source, and register 0 holds the
     * result, which goes to dst[0 .. ndst-1]. */
    HCCLX_FOLD_TREE = 2
} hcclx_fold_mode_t;

/* One contiguous run of `count` elements: nsrc sources (fold order), ndst destinations.
 * nsrc == 1 is a copy (to ndst places).  A destination may be the same run as one of the sources (an
 * in-place step); any other overlap between a destination and a source of the same launch is a race. */
typedef struct {
    uint64_t count;
    uint32_t nsrc;
    uint32_t ndst;
    const void *src[HCCLX_MAX_FAN];
    void *dst[HCCLX_MAX_FAN];
    uint8_t prog[2 * HCCLX_MAX_FAN]; /* HCCLX_FOLD_TREE: (dst register, src register) per step;
                                        HCCLX_FOLD_CHAIN: prog[k] != 0 swaps the operands of step k; else unused */
} hcclx_seg_t;

/* A segment with up to HCCLX_MAX_WIDE_FAN sources and destinations, for communicators of more than
 * HCCLX_MAX_FAN ranks.  The modes are those of hcclx_seg_t; a floating-point tree may have up to six levels.
 * Aliasing rules as for hcclx_seg_t, except HCCLX_FOLD_SELF_FIRST over floating-point types: there no
 * destination may overlap a source (the outputs are computed sixteen at a time by different workgroups, each of
 * which reads every source; such a call is rejected). */
#define HCCLX_MAX_WIDE_FAN 64
typedef struct {
    uint64_t count;
    uint32_t nsrc;
    uint32_t ndst;
    const void *src[HCCLX_MAX_WIDE_FAN];
    void *dst[HCCLX_MAX_WIDE_FAN];
    uint8_t prog[2 * HCCLX_MAX_WIDE_FAN]; /* as in hcclx_seg_t */
} hcclx_wide_seg_t;

/* Library set-up for the current device: creates the descriptor arena.  Idempotent.  Called lazily by the
 * other entry points; call it yourself to keep allocation out of the first timed call. */
int hcclx_init(void);

/* Text of the last error raised on this thread ("" if none). */
const char *hcclx_last_error(void);

/* Sets one of the launch-policy knobs of the current device at run time (the same knobs the HCCLX_* environment
 * variables set when the device context is made; name = the variable's name without the prefix, lower case):
 *   "waves_from"      bytes written from which self-first folds take the one-store-per-wavefront kernel (0 = never)
 *   "waves_max_fan"   widest segment (sources / destinations) that kernel is used for (2..16)
 *   "waves_chains"    non-zero: chains whose value goes to several places take it at every size (else up to 256 KiB
 *                     per place)
 *   "waves_pieces"    1 KiB pieces per source and workgroup (0 = chosen per launch; another value also takes the
 *                     launches for which the register kernel is otherwise kept)
 *   "fanout_from"     bytes read and written from which a fold with several destinations is split into fold + fan-out
 *   "store_through_upto"  bytes written up to which multi-destination folds store through the L2
 *   "moe_scatter_rows"  entries per workgroup of the MoE dispatch of long rows (1 or 2)
 * Plans made before the call keep the kernels they were made for.  The knobs are plain fields of the device's
 * context: set them while no other thread is planning a launch on that device.  Returns HCCL_E_PARA for an unknown
 * name or a value out of range.  No counterpart in the reference. */
int hcclx_tune(const char *name, uint64_t value);

/* Number of GPU kernels the calling host thread has launched through this library so far (a running count; take
 * the difference around a call to learn how many kernels it made -- a fold whose result fans out to many places is
 * two, a large AllGatherV one per length class of its runs).  No counterpart in the reference. */
uint64_t hcclx_kernels_launched(void);

/* Size in bytes of an HcclDataType (0 if unknown).  DATATYPE_SIZE_TABLE, alg_param.h:43-45. */
uint32_t hcclx_dtype_size(int dtype);

/* Fold (reduce and/or copy) a list of segments in one pass over HBM.
 * dtype: HcclDataType of the elements; reduce types are int8 int16 int32 int64 uint64 fp16 fp32 fp64 bf16.
 * For nsrc == 1 everywhere any dtype with a known size is accepted (pure copy).  op: HcclReduceOp.
 * All segments of a call share nsrc's upper bound HCCLX_MAX_FAN.  segs is a host array, copied before
 * return.  The launch table is uploaded at call time through a ring of pinned slots, so this call (like every
 * entry point that takes host tables and is not a plan) returns HCCL_E_NOT_SUPPORT on a stream that is being
 * captured into a HIP graph: create a plan outside the capture and capture hcclx_plan_launch. */
int hcclx_fold(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream);
/* The same for wide segments. */
int hcclx_fold_wide(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream);

/* hcclx_fold for callers that cannot allocate: code that runs under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same results bit for bit, but
 * the launch table lives in a fixed array of HCCLX_STATIC_TABLE_BYTES bytes that every GPU the library runs on
 * holds until the process ends, and reaches it through kernel arguments: the call makes no hipMalloc, hipFree,
 * hipHostMalloc or copy, also on its first use (hcclx_init() on the device beforehand does the one-time set-up).
 * At most HCCLX_STATIC_MAX_SEGS segments of at most HCCLX_MAX_FAN sources and destinations per call (more:
 * HCCL_E_PARA); always the register-resident kernels, one launch, so large many-destination folds run slower than
 * through hcclx_fold.  Every call on a GPU uses that GPU's one table.  Calls on the same stream follow each other
 * by stream order; a call on another stream than the previous call's first waits (hipStreamWaitEvent on an event
 * the library made at set-up, no allocation) for that call's fold kernel, and concurrent host threads take turns,
 * so eager calls on any mix of streams and threads are safe and merely serialise on the table.  The one case
 * left to the caller: a call captured into a HIP graph records no such event, so replays of that graph must not
 * overlap in time with other users of the table (other replays, or eager calls on other streams). */
#define HCCLX_STATIC_MAX_SEGS 128
#define HCCLX_STATIC_TABLE_BYTES 40960
int hcclx_fold_static(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, void *stream);

/* The same, split in two so that a repeated collective uploads its table once. */
typedef struct hcclx_plan hcclx_plan_t;
int hcclx_plan_create(const hcclx_seg_t *segs, uint32_t nseg, int dtype, int op, int mode, hcclx_plan_t **plan);
/* A plan over wide segments; launched, measured and destroyed like any other plan. */
int hcclx_plan_create_wide(const hcclx_wide_seg_t *segs, uint32_t nseg, int dtype, int op, int mode,
                           hcclx_plan_t **plan);
int hcclx_plan_launch(const hcclx_plan_t *plan, void *stream);
int hcclx_plan_destroy(hcclx_plan_t *plan);
/* Algorithmic bytes one launch of the plan moves: sum over segments of (nsrc + ndst) * count * size. */
uint64_t hcclx_plan_bytes(const hcclx_plan_t *plan);
/* Bytes of device memory the plan's launch tables occupy. */
uint64_t hcclx_plan_table_bytes(const hcclx_plan_t *plan);

/* AlltoAllV among n virtual ranks whose buffers live in this GPU.
 *   send[i], recv[i]      device base pointers of rank i                               (host arrays, n)
 *   send_counts[i*n + j]  elements rank i sends to rank j, taken at sdispls[i*n + j]
 *   rdispls[j*n + i]      element offset in recv[j] where the block from rank i lands
 * counts/displacements are uint64 in elements, row-major n x n.  If tables_on_device is non-zero the
 * three tables are device pointers (e.g. produced by an on-device router) and no host copy of them is
 * read; the kernel stages them into LDS and derives its tile map with a wavefront prefix sum. */
int hcclx_alltoallv(const void *const *send, void *const *recv, const uint64_t *send_counts,
                    const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, int dtype,
                    int tables_on_device, void *stream);

/* The same AlltoAllV with host tables as a plan: the tables are read once and turned into a block list in device
 * memory; hcclx_plan_launch then moves the data with no table travelling at launch time (a repeated exchange,
 * or one that is captured into a HIP graph).  Launched, measured and destroyed like any other plan. */
int hcclx_alltoallv_plan_create(const void *const *send, void *const *recv, const uint64_t *send_counts,
                                const uint64_t *sdispls, const uint64_t *rdispls, uint32_t n, int dtype, hcclx_plan_t **plan);

/* AllGatherV among n virtual ranks: recv[j][displs[i] .. displs[i]+counts[i]) = send[i][0 .. counts[i])
 * for every i and j; each source element is read once and written n times.  counts/displs as above. */
int hcclx_allgatherv(const void *const *send, void *const *recv, const uint64_t *counts,
                     const uint64_t *displs, uint32_t n, int dtype, int tables_on_device, void *stream);

/* Displacements that pack ragged blocks back to back, computed on the device by a wavefront prefix sum:
 * displs[r*n + i] = counts[r*n + 0] + ... + counts[r*n + i-1] for each of `rows` rows of n <= 64 counts, and, if
 * totals is not null, totals[r] = the row's sum.  All three are device arrays of uint64.  One row gives the recvDispls
 * of an AllGatherV whose counts were produced on the device (then hcclx_allgatherv with tables_on_device = 1); the
 * n rows of an AlltoAllV's send counts give its sdispls.  No counterpart in the reference, whose callers pass
 * finished displacement arrays (include/hccl.h:134-135). */
int hcclx_displs_from_counts(const uint64_t *counts, uint32_t rows, uint32_t n, uint64_t *displs, uint64_t *totals,
                             void *stream);

/* ---- The caller side of an MoE AlltoAllV, for n virtual ranks at once -------------------------------------
 * No counterpart in the reference, whose AlltoAllV takes finished send buffers and tables; the nearest code is
 * the staging either side of the transfer (PreCopy / PostCopy,
 * src/ops/all_to_all_v/template/aicpu/ins_temp_all_to_all_v_mesh_1D.cc:412-440).
 *
 * Every rank i holds `tokens` rows and `entries = tokens * topk` routing entries; entry e belongs to token
 * e / topk and goes to rank dest[i][e].  Rows are grouped by destination rank, and inside a group they keep
 * their entry order (a stable grouping).  An entry whose destination is outside 0 .. n-1 is dropped: it is
 * not sent, perm marks it 0xFFFFFFFF, and it adds nothing when results are combined.
 * All pointer arrays are host arrays of n device pointers; all tables are device arrays. */

/* Bytes of device workspace hcclx_moe_route needs. */
uint64_t hcclx_moe_workspace_bytes(uint32_t n, uint32_t entries);

/* From dest[i] (device int32[entries]) to the tables of the AlltoAllV that follows, all n x n row-major
 * uint64 in elements (row_elems per row), laid out as hcclx_alltoallv reads them with tables_on_device = 1:
 *   send_counts[i*n + j], sdispls[i*n + j]   what rank i sends to rank j and where it starts in i's packed buffer
 *   rdispls[j*n + i]                         where that block lands in rank j's receive buffer (blocks in rank order)
 *   recv_counts[j*n + i] = send_counts[i*n + j]   (the send counts of the way back)
 * and perm[i] (device uint32[entries]): the row of rank i's packed buffer that entry e goes to.
 * The AlltoAllV of the way back uses (recv_counts, rdispls, sdispls) in the places of
 * (send_counts, sdispls, rdispls). */
int hcclx_moe_route(const int32_t *const *dest, uint32_t n, uint32_t entries, uint64_t row_elems, uint64_t *send_counts,
                    uint64_t *sdispls, uint64_t *recv_counts, uint64_t *rdispls, uint32_t *const *perm, void *workspace,
                    void *stream);

/* packed[i][perm[i][e]] = tokens[i][e / topk]: rows of row_bytes bytes (a multiple of 16; buffers 16-byte
 * aligned). */
int hcclx_moe_pack(const void *const *tokens, const uint32_t *const *perm, uint32_t n, uint32_t entries, uint32_t topk,
                   uint64_t row_bytes, void *const *packed, void *stream);

/* out[i][t] = sum over j < topk of packed[i][perm[i][t*topk + j]], j ascending, dropped entries skipped (all
 * dropped: zeros).  topk == 1 is a pure row permute for any dtype.  topk > 1 takes fp32, fp16 or bf16; 16-bit
 * floats are accumulated in fp32 and narrowed once (round to nearest even). */
int hcclx_moe_combine(const void *const *packed, const uint32_t *const *perm, uint32_t n, uint32_t tokens, uint32_t topk,
                      uint64_t row_elems, int dtype, void *const *out, void *stream);

/* hcclx_moe_pack followed by hcclx_alltoallv(packed, recv, send_counts, sdispls, rdispls), in one pass and without
 * the packed buffers: the row of entry e of rank i goes to
 *   recv[j] + (rdispls[j*n + i] + perm[i][e] * row_elems - sdispls[i*n + j]) elements,  j = dest[i][e].
 * sdispls / rdispls: the device tables hcclx_moe_route wrote.  Rows of row_elems elements of `dtype` (a multiple
 * of 16 bytes; buffers 16-byte aligned). */
int hcclx_moe_dispatch(const void *const *tokens, const int32_t *const *dest, const uint32_t *const *perm, uint32_t n,
                       uint32_t entries, uint32_t topk, uint64_t row_elems, int dtype, const uint64_t *sdispls,
                       const uint64_t *rdispls, void *const *recv, void *stream);

/* The way back: hcclx_alltoallv(expert, back, recv_counts, rdispls, sdispls) followed by hcclx_moe_combine, in one
 * pass and without the `back` buffers.  expert[j] holds one row per row of recv[j], in the same places;
 * out[i][t] = sum over k < topk of the row of entry t*topk + k (k ascending, dropped entries skipped, all dropped:
 * zeros).  Types as for hcclx_moe_combine. */
int hcclx_moe_gather_combine(const void *const *expert, const int32_t *const *dest, const uint32_t *const *perm, uint32_t n,
                             uint32_t tokens, uint32_t topk, uint64_t row_elems, int dtype, const uint64_t *sdispls,
                             const uint64_t *rdispls, void *const *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCLX_H_ */
