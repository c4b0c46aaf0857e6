/*
 * hccl_comm.h -- communicators of virtual ranks.
 *
 * In the reference the communicator API lives in HCOMM (<hccl/hccl_comm.h>, included at include/hccl.h:15)
 * and one rank is one device.  Here all ranks of a communicator share one GPU; HcclCommInitAll keeps the
 * HCOMM signature (ndev handles at once), the hcclx* functions are additions for what has no counterpart
 * in the reference: the size of the per-rank scratch ("CCL") buffer, how the recorded schedule is run,
 * which algorithm and topology the selector sees, and what the last collective did.
 *
 * Calling convention of the collectives: each rank's call is queued and returns; when the last rank has
 * called, the collective is launched on that rank's stream (streams of the other ranks are joined with
 * events).  With one host thread driving all ranks the calls behave like a group: use the outputs after
 * the last rank's call.  With one host thread per rank set blocking mode, so that a call returns only
 * after the launch and the caller's later work on its stream is ordered after the collective.
 *
 * The first collective of a given kind (op, algorithm, type, count, buffers, mode) records the ranks' templates,
 * plans the launch and keeps the plan (up to 1024 plans or 256 MiB of launch tables per communicator, least
 * recently used out first); repeats only launch kernels -- no allocation, no copy -- and may therefore be issued
 * on a stream that is being captured into a HIP graph.  AllGather(V) and AlltoAll(V, VC) among up to 15 ranks carry
 * their tables in the kernel arguments and can be captured from the first call on; AlltoAll(V, VC) among more ranks
 * uploads a block list at call time and returns HCCL_E_NOT_SUPPORT on a capturing stream (a graph needs
 * hcclx_alltoallv_plan_create of hcclx.h there).
 */
#ifndef HCCL_AMD_HCCL_COMM_H_
#define HCCL_AMD_HCCL_COMM_H_

#include "hccl_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ndev communicator handles, rank i = comms[i], all on the current GPU.  devices may be NULL. */
HcclResult HcclCommInitAll(uint32_t ndev, int32_t *devices, HcclComm *comms);
HcclResult HcclCommDestroy(HcclComm comm);
HcclResult HcclGetRankSize(HcclComm comm, uint32_t *rankSize);
HcclResult HcclGetRankId(HcclComm comm, uint32_t *rank);

/* The same with an explicit scratch-buffer size per rank (bytes, > 1 MiB + 8 KiB; 0 = the default: 200 MiB, or
 * HCCL_BUFFSIZE megabytes).  dry != 0 creates a world without a GPU behind it: collectives record, order
 * and trace their schedule and launch nothing. */
HcclResult hcclxCommInitAll(uint32_t nranks, uint64_t cclBytes, int dry, HcclComm *comms);

typedef enum { HCCLX_EXEC_FUSED = 0, HCCLX_EXEC_STEP = 1 } hcclxExecMode;
/* FUSED (default): one pass per output, inputs read once, the template's fold order kept.
 * STEP: every copy / reduce step of the template is launched, through the scratch buffers. */
HcclResult hcclxCommSetExecMode(HcclComm comm, hcclxExecMode mode);
HcclResult hcclxCommSetBlocking(HcclComm comm, int blocking);

/* HcclCMDType values used by hcclxCommSetAlgorithm. */
typedef enum {
    HCCLX_CMD_ALLREDUCE = 2, HCCLX_CMD_ALLGATHER = 6, HCCLX_CMD_REDUCE_SCATTER = 7, HCCLX_CMD_ALLTOALLV = 8,
    HCCLX_CMD_ALLTOALLVC = 9, HCCLX_CMD_ALLTOALL = 10, HCCLX_CMD_ALLGATHER_V = 16, HCCLX_CMD_REDUCE_SCATTER_V = 17
} hcclxCmdType;
/* Forces the algorithm (executor name, e.g. "InsAllReduceRing") of an op type; NULL or "" = selector. */
HcclResult hcclxCommSetAlgorithm(HcclComm comm, int cmdType, const char *algName);
/* Topology the selectors see: levels (1 = one flat level), shape 0 = CLOS, 1 = 1-D mesh,
 * devicesPerServer (0 = all ranks in one server; 1 = single-device servers, which selects the NHR family). */
HcclResult hcclxCommSetTopo(HcclComm comm, uint32_t levels, int level0Shape, uint32_t devicesPerServer);

/* What the links between the ranks report to the templates.  The NHR templates (AllReduce, ReduceScatter,
 * AllGather, gather-then-fold ReduceScatter) and the AlltoAllV mesh template drive PCIe links in read mode -- the
 * receiver fetches -- and every other link in write mode (src/ops/op_common/template/alg_v2_template_base.cc:91-101;
 * e.g. src/ops/all_reduce/template/aicpu/ins_temp_all_reduce_nhr.cc:105-106, :231-239, :292-300).  Same values either
 * way; the recorded steps, and so the step-by-step launches, differ.  Default: HCCS (write mode); also
 * HCCL_VRANK_LINK_PROTOCOL=pcie|roce when the communicator is made. */
typedef enum { HCCLX_LINK_HCCS = 0, HCCLX_LINK_ROCE = 1, HCCLX_LINK_PCIE = 2 } hcclxLinkProtocol;
HcclResult hcclxCommSetLinkProtocol(HcclComm comm, int protocol);

typedef struct {
    char algName[64];
    uint32_t levels;        /* dependency levels of the recorded schedule */
    uint32_t launches;      /* GPU kernels the collective launched (a fold whose result fans out to many
                               places is two: the fold, then the copy to the other outputs) */
    uint32_t fusedSegments; /* segments of the fused plan */
    int fused;              /* 1 = ran as fused passes, 0 = step by step */
    int planCacheHit;
} hcclxLastOpInfo;
HcclResult hcclxCommGetLastOpInfo(HcclComm comm, hcclxLastOpInfo *info);

/* When tracing is on, every collective also produces the expression of each output piece as text, e.g.
 * "rank 2 out[0,4096) = (x3@0+(x1@0+(x0@0+x2@0)))": "(a+b)" means dst = b, src = a; "xK@B" is byte B of
 * rank K's send buffer.  hcclxCommGetLastTrace copies it (NUL-terminated, truncated to size) and returns
 * the full length. */
HcclResult hcclxCommSetTrace(HcclComm comm, int on);
uint64_t hcclxCommGetLastTrace(HcclComm comm, char *buf, uint64_t size);

/* Closed forms.  Some templates (mesh-chunk, gather-then-fold ReduceScatter, one-shot, two-shot, mesh ReduceScatter)
 * also state what their steps amount to directly; the world then plans from that statement instead of recording, ordering and
 * tracing the steps (nothing is recorded: hcclxLastOpInfo.levels is 0).  mode 0 = never, 1 = for plain launches
 * (the default; also HCCL_VRANK_CLOSED_FORM), 2 = also for traced and dry collectives, so that the trace of the
 * closed form can be compared with the trace of the recorded steps.  Never used while the schedule check is on, in
 * STEP mode, or among buffers that overlap. */
HcclResult hcclxCommSetClosedForm(HcclComm comm, int mode);

/* Schedule check.  When on (also: HCCL_VRANK_CHECK=1), every collective's recorded steps are verified before
 * anything is launched, the way the reference's system-test harness verifies a recorded task list
 * (test/st/algorithm/utils/src/hccl_verifier/): (1) every wait has a record and the handshakes do not deadlock,
 * (2) no two steps that the handshakes leave unordered touch the same bytes with at least one of them writing
 * (check_rank_mem / the task-graph race rules), (3) every output piece is what the collective's contract says:
 * reduced from each rank exactly once at the matching offset, or copied from the right rank and offset
 * (semantics_check/<op>_semantics_checker.cc), (4) when the template also states its result in closed form (see
 * hcclxCommSetClosedForm) and the ranks' buffers lie apart: that statement, piece by piece and in the same
 * association order, is what the recorded steps amount to -- a closed form is trusted when the check is off, so
 * this is where a plug-in template's statement is held against its steps.  A collective that fails returns
 * HCCL_E_INTERNAL and launches nothing.  Checked collectives bypass the plan cache. */
typedef struct {
    uint32_t steps, levels, copies, reduces;
    uint32_t races;
    uint32_t semanticErrors;
    int exhaustive;           /* 1: all pairs of steps were tested for order; 0 (schedules of more than 4096
                                 steps): only steps of the same dependency level */
    char firstProblem[256];
} hcclxCheckReport;
HcclResult hcclxCommSetCheck(HcclComm comm, int on);
HcclResult hcclxCommGetLastCheck(HcclComm comm, hcclxCheckReport *report);

#ifdef __cplusplus
}
#endif
#endif /* HCCL_AMD_HCCL_COMM_H_ */
