// The virtual-rank world: N ranks of one communicator whose buffers all live in one GPU's HBM.
//
// It stands where the reference has HCOMM (communicator, threads, channels, transport).  A rank's
// collective call is queued; when every rank of the world has a call at the head of its queue, the
// calls are checked for consistency, each rank's executor + template is run with a recording backend,
// and the recorded steps are launched on the GPU (schedule.h).
#pragma once
#include <condition_variable>
#include <deque>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

#include <hip/hip_runtime.h>

#include "alg_env_config.h"
#include "alg_param.h"

#include "hcclx.h"

struct hcclx_plan;

namespace ops_hccl {

enum class ItemKind : u8 { COPY, REDUCE, NOTIFY_RECORD, NOTIFY_WAIT };

// One primitive call, as recorded on a thread.
struct TaskItem {
    ItemKind kind = ItemKind::COPY;
    u8 dtype = 0;
    u8 op = 0;
    char *dst = nullptr;
    const char *src = nullptr;
    u64 bytes = 0;
    u64 count = 0;
    u64 key = 0;  // notify identity (who signals whom on which index) as a dense number of the world
    u32 seq = 0;  // n-th record / n-th wait on that identity: they pair up in order
};

struct World;

struct VThread {
    World *world = nullptr;
    u32 rank = 0;
    u32 index = 0;
    std::vector<TaskItem> items;
    std::vector<u32> notifySlot;  // by notify index of this thread: identity number + 1, 0 = none yet
};

struct VChannel {
    World *world = nullptr;
    u32 localRank = 0;
    u32 remoteRank = 0;
    std::vector<u32> notifySlot;  // by notify index, for signals from localRank to remoteRank: identity number + 1
};

enum class ExecMode {
    FUSED = 0,  // trace the recorded schedule symbolically and launch one fused pass per output
    STEP = 1,   // launch the recorded copy / reduce steps level by level, as the reference's engines would
};

struct RankComm {
    World *world = nullptr;
    u32 rank = 0;
};

struct QueuedOp {
    OpParam param;
    hipEvent_t ready = nullptr;  // recorded on the caller's stream when it differs from the launch stream
};

struct CachedPlan {
    std::vector<u64> key;
    std::vector<hcclx_plan *> plans;   // launched in this order
    std::vector<void *> buffers;       // device memory the plans use besides their tables (staged outputs)
    bool fused = true;                 // false: the recorded steps, one or two plans per level
    u32 levels = 0;
    u32 segments = 0;                  // segments of the fused plan
    u64 tableBytes = 0;                // device memory of the plans' tables
    void *lastStream = nullptr;        // where it was launched last
    bool manyStreams = false;          // it has been launched on more than one stream
};

// Plans of the collectives a world has run, most recently used first, found through a hash of the key.  What
// falls out at the far end (more than kPlanCacheEntries plans, or more than kPlanCacheBytes of tables) is not
// destroyed at once -- its kernels may still be queued -- but retired behind an event on its stream and freed
// when a later collective finds that event complete.
constexpr size_t kPlanCacheEntries = 1024;
constexpr u64 kPlanCacheBytes = 256ull << 20;
struct RetiredPlan {
    std::vector<hcclx_plan *> plans;
    std::vector<void *> buffers;
    void *event = nullptr;             // hipEvent_t
};
// One launch of a planned collective as the host keeps it: the segment list of one hcclx_plan_create /
// hcclx_fold call.  A shape's list of these is independent of where the ranks' buffers lie, up to a shift of every
// pointer by the distance its buffer has moved.
struct HostPart {
    bool wide = false;
    int dtype = 0;
    int op = 0;
    int mode = 0;
    std::vector<hcclx_seg_t> segs;
    std::vector<hcclx_wide_seg_t> wideSegs;
};
// The plan of a collective without its addresses: found by (op, algorithm, types, counts, tables, which ranks run in
// place), it is moved to the buffers of the call at hand by shifting pointers, with no template run and no trace.
struct ShapePlan {
    std::vector<u64> key;
    std::vector<HostPart> parts;     // launched in this order
    struct Buffer {
        u64 base, size;
    };
    std::vector<Buffer> buffers;     // the ranks' input and output buffers the parts' pointers refer to (2 per rank)
    std::vector<std::vector<uint16_t>> owners;   // per part and pointer: 1 + index of its buffer, 0 = none of them
    bool fused = true;
    u32 levels = 0;
    u32 segments = 0;
    u64 hostBytes = 0;
};
constexpr size_t kShapeCacheEntries = 256;
constexpr u64 kShapeCacheBytes = 128ull << 20;
struct PlanCache {
    std::list<CachedPlan> lru;
    std::unordered_multimap<u64, std::list<CachedPlan>::iterator> index;
    std::vector<RetiredPlan> retired;
    u64 bytes = 0;
    std::list<ShapePlan> shapes;     // most recently used first
    std::unordered_multimap<u64, std::list<ShapePlan>::iterator> shapeIndex;
    u64 shapeBytes = 0;
    std::vector<u64> seenOnce;       // hashes of address keys that were launched from a shape plan once (a ring)
    size_t seenAt = 0;
};

// What the schedule check found in the last collective (see hcclxCommSetCheck).
struct CheckReport {
    u32 steps = 0;           // copy + reduce steps recorded
    u32 levels = 0;
    u32 copies = 0;
    u32 reduces = 0;
    u32 races = 0;           // pairs of unordered steps that touch the same bytes, at least one writing
    u32 semanticErrors = 0;  // output pieces that are not what the collective's contract says
    bool exhaustive = false; // true: every pair of steps was tested for order; false: only steps of one level
    std::string firstProblem;
};

struct World {
    u32 rankSize = 0;
    int device = 0;
    u64 cclBytes = HCCL_CCL_BUFFER_DEFAULT;
    ExecMode mode = ExecMode::FUSED;
    bool blocking = false;  // a rank's call returns only after the collective was launched
    std::vector<std::unique_ptr<RankComm>> ranks;
    std::vector<char *> cclBuf;  // per rank: an address range of its own; device memory once a schedule runs step by step
    bool scratchIsMemory = false;
    std::vector<std::vector<std::unique_ptr<VThread>>> threads;    // [rank][thread]
    std::vector<std::vector<std::unique_ptr<VChannel>>> channels;  // [rank][peer]

    std::mutex mu;
    std::condition_variable cv;
    std::vector<std::deque<QueuedOp>> queue;  // per rank
    std::vector<u64> launched;                // per rank: collectives completed so far
    std::vector<HcclResult> lastResult;

    // recording state of the collective being expanded
    std::vector<u32> recordSeq;   // by notify identity: records / waits made so far
    std::vector<u32> waitSeq;

    // statistics of the last launched collective, for tests and the benchmark
    std::string lastAlgName;
    u32 lastLevels = 0;
    u32 lastLaunches = 0;
    u32 lastFusedSegments = 0;
    bool lastWasFused = false;
    int lastPlanCacheHit = 0;  // 0 planned, 1 a plan with these addresses replayed, 2 a plan of this shape moved to them
    std::string lastTrace;  // expression of every output piece, filled when traceText is set
    bool traceText = false;
    bool check = false;     // verify every schedule before it is launched
    int closedForm = 1;     // templates' closed forms: 0 never used, 1 for plain launches, 2 also when tracing / dry
    CheckReport lastCheck;

    PlanCache planCache;

    // configuration
    std::map<int, std::string> forcedAlg;  // per HcclCMDType; empty = selector decides
    HcclAlgoConfig algoConfig;             // HCCL_ALGO as it was when the world was made
    u32 topoLevels = 1;
    CommProtocol linkProtocol = CommProtocol::COMM_PROTOCOL_HCCS;   // what every channel of the world reports
    Level0Shape topoShape = Level0Shape::MESH_1D;
    u32 devicesPerServer = 0;
    // A dry world has no GPU behind it: scratch buffers are address ranges that are never touched, and a
    // collective stops after its schedule has been recorded, ordered and traced.  Used to check schedules
    // on a machine without a GPU.
    bool dryRun = false;

    ~World();
    HcclResult EnsureScratch(bool memory);
    void ResetRecording();
};

HcclResult WorldCreate(u32 rankSize, u64 cclBytes, bool dryRun, std::vector<HcclComm> &comms);
HcclResult WorldDestroyRank(HcclComm comm);
RankComm *AsRankComm(HcclComm comm);

// Resources a template asks for: `threadNum` threads of this rank and one channel per peer.
void FillResources(World *w, u32 rank, u32 threadNum, AlgResourceCtxSerializable &resCtx);

// Queues one rank's call; launches the collective when all ranks have one queued.
HcclResult SubmitOp(RankComm *rc, const OpParam &param);

}  // namespace ops_hccl
