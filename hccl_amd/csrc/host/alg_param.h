// Parameter carriers between op entry, selector, executor and template.
//
// Same names and meaning as the reference (src/ops/op_common/inc/alg_param.h:378-392, :527-609;
// src/ops/op_common/template/template_utils.h:56-81, :90-193, :237-345), reduced to the fields the
// AICPU-engine hot path reads.  Variable-length operands (AlltoAllV / AllGatherV tables) are vectors
// instead of the reference's trailing varData blob; their order in that blob is kept in the field names.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "base.h"

namespace ops_hccl {

struct HcclMem {
    void *addr = nullptr;
    u64 size = 0;
};

// What a link is made of.  The reference takes the enumeration from the transport library; the templates only ask
// one question of it: a PCIe link is driven in read mode (the receiver fetches), every other one in write mode
// (src/ops/op_common/template/alg_v2_template_base.cc:91-101).
enum class CommProtocol : u32 {
    COMM_PROTOCOL_HCCS = 0,
    COMM_PROTOCOL_ROCE = 1,
    COMM_PROTOCOL_PCIE = 2,
    COMM_PROTOCOL_SIO = 3,
    COMM_PROTOCOL_RESERVED = 0xFFFFFFFFu
};

struct ChannelInfo {
    bool isValid = false;
    u32 remoteRank = INVALID_VALUE_RANKID;
    CommProtocol protocol = CommProtocol::COMM_PROTOCOL_RESERVED;
    u32 notifyNum = 0;
    u32 portGroupSize = 1;
    ChannelHandle handle = 0;
    HcclMem remoteCclMem;  // the peer's scratch ("CCL") buffer: same address space, one GPU
};

struct DataSlice {
    void *addr_ = nullptr;
    u64 offset_{0};  // bytes from addr_
    u64 size_{0};    // bytes
    u64 count_{0};   // elements
    DataSlice() = default;
    DataSlice(void *addr, u64 offset, u64 size, u64 count) : addr_(addr), offset_(offset), size_(size), count_(count) {}
    DataSlice(void *addr, u64 offset, u64 size) : addr_(addr), offset_(offset), size_(size), count_(0) {}
};

inline void *GetSliceAddr(const DataSlice &s) { return static_cast<char *>(s.addr_) + s.offset_; }

struct SlicesList {
    std::vector<DataSlice> srcSlices_;
    std::vector<DataSlice> dstSlices_;
    SlicesList(const std::vector<DataSlice> &src, const std::vector<DataSlice> &dst) : srcSlices_(src), dstSlices_(dst) {}
};

struct DataInfo {
    ChannelInfo channel_;
    SlicesList slices_;
    HcclDataType dataType_ = HCCL_DATA_TYPE_RESERVED;
    DataInfo(const ChannelInfo &c, const SlicesList &s) : channel_(c), slices_(s) {}
    DataInfo(const ChannelInfo &c, const SlicesList &s, HcclDataType dt) : channel_(c), slices_(s), dataType_(dt) {}
};

struct DataReduceInfo {
    ChannelInfo channel_;
    SlicesList slices_;
    HcclDataType dataType_;
    HcclReduceOp reduceType_;
    DataReduceInfo(const ChannelInfo &c, const SlicesList &s, HcclDataType dt, HcclReduceOp op)
        : channel_(c), slices_(s), dataType_(dt), reduceType_(op) {}
};

struct TxRxChannels {
    ChannelInfo txChannel_;
    ChannelInfo rxChannel_;
    TxRxChannels(const ChannelInfo &tx, const ChannelInfo &rx) : txChannel_(tx), rxChannel_(rx) {}
};

struct TxRxSlicesList {
    SlicesList txSlicesList_;
    SlicesList rxSlicesList_;
    TxRxSlicesList(const SlicesList &tx, const SlicesList &rx) : txSlicesList_(tx), rxSlicesList_(rx) {}
};

struct SendRecvInfo {
    TxRxChannels sendRecvChannels_;
    TxRxSlicesList sendRecvSlices_;
    HcclDataType dataType_ = HCCL_DATA_TYPE_RESERVED;
    SendRecvInfo(const TxRxChannels &c, const TxRxSlicesList &s) : sendRecvChannels_(c), sendRecvSlices_(s) {}
    SendRecvInfo(const TxRxChannels &c, const TxRxSlicesList &s, HcclDataType dt)
        : sendRecvChannels_(c), sendRecvSlices_(s), dataType_(dt) {}
};

struct SendRecvReduceInfo {
    TxRxChannels sendRecvChannels_;
    TxRxSlicesList sendRecvSlices_;
    HcclDataType dataType_;
    HcclReduceOp reduceType_;
    SendRecvReduceInfo(const TxRxChannels &c, const TxRxSlicesList &s, HcclDataType dt, HcclReduceOp op)
        : sendRecvChannels_(c), sendRecvSlices_(s), dataType_(dt), reduceType_(op) {}
};

struct BuffInfo {
    void *inputPtr = nullptr;
    void *outputPtr = nullptr;
    HcclMem hcclBuff;
    BufferType inBuffType = BufferType::INPUT;
    BufferType outBuffType = BufferType::OUTPUT;
    BufferType hcclBuffType = BufferType::HCCL_BUFFER;
    u64 inputSize = 0;
    u64 outputSize = 0;
    u64 hcclBuffSize = 0;
    u64 inBuffBaseOff = 0;
    u64 outBuffBaseOff = 0;
    u64 hcclBuffBaseOff = 0;
};

struct TemplateDataParams {
    BuffInfo buffInfo;
    u64 count{0};
    u64 sliceSize{0};
    u64 inputSliceStride{0};
    u64 outputSliceStride{0};
    u64 repeatNum{0};
    u64 inputRepeatStride{0};
    u64 outputRepeatStride{0};
    u64 tailSize{0};
    bool enableRemoteMemAccess{false};
    u64 processedDataCount{0};
    HcclDataType dataType{HCCL_DATA_TYPE_INT8};
    std::vector<u64> allRankSliceSize;
    std::vector<u64> allRankDispls;
    std::vector<u64> allRankProcessedDataCount;
    // AlltoAllV per-loop operands
    std::vector<u64> sendCounts;
    std::vector<u64> recvCounts;
    std::vector<u64> sdispls;
    std::vector<u64> rdispls;
};

struct TemplateResource {
    std::map<u32, std::vector<ChannelInfo>> channels;
    std::vector<ThreadHandle> threads;
};

struct TopoInfo {
    u32 userRank = 0;
    u32 userRankSize = 0;
    u32 topoLevelNums = 1;
    Level0Shape level0Shape = Level0Shape::MESH_1D;
};

// What the executor gets from resource set-up (AlgResourceCtxSerializable, alg_param.h:419-512).
struct AlgResourceCtxSerializable {
    TopoInfo topoInfo;
    std::vector<std::vector<u32>> subCommRanks;  // algHierarchyInfo.infos[0]: ranks 0..N-1 in one level
    HcclMem cclMem;
    std::vector<ThreadHandle> threads;
    std::map<u32, std::vector<ChannelInfo>> channels;
};

struct OpParam {
    void *hcclComm = nullptr;
    std::string tag;
    std::string algTag;
    aclrtStream stream = nullptr;
    void *inputPtr = nullptr;
    u64 inputSize = 0;
    void *outputPtr = nullptr;
    u64 outputSize = 0;
    HcclReduceOp reduceType = HCCL_REDUCE_RESERVED;
    u32 root = INVALID_VALUE_RANKID;
    OpMode opMode = OpMode::OPBASE;
    CommEngine engine = CommEngine::COMM_ENGINE_AICPU_TS;
    struct {
        u64 count = 0;
        HcclDataType dataType = HCCL_DATA_TYPE_RESERVED;
        HcclDataType outputType = HCCL_DATA_TYPE_RESERVED;
    } DataDes;
    struct {
        HcclDataType sendType = HCCL_DATA_TYPE_RESERVED;
        HcclDataType recvType = HCCL_DATA_TYPE_RESERVED;
        u64 sendCount = 0;
        u64 recvCount = 0;
    } all2AllDataDes;
    // varData of the V ops.  AllGatherV / ReduceScatterV: [counts, displs] (kernel_launch.cc:766-768);
    // AlltoAllV: [sendCounts, recvCounts, sdispls, rdispls] (kernel_launch.cc:739-748).
    struct {
        std::vector<u64> counts;
        std::vector<u64> displs;
        HcclDataType dataType = HCCL_DATA_TYPE_RESERVED;
    } vDataDes;
    struct {
        HcclDataType sendType = HCCL_DATA_TYPE_RESERVED;
        HcclDataType recvType = HCCL_DATA_TYPE_RESERVED;
        std::vector<u64> sendCounts;
        std::vector<u64> recvCounts;
        std::vector<u64> sdispls;
        std::vector<u64> rdispls;
    } all2AllVDataDes;
    HcclCMDType opType = HcclCMDType::HCCL_CMD_INVALID;
    std::string algName;
};

struct AicpuNHRStepInfo {
    u32 step = 0;
    u32 myRank = 0;
    u32 nSlices = 0;
    u32 toRank = 0;
    u32 fromRank = 0;
    std::vector<u32> txSliceIdxs;
    std::vector<u32> rxSliceIdxs;
};
using NHRStepInfo = AicpuNHRStepInfo;

struct SliceInfo {
    u64 offset = 0;
    u64 size = 0;
    u64 count = 0;
    SliceInfo() = default;
    SliceInfo(u64 o, u64 s, u64 c = 0) : offset(o), size(s), count(c) {}
};

// One piece of a collective's result in closed form: `bytes` bytes that are the fold of the ranks' input pieces
// src[0], src[1], ... (src[0] is what the others are reduced onto, one after the other, each as the source operand
// of its step), delivered to every piece in dst.  A piece is (rank, byte offset in that rank's input -- for src --
// or output -- for dst).  What a template's recorded steps amount to when they are traced, written down directly.
struct ClosedFold {
    struct Ref {
        u32 rank;
        u64 offset;
    };
    std::vector<Ref> src;
    std::vector<Ref> dst;
    u64 bytes = 0;
    // true: the value accumulated so far is the source operand of every step and src[k] the destination operand
    // (a ring: the partial result arrives and is reduced onto the rank's own data)
    bool accIsSource = false;
    // A tree instead of a chain: its inner nodes over src[] as leaves, children before parents, the root last.  A
    // child c < src.size() is leaf c, any other is inner node c - src.size().  Every node is one reduce step,
    // value = value(srcChild) (+) value(dstChild).  Empty: the chain of src.
    struct Step {
        u32 srcChild;
        u32 dstChild;
    };
    std::vector<Step> tree;
};

u32 GetNHRStepNum(u32 rankSize);
HcclResult GetAlgRank(u32 virtRank, const std::vector<u32> &rankIds, u32 &algRank);

}  // namespace ops_hccl
