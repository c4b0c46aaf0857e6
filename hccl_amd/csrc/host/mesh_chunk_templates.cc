// The large-message "mesh chunk" templates, restated from the reference:
//   InsTempReduceScatterMesh1DMeshChunk      src/ops/reduce_scatter/template/aicpu/
//                                            ins_temp_reduce_scatter_mesh_1D_meshchunk.cc:69-227
//   InsTempAllReduceMesh1DTwoShotMeshChunk   src/ops/all_reduce/template/aicpu/
//                                            ins_temp_all_reduce_mesh_1D_two_shot_mesh_chunk.cc:49-311
//
// A rank's shard is cut into N-1 chunks and reduced in place in the owner's scratch buffer: in step s
// every rank reduce-writes one chunk to every peer, chunk i going to the peer N_(s,i) places below it, so
// that in one step the N-1 chunks of a shard are written by N-1 different peers, and over the N-1 steps
// chunk i takes the peers in the rotation  owner + i + 1, owner + i + 2, ...  (the owner's own data first).
// No scratch slot per rank is needed, which is why the reference moves to these templates for large
// messages.
#include "data_move_templates.h"

namespace ops_hccl {

namespace {

// Distance to the peer that chunk i goes to in step s: s + i + 1, skipping the multiples of n.
u32 ChunkDistance(u32 step, u32 chunk, u32 n)
{
    u32 d = step + chunk + 1;
    if (d >= n) d += 1;
    return d % n;
}

// The per-step barrier between a rank's threads (notify indices of the reference: main -> sub 1,
// sub -> main idx + (threads - 1)).
HcclResult StepBarrier(const std::vector<ThreadHandle> &threads)
{
    if (threads.size() <= 1) return HCCL_SUCCESS;
    std::vector<ThreadHandle> subs(threads.begin() + 1, threads.end());
    const u32 m = static_cast<u32>(subs.size());
    std::vector<u32> up, down(m, 1);
    for (u32 i = 0; i < m; ++i) up.push_back(i + m);
    CHK_RET(PostSyncInterThreads(threads[0], subs, up));
    return PreSyncInterThreads(threads[0], subs, down);
}

// count elements in `parts` chunks, the first count % parts one element longer.
std::vector<u64> SplitEven(u64 count, u64 parts, u64 esz)
{
    std::vector<u64> sizes;
    for (u64 i = 0; i < parts; ++i) sizes.push_back((count / parts + (i < count % parts ? 1 : 0)) * esz);
    return sizes;
}

// A ReduceScatter shard of `size` bytes in N-1 chunks: all but the last rounded down to 4 KiB, the last takes the
// rest; shards too small for that are cut evenly by elements (mesh_1D_meshchunk.cc:139-162).
std::vector<u64> ShardChunks(u64 size, u32 n, u64 esz)
{
    const u64 parts = n - 1;
    const u64 aligned = (size / parts) / AICPU_ALIGN_SIZE * AICPU_ALIGN_SIZE;
    if (parts >= 2 && aligned > 0) {
        std::vector<u64> chunk(parts - 1, aligned);
        chunk.push_back(size - aligned * (parts - 1));
        return chunk;
    }
    return SplitEven(size / esz, parts, esz);
}

// The ranks whose data chunk `chunk` of `owner`'s shard takes, in the order it takes them: the owner's own first,
// then the writer of step 0, 1, ... N-2.
void ChunkOrder(u32 owner, u32 chunk, u32 n, std::vector<u32> &ranks)
{
    ranks.assign(1, owner);
    for (u32 step = 0; step + 1 < n; ++step) ranks.push_back((owner + ChunkDistance(step, chunk, n)) % n);
}

}  // namespace

HcclResult InsTempReduceScatterMesh1DMeshChunk::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                          TemplateResource &res)
{
    const u32 n = templateRankSize_;
    CHK_PRT_RET(n == 0, HCCL_ERROR("[RS mesh chunk] rank size is 0"), HCCL_E_INTERNAL);
    threadNum_ = static_cast<u32>(GetThreadNum());
    CHK_PRT_RET(res.threads.size() < threadNum_, HCCL_ERROR("[RS mesh chunk] thread num is invalid"), HCCL_E_INTERNAL);
    std::vector<ThreadHandle> threads(res.threads.begin(), res.threads.begin() + threadNum_);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    const u64 size = p.sliceSize;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    void *in = p.buffInfo.inputPtr;
    void *ccl = p.buffInfo.hcclBuff.addr;

    // own shard into the scratch buffer: everything else is reduced onto it there
    for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
        CHK_RET(LocalCopy(threads[0],
                          DataSlice(in, p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride + me * p.inputSliceStride, size),
                          DataSlice(ccl, p.buffInfo.hcclBuffBaseOff, size)));
    }
    CHK_RET(PreSync(threads));

    if (n > 1) {
        const std::vector<u64> chunk = ShardChunks(size, n, esz);
        for (u32 step = 0; step + 1 < n; ++step) {
            u64 off = 0;
            for (u32 i = 0; i + 1 < n; ++i) {
                const u32 peer = (me + n - ChunkDistance(step, i, n)) % n;       // whose shard this chunk belongs to
                const u32 from = (me + ChunkDistance(step, i, n)) % n;           // who writes chunk i of my shard now
                const ChannelInfo &link = res.channels.at(subCommRanks_[0][peer])[0];
                const ThreadHandle th = threads[peer < me ? peer : peer - 1];
                std::vector<DataSlice> txSrc, txDst, rxSrc, rxDst;
                for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
                    const u64 inOff = p.buffInfo.inBuffBaseOff + rpt * p.inputRepeatStride;
                    txSrc.emplace_back(in, inOff + peer * p.inputSliceStride + off, chunk[i], chunk[i] / esz);
                    txDst.emplace_back(link.remoteCclMem.addr, p.buffInfo.hcclBuffBaseOff + off, chunk[i], chunk[i] / esz);
                    // what arrives here in this step (descriptive: the peer writes, this side only waits)
                    rxSrc.emplace_back(res.channels.at(subCommRanks_[0][from])[0].remoteCclMem.addr,
                                       inOff + me * p.inputSliceStride + off, chunk[i], chunk[i] / esz);
                    rxDst.emplace_back(ccl, p.buffInfo.hcclBuffBaseOff + off, chunk[i], chunk[i] / esz);
                }
                SendRecvReduceInfo info{{link, link}, {{txSrc, txDst}, {rxSrc, rxDst}}, dataType_, reduceOp_};
                CHK_RET(SendRecvBatchWriteReduce(info, th));
                off += chunk[i];
            }
            if (step + 2 < n) CHK_RET(StepBarrier(threads));
        }
    }
    CHK_RET(PostSync(threads));

    for (u64 rpt = 0; rpt < p.repeatNum; ++rpt) {
        CHK_RET(LocalCopy(threads[0], DataSlice(ccl, p.buffInfo.hcclBuffBaseOff, size),
                          DataSlice(p.buffInfo.outputPtr, p.buffInfo.outBuffBaseOff, size)));
    }
    return HCCL_SUCCESS;
}

// What the steps above amount to: chunk i of rank r's shard is r's own data with the peers' reduced onto it in the
// rotation of ChunkOrder, and lands in r's output.
bool InsTempReduceScatterMesh1DMeshChunk::ClosedForm(const TemplateDataParams &p, u64 esz, std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n == 0 || p.repeatNum != 1) return false;
    const u64 size = p.sliceSize;
    if (size == 0) return true;
    std::vector<u64> chunk(1, size);
    if (n > 1) chunk = ShardChunks(size, n, esz);
    std::vector<u32> order;
    for (u32 r = 0; r < n; ++r) {
        u64 off = 0;
        for (u32 i = 0; i < chunk.size(); ++i) {
            if (chunk[i] != 0) {
                ClosedFold f;
                f.bytes = chunk[i];
                ChunkOrder(r, i, n, order);
                for (u32 from : order) f.src.push_back({from, p.buffInfo.inBuffBaseOff + r * p.inputSliceStride + off});
                f.dst.push_back({r, p.buffInfo.outBuffBaseOff + off});
                out.push_back(std::move(f));
            }
            off += chunk[i];
        }
    }
    return true;
}

HcclResult InsTempAllReduceMesh1DTwoShotMeshChunk::KernelRun(const OpParam &param, const TemplateDataParams &p,
                                                             TemplateResource &res)
{
    const u32 n = templateRankSize_;
    threadNum_ = static_cast<u32>(res.threads.size());
    CHK_PRT_RET(threadNum_ != n, HCCL_ERROR("[AR mesh chunk] thread num is invalid"), HCCL_E_INTERNAL);
    dataType_ = param.DataDes.dataType;
    const u64 esz = DATATYPE_SIZE_TABLE[dataType_];
    if (p.count == 0) return HCCL_SUCCESS;
    u32 me = 0;
    CHK_RET(GetAlgRank(myRank_, subCommRanks_[0], me));
    void *in = p.buffInfo.inputPtr;
    void *out = p.buffInfo.outputPtr;
    void *ccl = p.buffInfo.hcclBuff.addr;
    const u64 inBase = p.buffInfo.inBuffBaseOff;
    const u64 outBase = p.buffInfo.outBuffBaseOff;
    const u64 cclBase = p.buffInfo.hcclBuffBaseOff;

    // first level: ceil(count / N) elements per rank, the tail short or empty (mesh_chunk.cc:49-70);
    // second level: every rank's slice in N-1 chunks, the first (count % (N-1)) one element longer (:126-142)
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    std::vector<std::vector<u64>> chunk(n);
    for (u32 r = 0; r < n && n > 1; ++r) chunk[r] = SplitEven(sl[r].size / esz, n - 1, esz);

    if (sl[me].size != 0) {
        CHK_RET(LocalCopy(res.threads[0], DataSlice(in, inBase + sl[me].offset, sl[me].size, sl[me].count),
                          DataSlice(ccl, cclBase + sl[me].offset, sl[me].size, sl[me].count)));
    }

    // --- reduce-scatter in the owners' scratch buffers
    CHK_RET(PreSync(res.threads));
    for (u32 step = 0; step + 1 < n; ++step) {
        for (u32 c = 0; c + 1 < n; ++c) {
            const u32 peer = (me + n - ChunkDistance(step, c, n)) % n;
            const u32 from = (me + ChunkDistance(step, c, n)) % n;
            u64 txOff = 0;
            u64 rxOff = 0;
            for (u32 m = 0; m < c; ++m) {
                txOff += chunk[peer][m];
                rxOff += chunk[me][m];
            }
            const ChannelInfo &link = res.channels.at(subCommRanks_[0][peer])[0];
            const u64 txSize = chunk[peer][c];
            const u64 rxSize = chunk[me][c];
            DataSlice txSrc(in, inBase + sl[peer].offset + txOff, txSize, txSize / esz);
            DataSlice txDst(link.remoteCclMem.addr, cclBase + sl[peer].offset + txOff, txSize, txSize / esz);
            DataSlice rxSrc(res.channels.at(subCommRanks_[0][from])[0].remoteCclMem.addr, inBase + sl[me].offset + rxOff,
                            rxSize, rxSize / esz);
            DataSlice rxDst(ccl, cclBase + sl[me].offset + rxOff, rxSize, rxSize / esz);
            SendRecvReduceInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_, reduceOp_};
            CHK_RET(SendRecvBatchWriteReduce(info, res.threads[peer < me ? peer : peer - 1]));
        }
        if (step + 2 < n) CHK_RET(StepBarrier(res.threads));
    }
    CHK_RET(PostSync(res.threads));

    // --- all-gather: every rank reads every owner's reduced slice out of that owner's scratch buffer
    if (n > 1) {
        std::vector<ThreadHandle> subs(res.threads.begin() + 1, res.threads.end());
        CHK_RET(PreSyncInterThreads(res.threads[0], subs, std::vector<u32>(subs.size(), 2)));
    }
    for (u32 k = 0; k < n; ++k) {
        if (k == me) {
            if (sl[k].size != 0) {
                CHK_RET(LocalCopy(res.threads[0], DataSlice(ccl, cclBase + sl[k].offset, sl[k].size, sl[k].count),
                                  DataSlice(out, outBase + sl[k].offset, sl[k].size, sl[k].count)));
            }
            continue;
        }
        const ChannelInfo &link = res.channels.at(subCommRanks_[0][k])[0];
        DataSlice rxSrc(link.remoteCclMem.addr, cclBase + sl[k].offset, sl[k].size, sl[k].count);
        DataSlice rxDst(out, outBase + sl[k].offset, sl[k].size, sl[k].count);
        DataSlice txSrc(ccl, cclBase + sl[me].offset, sl[me].size, sl[me].count);
        DataSlice txDst(link.remoteCclMem.addr, outBase + sl[me].offset, sl[me].size, sl[me].count);
        SendRecvInfo info{{link, link}, {{{txSrc}, {txDst}}, {{rxSrc}, {rxDst}}}, dataType_};
        CHK_RET(SendRecvRead(info, res.threads[k < me ? k : k - 1]));
    }
    if (n > 1) {
        std::vector<ThreadHandle> subs(res.threads.begin() + 1, res.threads.end());
        std::vector<u32> up;
        for (u32 i = 0; i < subs.size(); ++i) up.push_back(3 * static_cast<u32>(subs.size()) - i - 1);
        CHK_RET(PostSyncInterThreads(res.threads[0], subs, up));
    }
    return HCCL_SUCCESS;
}

// What the steps above amount to: chunk c of owner k's slice is k's own data with the peers' reduced onto it in the
// rotation of ChunkOrder, and every rank reads it into the same place of its output.
bool InsTempAllReduceMesh1DTwoShotMeshChunk::ClosedForm(const TemplateDataParams &p, u64 esz,
                                                        std::vector<ClosedFold> &out) const
{
    const u32 n = templateRankSize_;
    if (n == 0) return false;
    if (p.count == 0) return true;
    const std::vector<SliceInfo> sl = SplitDataByRank(p.count, n, esz);
    std::vector<u32> order;
    for (u32 k = 0; k < n; ++k) {
        if (sl[k].size == 0) continue;
        std::vector<u64> chunk(1, sl[k].size);
        if (n > 1) chunk = SplitEven(sl[k].size / esz, n - 1, esz);
        u64 off = 0;
        for (u32 c = 0; c < chunk.size(); ++c) {
            if (chunk[c] != 0) {
                ClosedFold f;
                f.bytes = chunk[c];
                ChunkOrder(k, c, n, order);
                for (u32 from : order) f.src.push_back({from, p.buffInfo.inBuffBaseOff + sl[k].offset + off});
                for (u32 r = 0; r < n; ++r) f.dst.push_back({r, p.buffInfo.outBuffBaseOff + sl[k].offset + off});
                out.push_back(std::move(f));
            }
            off += chunk[c];
        }
    }
    return true;
}

}  // namespace ops_hccl
