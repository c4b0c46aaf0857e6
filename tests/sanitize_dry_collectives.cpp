// Driver of tests/test_host_sanitize.py: dry worlds (no GPU behind them) through the public C ABI, meant to be built
// with AddressSanitizer and UndefinedBehaviorSanitizer against a host runtime built the same way.  Every AllReduce /
// ReduceScatter template, recorded and in closed form, FUSED and STEP, with the schedule check and the trace on, in
// and out of place; the V collectives and the AlltoAll family with ragged tables; write and read mode.  Prints the
// number of collectives it drove and exits non-zero when one of them failed; a sanitizer report ends the process on
// its own.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "hccl.h"
#include "hccl_comm.h"

namespace {

void *InPtr(uint32_t r) { return reinterpret_cast<void *>(0x100000000000ull + r * 0x001000000000ull); }
void *OutPtr(uint32_t r) { return reinterpret_cast<void *>(0x200000000000ull + r * 0x001000000000ull); }
aclrtStream Stream() { return reinterpret_cast<aclrtStream>(1); }

long g_runs = 0;
long g_failed = 0;

void Note(int rc, const char *what, uint32_t n, const char *alg, uint64_t count)
{
    ++g_runs;
    if (rc != HCCL_SUCCESS) {
        ++g_failed;
        if (g_failed <= 20) std::printf("FAILED rc=%d %s n=%u alg=%s count=%llu\n", rc, what, n, alg, static_cast<unsigned long long>(count));
    }
}

// the trace is read back through a buffer that is deliberately smaller than some traces: truncation must be clean
void ReadTrace(HcclComm comm)
{
    char small[257];
    const uint64_t full = hcclxCommGetLastTrace(comm, small, sizeof(small));
    std::vector<char> all(static_cast<size_t>(full) + 1);
    (void)hcclxCommGetLastTrace(comm, all.data(), all.size());
    hcclxLastOpInfo info;
    (void)hcclxCommGetLastOpInfo(comm, &info);
    hcclxCheckReport rep;
    (void)hcclxCommGetLastCheck(comm, &rep);
}

const char *kAllReduce[] = {"", "InsAllReduceMesh1DOneShot", "InsAllReduceMesh1DTwoShot", "InsAllReduceNHR",
                            "InsAllReduceAicpuReduceNHR", "InsAllReduceMesh1DTwoShotMeshChunk", "InsAllReduceRing",
                            "InsAllReduceRHD"};
const char *kReduceScatter[] = {"", "InsReduceScatterMesh1D", "InsReduceScatterNHR", "InsReduceScatterAicpuReduceNHR",
                                "InsReduceScatterMesh1DMeshChunk", "ReduceScatterOrderPreserved",
                                "ReduceScatterOrderPreservedGroup"};

struct Setting {
    int closedForm;   // 0 recorded, 2 closed form also when traced
    int step;
    int check;
    int link;
};

void Reductions(uint32_t n, const Setting &s, bool inPlace)
{
    std::vector<HcclComm> comm(n);
    if (hcclxCommInitAll(n, 1024 * 1024 + 64 * 1024, 1, comm.data()) != HCCL_SUCCESS) {
        std::printf("FAILED hcclxCommInitAll n=%u\n", n);
        ++g_failed;
        return;
    }
    (void)hcclxCommSetClosedForm(comm[0], s.closedForm);
    (void)hcclxCommSetExecMode(comm[0], s.step ? HCCLX_EXEC_STEP : HCCLX_EXEC_FUSED);
    (void)hcclxCommSetCheck(comm[0], s.check);
    (void)hcclxCommSetTrace(comm[0], 1);
    (void)hcclxCommSetLinkProtocol(comm[0], s.link);
    struct Case {
        uint64_t count;
        HcclDataType dt;
        HcclReduceOp op;
    };
    // short, ragged against every slice rule, and past one scratch slot (several executor loops)
    const Case cases[] = {{1, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_SUM},
                          {n + 3ull, HCCL_DATA_TYPE_INT8, HCCL_REDUCE_MAX},
                          {4099, HCCL_DATA_TYPE_BFP16, HCCL_REDUCE_SUM},
                          {100003, HCCL_DATA_TYPE_FP32, HCCL_REDUCE_PROD},
                          {70001, HCCL_DATA_TYPE_INT64, HCCL_REDUCE_MIN}};
    for (const Case &c : cases) {
        for (const char *alg : kAllReduce) {
            (void)hcclxCommSetAlgorithm(comm[0], HCCLX_CMD_ALLREDUCE, alg);
            int rc = HCCL_SUCCESS;
            for (uint32_t r = 0; r < n; ++r) {
                rc = HcclAllReduce(InPtr(r), inPlace ? InPtr(r) : OutPtr(r), c.count, c.dt, c.op, comm[r], Stream());
            }
            Note(rc, "HcclAllReduce", n, alg, c.count);
            ReadTrace(comm[0]);
        }
        if (inPlace) continue;
        for (const char *alg : kReduceScatter) {
            (void)hcclxCommSetAlgorithm(comm[0], HCCLX_CMD_REDUCE_SCATTER, alg);
            int rc = HCCL_SUCCESS;
            for (uint32_t r = 0; r < n; ++r) rc = HcclReduceScatter(InPtr(r), OutPtr(r), c.count / 4 + 1, c.dt, c.op, comm[r], Stream());
            Note(rc, "HcclReduceScatter", n, alg, c.count / 4 + 1);
            ReadTrace(comm[0]);
        }
    }
    for (uint32_t r = 0; r < n; ++r) (void)HcclCommDestroy(comm[r]);
}

void DataMovement(uint32_t n, const Setting &s)
{
    std::vector<HcclComm> comm(n);
    if (hcclxCommInitAll(n, 1024 * 1024 + 64 * 1024, 1, comm.data()) != HCCL_SUCCESS) {
        ++g_failed;
        return;
    }
    (void)hcclxCommSetExecMode(comm[0], s.step ? HCCLX_EXEC_STEP : HCCLX_EXEC_FUSED);
    (void)hcclxCommSetCheck(comm[0], s.check);
    (void)hcclxCommSetTrace(comm[0], 1);
    (void)hcclxCommSetLinkProtocol(comm[0], s.link);
    // ragged tables with empty blocks and one block larger than a scratch slot
    std::vector<uint64_t> counts(n), displs(n);
    uint64_t at = 2;
    for (uint32_t k = 0; k < n; ++k) {
        counts[k] = (k % 3 == 1) ? 0 : (k == 2 ? 70000 : 100 + 37 * k);
        displs[k] = at;
        at += counts[k] + 1;
    }
    int rc = HCCL_SUCCESS;
    for (uint32_t r = 0; r < n; ++r) {
        rc = HcclReduceScatterV(InPtr(r), counts.data(), displs.data(), OutPtr(r), counts[r], HCCL_DATA_TYPE_INT32, HCCL_REDUCE_MAX,
                                comm[r], Stream());
    }
    Note(rc, "HcclReduceScatterV", n, "", at);
    ReadTrace(comm[0]);
    for (uint32_t r = 0; r < n; ++r) {
        rc = HcclAllGatherV(InPtr(r), counts[r], OutPtr(r), counts.data(), displs.data(), HCCL_DATA_TYPE_FP16, comm[r], Stream());
    }
    Note(rc, "HcclAllGatherV", n, "", at);
    ReadTrace(comm[0]);
    for (const char *alg : {"InsAllGatherMesh1D", "InsAllGatherNHR"}) {
        (void)hcclxCommSetAlgorithm(comm[0], HCCLX_CMD_ALLGATHER, alg);
        for (uint32_t r = 0; r < n; ++r) rc = HcclAllGather(InPtr(r), OutPtr(r), 20001, HCCL_DATA_TYPE_FP16, comm[r], Stream());
        Note(rc, "HcclAllGather", n, alg, 20001);
        ReadTrace(comm[0]);
    }
    // count matrix: row i = what rank i sends
    std::vector<uint64_t> m(static_cast<size_t>(n) * n);
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t j = 0; j < n; ++j) m[i * n + j] = ((3 * i + 5 * j) % 7 == 0) ? 0 : (i == 1 && j == 0 ? 90000 : 10 + (i * 31 + j * 17) % 400);
    }
    for (uint32_t r = 0; r < n; ++r) {
        std::vector<uint64_t> sc(n), sd(n), rcv(n), rd(n);
        uint64_t s0 = 0, r0 = 0;
        for (uint32_t k = 0; k < n; ++k) {
            sc[k] = m[r * n + k];
            rcv[k] = m[k * n + r];
            sd[k] = s0;
            rd[k] = r0;
            s0 += sc[k];
            r0 += rcv[k];
        }
        rc = HcclAlltoAllV(InPtr(r), sc.data(), sd.data(), HCCL_DATA_TYPE_BFP16, OutPtr(r), rcv.data(), rd.data(), HCCL_DATA_TYPE_BFP16,
                           comm[r], Stream());
    }
    Note(rc, "HcclAlltoAllV", n, "", 0);
    ReadTrace(comm[0]);
    for (uint32_t r = 0; r < n; ++r) {
        rc = HcclAlltoAllVC(InPtr(r), m.data(), HCCL_DATA_TYPE_INT8, OutPtr(r), HCCL_DATA_TYPE_INT8, comm[r], Stream());
    }
    Note(rc, "HcclAlltoAllVC", n, "", 0);
    ReadTrace(comm[0]);
    for (uint32_t r = 0; r < n; ++r) rc = HcclAlltoAll(InPtr(r), 333, HCCL_DATA_TYPE_FP32, OutPtr(r), 333, HCCL_DATA_TYPE_FP32, comm[r], Stream());
    Note(rc, "HcclAlltoAll", n, "", 333);
    ReadTrace(comm[0]);
    for (uint32_t r = 0; r < n; ++r) (void)HcclCommDestroy(comm[r]);
}

}  // namespace

int main(int argc, char **argv)
{
    const bool wide = argc > 1 && std::string(argv[1]) == "wide";   // also the communicators of 40 and 64 ranks
    std::vector<uint32_t> sizes = {1, 2, 3, 5, 8, 13};
    if (wide) {
        sizes.push_back(17);
        sizes.push_back(40);
        sizes.push_back(64);
    }
    const Setting settings[] = {{0, 0, 1, HCCLX_LINK_HCCS}, {2, 0, 0, HCCLX_LINK_HCCS}, {0, 1, 0, HCCLX_LINK_HCCS},
                                {0, 0, 1, HCCLX_LINK_PCIE}, {0, 1, 1, HCCLX_LINK_PCIE}};
    for (uint32_t n : sizes) {
        for (const Setting &s : settings) {
            if (n >= 40 && s.check) continue;   // the exhaustive race scan among 64 ranks takes minutes under a sanitizer
            if (n >= 13 && s.link == HCCLX_LINK_PCIE && s.step) continue;
            Reductions(n, s, false);
            if (s.closedForm != 0 || n <= 8) Reductions(n, s, true);
            if (s.closedForm == 0) DataMovement(n, s);
        }
    }
    std::printf("collectives: %ld failed: %ld\n", g_runs, g_failed);
    return g_failed == 0 ? 0 : 1;
}
