#include "alg_env_config.h"

#include <algorithm>
#include <cctype>

namespace ops_hccl {

namespace {

// "a<sep>b<sep>c" -> pieces; an empty piece (leading, trailing or doubled separator) is an error
bool Split(const std::string &s, char sep, std::vector<std::string> &out)
{
    size_t at = 0;
    while (true) {
        const size_t next = s.find(sep, at);
        const std::string piece = s.substr(at, next == std::string::npos ? std::string::npos : next - at);
        if (piece.empty()) return false;
        out.push_back(piece);
        if (next == std::string::npos) return true;
        at = next + 1;
    }
}

HcclResult ParseLevels(const std::string &text, std::vector<HcclAlgoType> &levels)
{
    static const std::map<std::string, u32> levelNames = {{"level0", 0}, {"level1", 1}, {"level2", 2}, {"level3", 3}};
    static const std::map<std::string, HcclAlgoType> algoNames = {
        {"null", HcclAlgoType::HCCL_ALGO_TYPE_NULL},         {"ring", HcclAlgoType::HCCL_ALGO_TYPE_RING},
        {"pipeline", HcclAlgoType::HCCL_ALGO_TYPE_PIPELINE}, {"fullmesh", HcclAlgoType::HCCL_ALGO_TYPE_FULLMESH},
        {"H-D_R", HcclAlgoType::HCCL_ALGO_TYPE_HDR},         {"pairwise", HcclAlgoType::HCCL_ALGO_TYPE_PAIRWISE},
        {"NHR", HcclAlgoType::HCCL_ALGO_TYPE_NHR},           {"NHR_V1", HcclAlgoType::HCCL_ALGO_TYPE_NHR_V1},
        {"AHC", HcclAlgoType::HCCL_ALGO_TYPE_AHC},           {"AHC_BROKE", HcclAlgoType::HCCL_ALGO_TYPE_AHC_BROKE},
        {"NB", HcclAlgoType::HCCL_ALGO_TYPE_NB},             {"NA", HcclAlgoType::HCCL_ALGO_TYPE_NA},
    };
    levels.assign(HCCL_ALGO_LEVEL_NUM, HcclAlgoType::HCCL_ALGO_TYPE_DEFAULT);
    std::vector<std::string> parts;
    CHK_PRT_RET(!Split(text, ';', parts) || parts.size() > HCCL_ALGO_LEVEL_NUM,
                HCCL_ERROR("[HCCL_ALGO] '%s': expected level0:<algo>;level1:<algo>", text.c_str()), HCCL_E_PARA);
    for (const std::string &part : parts) {
        const size_t colon = part.find(':');
        CHK_PRT_RET(colon == std::string::npos || colon == 0 || colon + 1 == part.size(),
                    HCCL_ERROR("[HCCL_ALGO] '%s' is not <level>:<algo>", part.c_str()), HCCL_E_PARA);
        const auto level = levelNames.find(part.substr(0, colon));
        const auto algo = algoNames.find(part.substr(colon + 1));
        CHK_PRT_RET(level == levelNames.end(), HCCL_ERROR("[HCCL_ALGO] unknown level in '%s'", part.c_str()), HCCL_E_PARA);
        CHK_PRT_RET(algo == algoNames.end(), HCCL_ERROR("[HCCL_ALGO] unknown algorithm in '%s'", part.c_str()), HCCL_E_PARA);
        CHK_PRT_RET(levels[level->second] != HcclAlgoType::HCCL_ALGO_TYPE_DEFAULT,
                    HCCL_ERROR("[HCCL_ALGO] %s is set twice", level->first.c_str()), HCCL_E_PARA);
        levels[level->second] = algo->second;
    }
    return HCCL_SUCCESS;
}

const HcclCMDType kAllOps[] = {HcclCMDType::HCCL_CMD_BROADCAST,      HcclCMDType::HCCL_CMD_ALLREDUCE,
                               HcclCMDType::HCCL_CMD_REDUCE,         HcclCMDType::HCCL_CMD_SEND,
                               HcclCMDType::HCCL_CMD_RECEIVE,        HcclCMDType::HCCL_CMD_ALLGATHER,
                               HcclCMDType::HCCL_CMD_REDUCE_SCATTER, HcclCMDType::HCCL_CMD_ALLTOALLV,
                               HcclCMDType::HCCL_CMD_ALLTOALLVC,     HcclCMDType::HCCL_CMD_ALLTOALL,
                               HcclCMDType::HCCL_CMD_GATHER,         HcclCMDType::HCCL_CMD_SCATTER,
                               HcclCMDType::HCCL_CMD_BATCH_SEND_RECV, HcclCMDType::HCCL_CMD_ALLGATHER_V,
                               HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V};

}  // namespace

HcclResult SetHcclAlgoConfig(const std::string &hcclAlgo, HcclAlgoConfig &config)
{
    config.clear();
    std::string text = hcclAlgo;
    text.erase(std::remove(text.begin(), text.end(), ' '), text.end());
    if (text.empty()) return HCCL_SUCCESS;   // built-in selection
    std::vector<std::string> perOp;
    CHK_PRT_RET(!Split(text, '/', perOp), HCCL_ERROR("[HCCL_ALGO] empty setting between '/'"), HCCL_E_PARA);
    size_t specific = 0;
    for (const std::string &one : perOp) {
        const size_t eq = one.find('=');
        CHK_PRT_RET(eq == 0 || eq + 1 == one.size(), HCCL_ERROR("[HCCL_ALGO] '%s' is not <op>=<levels>", one.c_str()),
                    HCCL_E_PARA);
        if (eq != std::string::npos) specific++;
    }
    CHK_PRT_RET(specific != 0 && specific != perOp.size(),
                HCCL_ERROR("[HCCL_ALGO] a common setting and per-op settings cannot be mixed"), HCCL_E_PARA);
    CHK_PRT_RET(specific == 0 && perOp.size() > 1, HCCL_ERROR("[HCCL_ALGO] only one common setting is allowed"),
                HCCL_E_PARA);
    std::vector<HcclAlgoType> levels;
    if (specific == 0) {
        CHK_RET(ParseLevels(perOp[0], levels));
        for (HcclCMDType t : kAllOps) config[t] = levels;
        return HCCL_SUCCESS;
    }
    static const std::map<std::string, HcclCMDType> opNames = {
        {"broadcast", HcclCMDType::HCCL_CMD_BROADCAST}, {"allreduce", HcclCMDType::HCCL_CMD_ALLREDUCE},
        {"reduce", HcclCMDType::HCCL_CMD_REDUCE},       {"send", HcclCMDType::HCCL_CMD_SEND},
        {"receive", HcclCMDType::HCCL_CMD_RECEIVE},     {"allgather", HcclCMDType::HCCL_CMD_ALLGATHER},
        {"reducescatter", HcclCMDType::HCCL_CMD_REDUCE_SCATTER}, {"alltoall", HcclCMDType::HCCL_CMD_ALLTOALL},
        {"gather", HcclCMDType::HCCL_CMD_GATHER},       {"scatter", HcclCMDType::HCCL_CMD_SCATTER},
        {"sendrecv", HcclCMDType::HCCL_CMD_BATCH_SEND_RECV},
    };
    // "others" first: it sets every op, the named ops then override it (alg_env_config.cc:385-396)
    for (const std::string &one : perOp) {
        const size_t eq = one.find('=');
        if (one.substr(0, eq) != "others") continue;
        CHK_RET(ParseLevels(one.substr(eq + 1), levels));
        for (HcclCMDType t : kAllOps) config[t] = levels;
    }
    for (const std::string &one : perOp) {
        const size_t eq = one.find('=');
        const std::string name = one.substr(0, eq);
        if (name == "others") continue;
        const auto op = opNames.find(name);
        CHK_PRT_RET(op == opNames.end(), HCCL_ERROR("[HCCL_ALGO] unknown op type '%s'", name.c_str()), HCCL_E_PARA);
        CHK_RET(ParseLevels(one.substr(eq + 1), levels));
        CHK_PRT_RET(levels[0] == HcclAlgoType::HCCL_ALGO_TYPE_NULL,
                    HCCL_ERROR("[HCCL_ALGO] a per-op setting cannot put null at level0"), HCCL_E_PARA);
        config[op->second] = levels;
    }
    if (config.count(HcclCMDType::HCCL_CMD_ALLTOALL)) {
        config[HcclCMDType::HCCL_CMD_ALLTOALLV] = config[HcclCMDType::HCCL_CMD_ALLTOALL];
        config[HcclCMDType::HCCL_CMD_ALLTOALLVC] = config[HcclCMDType::HCCL_CMD_ALLTOALL];
    }
    // the ragged variants follow their regular op
    if (config.count(HcclCMDType::HCCL_CMD_ALLGATHER) && !config.count(HcclCMDType::HCCL_CMD_ALLGATHER_V)) {
        config[HcclCMDType::HCCL_CMD_ALLGATHER_V] = config[HcclCMDType::HCCL_CMD_ALLGATHER];
    }
    if (config.count(HcclCMDType::HCCL_CMD_REDUCE_SCATTER) && !config.count(HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V)) {
        config[HcclCMDType::HCCL_CMD_REDUCE_SCATTER_V] = config[HcclCMDType::HCCL_CMD_REDUCE_SCATTER];
    }
    return HCCL_SUCCESS;
}

std::string AlgNameFromConfig(const HcclAlgoConfig &config, HcclCMDType type, bool cpuReduce)
{
    const auto it = config.find(type);
    if (it == config.end()) return "";
    auto names = [](HcclAlgoType a) {
        return a != HcclAlgoType::HCCL_ALGO_TYPE_DEFAULT && a != HcclAlgoType::HCCL_ALGO_TYPE_NA &&
               a != HcclAlgoType::HCCL_ALGO_TYPE_NULL;
    };
    const HcclAlgoType algo = names(it->second[1]) ? it->second[1] : it->second[0];
    switch (type) {
        case HcclCMDType::HCCL_CMD_ALLREDUCE:
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_RING) return "InsAllReduceRing";
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_HDR) return "InsAllReduceRHD";
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR || algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR_V1) {
                return cpuReduce ? "InsAllReduceAicpuReduceNHR" : "InsAllReduceNHR";
            }
            return "";   // fullmesh: the selector's one-shot / two-shot / chunked choice by size
        case HcclCMDType::HCCL_CMD_REDUCE_SCATTER:
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR || algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR_V1) {
                return cpuReduce ? "InsReduceScatterAicpuReduceNHR" : "InsReduceScatterNHR";
            }
            return "";
        case HcclCMDType::HCCL_CMD_ALLGATHER:
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR || algo == HcclAlgoType::HCCL_ALGO_TYPE_NHR_V1) return "InsAllGatherNHR";
            if (algo == HcclAlgoType::HCCL_ALGO_TYPE_FULLMESH) return "InsAllGatherMesh1D";
            return "";
        default:
            return "";   // one template each: nothing to choose
    }
}

HcclResult ParseDeterministic(const std::string &text, u8 &level)
{
    std::string t = text;
    std::transform(t.begin(), t.end(), t.begin(), [](unsigned char c) { return static_cast<char>(std::toupper(c)); });
    if (t == "FALSE") {
        level = static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_DISABLE);
    } else if (t == "TRUE") {
        level = static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_ENABLE);
    } else if (t == "STRICT") {
        level = static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_STRICT);
    } else {
        HCCL_ERROR("HCCL_DETERMINISTIC is set to [%s]: should be true, false or strict", text.c_str());
        return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

namespace {
u8 g_deterministic = static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_DISABLE);
}
u8 GetExternalInputHcclDeterministic() { return g_deterministic; }
void SetExternalInputHcclDeterministic(u8 level) { g_deterministic = level; }

bool IsNeedStrictModeForOrderPreserved(HcclDataType dataType, HcclReduceOp reduceType, u32 rankSize)
{
    return GetExternalInputHcclDeterministic() == static_cast<u8>(DeterministicEnableLevel::DETERMINISTIC_STRICT) &&
           (dataType == HCCL_DATA_TYPE_FP16 || dataType == HCCL_DATA_TYPE_FP32 || dataType == HCCL_DATA_TYPE_BFP16 ||
            dataType == HCCL_DATA_TYPE_FP64) &&
           (reduceType == HCCL_REDUCE_SUM || reduceType == HCCL_REDUCE_PROD) &&
           rankSize > MIN_STRICT_RANK_NUM_ORDER_PRESERVED;
}

}  // namespace ops_hccl
