// HCCL_ALGO: the environment override of the algorithm choice.
//
// Grammar and checks follow the reference's parser (src/common/alg_env_config.cc:330-349, :370-590):
//   one common setting           level0:<algo>;level1:<algo>[;level2:..;level3:..]
//   or one setting per op type   <op>=level0:..;level1:.. / <op>=..   (op: allreduce allgather reducescatter
//                                alltoall broadcast reduce send receive gather scatter sendrecv others)
// Blanks are ignored; the two forms cannot be mixed; a level may appear once; algo is one of
//   null ring pipeline fullmesh H-D_R pairwise NHR NHR_V1 AHC AHC_BROKE NB NA.
// A per-op setting must not put null at level 0; alltoall settings also cover alltoallv / alltoallvc.
//
// The reference's AICPU selectors receive this map and ignore it (all_reduce_auto_selector.cc:354).  Here
// the ranks form one flat level, and the setting picks the template of that level: level1 when it names an
// algorithm, otherwise level0.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "base.h"

namespace ops_hccl {

enum class HcclAlgoType {
    HCCL_ALGO_TYPE_DEFAULT = 0,
    HCCL_ALGO_TYPE_RING,
    HCCL_ALGO_TYPE_PIPELINE,
    HCCL_ALGO_TYPE_FULLMESH,
    HCCL_ALGO_TYPE_HDR,
    HCCL_ALGO_TYPE_PAIRWISE,
    HCCL_ALGO_TYPE_NHR,
    HCCL_ALGO_TYPE_NHR_V1,
    HCCL_ALGO_TYPE_AHC,
    HCCL_ALGO_TYPE_AHC_BROKE,
    HCCL_ALGO_TYPE_NB,
    HCCL_ALGO_TYPE_NULL,
    HCCL_ALGO_TYPE_NA,
};
constexpr u32 HCCL_ALGO_LEVEL_NUM = 4;

using HcclAlgoConfig = std::map<HcclCMDType, std::vector<HcclAlgoType>>;

// Parses a HCCL_ALGO value into per-op level settings (ops that are not mentioned stay absent).
HcclResult SetHcclAlgoConfig(const std::string &hcclAlgo, HcclAlgoConfig &config);

// The executor name the setting asks for on a flat world, "" when it leaves the choice to the selector.
// cpuReduce: 64-bit types and PROD, which take the CPU-reduce variants.
std::string AlgNameFromConfig(const HcclAlgoConfig &config, HcclCMDType type, bool cpuReduce);

// HCCL_DETERMINISTIC: false / true / strict, any case (src/common/alg_env_config.cc:948-990).  strict asks for
// a reduction order that does not depend on which rank computes: the order-preserved ReduceScatter.
enum class DeterministicEnableLevel : u8 { DETERMINISTIC_DISABLE = 0, DETERMINISTIC_ENABLE, DETERMINISTIC_STRICT };
HcclResult ParseDeterministic(const std::string &text, u8 &level);
// Process-wide value, as the selectors read it; set from the environment whenever a world is made.
u8 GetExternalInputHcclDeterministic();
void SetExternalInputHcclDeterministic(u8 level);

// Strict mode applies to floating-point SUM / PROD among more than two ranks (src/common/order_preserved_common.h:63-76).
constexpr u32 MIN_STRICT_RANK_NUM_ORDER_PRESERVED = 2;
constexpr u32 MAX_RANK_NUM_FOR_ORDER_PRESERVED = 32;
bool IsNeedStrictModeForOrderPreserved(HcclDataType dataType, HcclReduceOp reduceType, u32 rankSize);

}  // namespace ops_hccl
