// From recorded steps to GPU launches.
//
// RunCollective is called once all ranks of a world have queued the same collective.  It selects the
// algorithm, runs every rank's executor + template against the recording backend, orders the recorded
// steps by their notify dependencies (the reference's system-test harness builds the same graph from the
// same records: test/st/algorithm/utils/src/hccl_verifier/task_graph_generator/), and then either
//   * STEP mode: launches the copies and reduces level by level -- every step of the template runs as the
//     reference's engines would run it, through the scratch buffers; or
//   * FUSED mode: executes the schedule symbolically (which input bytes, combined in which order, reach
//     each output byte -- the analysis of task_check_op_semantics.cc:477-657, kept as expression trees
//     instead of source sets), and launches one fold per distinct expression: every input read once,
//     every output written once, no scratch traffic, same association order.
#pragma once
#include <string>
#include <vector>

#include "vcomm.h"

namespace ops_hccl {

HcclResult RunCollective(World *w, std::vector<OpParam> &params);

// Forces the algorithm of an op type for a world ("" = let the selector choose).
void SetForcedAlgorithm(World *w, HcclCMDType type, const std::string &algName);
std::string GetForcedAlgorithm(World *w, HcclCMDType type);

// Topology the selectors see; default: one level, 1-D mesh.
struct TopoInfoWithNetLayerDetails;
void SetWorldTopo(World *w, u32 levels, Level0Shape shape, u32 devicesPerServer);
// What the channels handed to the templates report as their link; PCIe puts the templates that have one into read mode.
void SetWorldLinkProtocol(World *w, CommProtocol protocol);

}  // namespace ops_hccl
