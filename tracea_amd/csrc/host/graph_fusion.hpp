// Producer/consumer fusion over an operator graph: activation, BatchNorm and
// residual-add nodes that follow a Conv2d / Linear / Gemm node become entries of
// that node's epilogue list, in graph order, until nothing more can be merged.
//
// Rules and JSON shape are the reference's (src/core/optimizer.rs:12-160 over
// GraphTopology / OperatorTopology of src/policy/types.rs:29-95,189-192 in
// serde's externally tagged form):
//   {"operators": [{"Conv2d": {"op_id": 1, ..., "epilogue": []}}, {"Relu": {...}}],
//    "dependencies": [[producer, consumer], ...]}
// epilogue entries: "ReLU", {"BatchNorm": {op_id, gamma_id, beta_id, mean_id,
// var_id, epsilon}}, {"ResidualAdd": {"residual_ptr": <op id of the skip input>}}.
#pragma once
#include <string>

#include "pipeline_config.hpp"

namespace tracea_amd {

// Rewrites `graph` in place.  Returns false and sets *err on a malformed graph.
// Surviving dependencies come out sorted by (producer, consumer).
bool fuse_graph(Json *graph, std::string *err);

}  // namespace tracea_amd
