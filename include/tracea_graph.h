/* Graph-level fusion for libtracea.so: turns Conv2d / Linear / Gemm nodes
 * followed by ReLU, BatchNorm or a residual Add into single nodes whose
 * epilogue list names the merged operators in order — the lists that
 * tracea_conv2d_ex / tracea_gemm_ex execute in one launch.
 *
 * Carries GraphOptimizer::optimize of the reference (src/core/optimizer.rs:7-160)
 * over the JSON form of its GraphTopology (src/policy/types.rs:189-192). */
#ifndef TRACEA_GRAPH_H
#define TRACEA_GRAPH_H

#include "tracea.h"

#ifdef __cplusplus
extern "C" {
#endif

/* graph_json: {"operators": [{"<Kind>": {"op_id": n, ...}}, ...],
 *              "dependencies": [[producer_id, consumer_id], ...]}.
 * Merge rules, applied until none fires: the node has exactly one consumer and
 * that consumer is  Relu with 1 producer            -> "ReLU"
 *                   BatchNorm with 5 producers      -> {"BatchNorm": {op_id, gamma_id,
 *                     (x, gamma, beta, mean, var)       beta_id, mean_id, var_id, epsilon}}
 *                   Elementwise kind "Add", 2 prod. -> {"ResidualAdd": {"residual_ptr": id
 *                                                       of the other producer}}
 * Returns the rewritten graph (caller frees with tracea_free_string), or NULL
 * with the reason in tracea_get_last_error. */
char *tracea_graph_fuse(const char *graph_json);

#ifdef __cplusplus
}
#endif
#endif /* TRACEA_GRAPH_H */
