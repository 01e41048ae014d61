/* Execution plans for libtracea.so: a (fused) operator graph compiled into a
 * linear list of launches over one arena of device memory, the way the
 * reference's GraphCompiler turns a GraphTopology into an ExecutionPlan
 * (src/runtime/plan.rs:10-53, src/runtime/compiler.rs:100-156) and its
 * executor walks it.  Graph JSON: see tracea_graph.h; run tracea_graph_fuse
 * first so that ReLU / BatchNorm / residual nodes ride in the epilogues of the
 * contractions.  Nodes that stay on their own (Relu, BatchNorm with its four
 * parameter inputs, Elementwise "Add", GlobalAveragePool, Softmax, Attention)
 * have kernels too.
 *
 * Activations are NHWC tensors of the plan's dtype (f16 or bf16); BatchNorm
 * parameters are f32 vectors; every intermediate lives in the arena at a
 * 256-byte aligned offset and gives its bytes back after its last consumer has
 * run.  A plan owns no device memory, and tracea_plan_run only launches kernels
 * on the given stream: it can be captured into a HIP graph and replayed. */
#ifndef TRACEA_PLAN_H
#define TRACEA_PLAN_H

#include "tracea.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct TraceaPlan TraceaPlan;

/* Returns NULL with the reason in tracea_get_last_error. */
TraceaPlan *tracea_plan_compile(const char *graph_json, TraceaDType dtype);
void tracea_plan_destroy(TraceaPlan *plan);

/* ExecutionPlan::arena_size (plan.rs:14). */
size_t tracea_plan_arena_size(const TraceaPlan *plan);

/* {"arena_size": n, "steps": [{"op_id", "kind", "name", "inputs", "epilogue", "offset", "bytes",
 *  "elements", "last_use"}, ...], "output_map": {"<op_id>": [offset, bytes], ...}} (plan.rs:10-18);
 * free with tracea_free_string. */
char *tracea_plan_describe(const TraceaPlan *plan);

/* ExecutionPlan::output_map lookup. */
TraceaStatus tracea_plan_output(const TraceaPlan *plan, uint64_t op_id, size_t *offset, size_t *bytes);

/* slot "input": device memory of an Input node (KernelArgSpec::ExternalInput, plan.rs:43);
 * "weight": filters [K,R,S,C] of a Conv2d node, right operand [K,N] of a Linear / Gemm node;
 * "weight_rsck" / "weight_t": the same in [R,S,C,K] / [N,K] storage. */
TraceaStatus tracea_plan_bind(TraceaPlan *plan, uint64_t op_id, const char *slot, void *device_ptr);
/* The same for callers that know what lies behind the pointer: `bytes` of memory holding elements of
 * `dtype` (a TraceaDType, or -1 when unknown).  TRACEA_INVALID_PARAMS when a consumer of the Input node
 * reads more bytes than that or reads another element type (data in the plan's type; the parameters of a
 * BatchNorm are float32 channel vectors, given in the order gamma, beta, mean, var after the data input
 * of a BatchNorm node and as gamma_id .. var_id of a fused one), or when a weight bank is shorter than
 * K*R*S*C (Conv2d) or K*N (Linear, Gemm) elements of the plan's type.  (The reference's executor receives
 * sized buffers from its runtime manager, src/runtime/plan.rs:40-53; a raw pointer carries no size.) */
TraceaStatus tracea_plan_bind_sized(TraceaPlan *plan, uint64_t op_id, const char *slot, void *device_ptr,
                                    size_t bytes, int32_t dtype);

/* Launches every step on `stream`.  `arena` holds tracea_plan_arena_size bytes on `device`,
 * 256-byte aligned. */
TraceaStatus tracea_plan_run(const TraceaPlan *plan, void *arena, int32_t device, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TRACEA_PLAN_H */
