// ExecutionPlan: a (fused) operator graph compiled into a linear list of launches
// over one arena of device memory.
//
// Counterpart of the reference's plan layer (src/runtime/plan.rs:10-53: steps,
// arena_size, output_map; src/runtime/compiler.rs:100-156: schedule by operator
// id, 256-byte aligned arena offsets).  The reference bump-allocates every
// intermediate and pads the total by 10 %; here an intermediate's bytes are
// returned to a free list after its last consumer has run, so a deep network
// needs the arena of its widest cut, not of its sum.  A plan holds no device
// memory: the caller passes the arena to run(), and run() only launches kernels on
// the given stream (and, where TRACEA_PLAN_SIDE_BY_SIDE=1 was set at compile(), for the
// second of two neighbouring steps that do not depend on each other, on a side stream of
// the plan's own that forks from it and joins it again through events), so the whole plan
// can be captured into a HIP graph and replayed.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "dispatch.hpp"
#include "pipeline_config.hpp"

namespace tracea_amd {

struct PlanTensor {
  uint64_t id = 0;
  bool external = false;   // an Input node: memory comes from bind()
  void *ext = nullptr;
  int dtype = 0;           // TraceaDType
  long long elems = 0;     // 0 for an Input whose size no consumer states
  int channels = 0;        // innermost extent (NHWC channels, GEMM N); 0 if unknown
  size_t offset = 0, bytes = 0;  // place in the arena (256-byte aligned)
  long long need_bytes = 0;      // an Input node: the most bytes any consumer reads from it (0: unknown)
  int need_dtype = -1;           // ... and the element type they read it as (-1: unknown)
  int born = -1, last_use = -1;  // step indices; last_use = steps.size() for graph outputs
};

struct PlanEpilogue {
  int kind = 0;            // TraceaEpilogueOpKind
  float epsilon = 0.0f;
  uint64_t ids[4] = {0, 0, 0, 0};  // tensors of p0..p3
  int n_ids = 0;
};

struct PlanStep {
  std::string kind, name;
  uint64_t id = 0;
  std::vector<uint64_t> inputs;     // data inputs, in dependency order
  std::vector<PlanEpilogue> epilogue;
  long long g[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};  // geometry, meaning per kind (see compile)
  float epsilon = 0.0f;
  const void *weight = nullptr;     // bind(op_id, "weight", ...)
  int weight_layout = 0;            // 0: [K,R,S,C] / [K,N];  1: [R,S,C,K] / [N,K]
  // A Linear step that took over the GlobalAveragePool node in front of it (one launch for both): the pooling
  // node's id (its output is still written), its pixels per image; 0: none.  inputs[0] is then the pooling
  // node's input.
  uint64_t pool_id = 0;
  long long pool_hw = 0;
  // 1: the next step does not depend on this one and runs beside it on the side stream; 2: this step is
  // that second one (the side stream forks in front of the first and joins behind the second)
  int fork = 0;
};

class ExecutionPlan {
 public:
  ExecutionPlan() = default;
  ExecutionPlan(const ExecutionPlan &) = delete;
  ExecutionPlan &operator=(const ExecutionPlan &) = delete;
  ~ExecutionPlan();
  // Builds the plan; false and *err on a malformed or unsupported graph.
  bool compile(const Json &graph, int dtype, std::string *err);
  size_t arena_size() const { return arena_size_; }
  Json describe() const;
  // slot "input": memory of an Input node; "weight" / "weight_rsck" / "weight_t": the filter
  // bank or right operand of a Conv2d / Linear / Gemm node.
  TraceaStatus bind(uint64_t op_id, const std::string &slot, void *ptr);
  // The same with the extent and element type (TraceaDType, or -1) of the memory behind `ptr`: refused
  // when a consumer of the node reads more bytes than that, or reads another type.
  TraceaStatus bind_sized(uint64_t op_id, const std::string &slot, void *ptr, size_t bytes, int dtype);
  TraceaStatus run(void *arena, int device, void *stream) const;
  bool output(uint64_t op_id, size_t *offset, size_t *bytes) const;

 private:
  void *address(uint64_t id, void *arena) const;
  int dtype_ = 0;
  std::vector<PlanStep> steps_;
  std::map<uint64_t, PlanTensor> tensors_;
  size_t arena_size_ = 0;
  // side stream (default priority) and fork/join events, made at compile() for the device current then and
  // again at a run() on another device (outside a stream capture; inside one such a run stays serial)
  bool ensure_side(int device, void *stream) const;
  mutable void *side_stream_ = nullptr, *ev_fork_ = nullptr, *ev_join_ = nullptr;
  mutable int side_device_ = -1;
};

}  // namespace tracea_amd
