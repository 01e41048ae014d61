// C entry points of include/tracea_plan.h.
#include <exception>

#include "host/dispatch.hpp"
#include "host/execution_plan.hpp"
#include "tracea_plan.h"

using namespace tracea_amd;

struct TraceaPlan {
  ExecutionPlan plan;
};

#define PLAN_GUARDED(fallback, body)                                   \
  try {                                                                \
    body                                                               \
  } catch (const std::exception &e) {                                  \
    fail(TRACEA_UNKNOWN_ERROR, "internal error: %s", e.what());        \
  } catch (...) {                                                      \
    fail(TRACEA_UNKNOWN_ERROR, "internal error");                      \
  }                                                                    \
  return fallback;

#pragma GCC visibility push(default)
extern "C" {

TraceaPlan *tracea_plan_compile(const char *graph_json, TraceaDType dtype) {
  PLAN_GUARDED(nullptr, {
    if (graph_json == nullptr) {
      fail(TRACEA_INVALID_PARAMS, "graph JSON is NULL");
      return nullptr;
    }
    Json graph;
    std::string err;
    TraceaPlan *p = new TraceaPlan();
    if (!Json::parse(graph_json, &graph, &err) || !p->plan.compile(graph, (int)dtype, &err)) {
      delete p;
      fail(TRACEA_INVALID_PARAMS, "plan: %s", err.c_str());
      return nullptr;
    }
    return p;
  })
}

void tracea_plan_destroy(TraceaPlan *plan) { delete plan; }

size_t tracea_plan_arena_size(const TraceaPlan *plan) { return plan ? plan->plan.arena_size() : 0; }

char *tracea_plan_describe(const TraceaPlan *plan) {
  PLAN_GUARDED(nullptr, {
    if (plan == nullptr) {
      fail(TRACEA_INVALID_PARAMS, "plan is NULL");
      return nullptr;
    }
    return dup_cstr(plan->plan.describe().dump());
  })
}

TraceaStatus tracea_plan_output(const TraceaPlan *plan, uint64_t op_id, size_t *offset, size_t *bytes) {
  PLAN_GUARDED(TRACEA_UNKNOWN_ERROR, {
    if (plan == nullptr || offset == nullptr || bytes == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_output: NULL argument");
    if (!plan->plan.output(op_id, offset, bytes))
      return fail(TRACEA_INVALID_PARAMS, "tracea_plan_output: op %llu has no place in the arena", (unsigned long long)op_id);
    return TRACEA_SUCCESS;
  })
}

TraceaStatus tracea_plan_bind(TraceaPlan *plan, uint64_t op_id, const char *slot, void *device_ptr) {
  PLAN_GUARDED(TRACEA_UNKNOWN_ERROR, {
    if (plan == nullptr || slot == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: NULL argument");
    return plan->plan.bind(op_id, slot, device_ptr);
  })
}

TraceaStatus tracea_plan_bind_sized(TraceaPlan *plan, uint64_t op_id, const char *slot, void *device_ptr,
                                    size_t bytes, int32_t dtype) {
  PLAN_GUARDED(TRACEA_UNKNOWN_ERROR, {
    if (plan == nullptr || slot == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: NULL argument");
    return plan->plan.bind_sized(op_id, slot, device_ptr, bytes, dtype);
  })
}

TraceaStatus tracea_plan_run(const TraceaPlan *plan, void *arena, int32_t device, void *stream) {
  PLAN_GUARDED(TRACEA_UNKNOWN_ERROR, {
    if (plan == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: plan is NULL");
    if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_plan_run: tracea_init has not been called");
    return plan->plan.run(arena, device, stream);
  })
}

}  // extern "C"
#pragma GCC visibility pop
