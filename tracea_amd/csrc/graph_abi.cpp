// C entry points of include/tracea_graph.h.
#include <exception>

#include "host/dispatch.hpp"
#include "host/graph_fusion.hpp"
#include "tracea_graph.h"

using namespace tracea_amd;

#pragma GCC visibility push(default)
extern "C" char *tracea_graph_fuse(const char *graph_json) {
  try {
    if (graph_json == nullptr) {
      fail(TRACEA_INVALID_PARAMS, "graph JSON is NULL");
      return nullptr;
    }
    Json graph;
    std::string err;
    if (!Json::parse(graph_json, &graph, &err) || !fuse_graph(&graph, &err)) {
      fail(TRACEA_INVALID_PARAMS, "graph: %s", err.c_str());
      return nullptr;
    }
    return dup_cstr(graph.dump());
  } catch (const std::exception &e) {
    fail(TRACEA_UNKNOWN_ERROR, "internal error: %s", e.what());
  } catch (...) {
    fail(TRACEA_UNKNOWN_ERROR, "internal error");
  }
  return nullptr;
}
#pragma GCC visibility pop
