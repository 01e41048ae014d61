// C entry points of include/tracea_ttg.h: layout handles, their device tables, and the
// GEMM launch over a tile list.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <exception>
#include <map>
#include <mutex>
#include <numeric>

#include "host/dispatch.hpp"
#include "host/tile_graph.hpp"
#include "tracea_ttg.h"

using namespace tracea_amd;

static_assert(sizeof(TraceaTileMetadata) == sizeof(TileMetadata), "record layout");
static_assert(sizeof(TraceaTileEdge) == sizeof(TileEdge), "edge layout");

namespace {

struct DeviceCopy {
  void *l1 = nullptr, *l2 = nullptr, *slice = nullptr, *counts = nullptr;
  bool owns_tables = false;  // l1 / l2 allocated here (slice and counts always are)
};

// What a launch needs to know about the listed records, found once per layout.
struct LaunchInfo {
  std::vector<uint32_t> physical;  // workgroup -> record: the ordered level-1 map, regrouped per XCD
  std::vector<uint32_t> slice;     // workgroup -> how many earlier records (in table order) share its tile
  std::vector<uint32_t> counts;    // records per tile of the grid; filled when the tiles differ in that
  uint32_t slices = 1, k_gcd = 0, start_gcd = 0;
  std::string error;               // non-empty: the layout cannot be launched, and why
};

}  // namespace

struct TraceaTtgLayout {
  TileLayout layout;
  LaunchInfo info;
  std::mutex mu;
  std::map<int, DeviceCopy> copies;
};

namespace {

// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: XCD x receives
// the x-th contiguous run of the ordered list, so that records that are neighbours in the
// reuse order share an L2.
std::vector<uint32_t> regroup_for_xcds(const std::vector<uint32_t> &ordered) {
  const size_t count = ordered.size();
  std::vector<uint32_t> out(count);
  const size_t q = count / 8, rem = count % 8;
  for (size_t p = 0; p < count; ++p) {
    const size_t x = p % 8, j = p / 8;
    const size_t start = x * q + std::min(x, rem);
    out[p] = ordered[start + j];
  }
  return out;
}

void analyse(TraceaTtgLayout *h) {
  const TileLayout &l = h->layout;
  LaunchInfo &info = h->info;
  info.physical = regroup_for_xcds(l.l1_map_ordered());
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  // occurrence number of every listed record among the listed records of its tile, in table order
  std::vector<uint32_t> listed = l.l1_map;
  std::sort(listed.begin(), listed.end());
  std::vector<uint32_t> occurrence(l.l2_table.size(), 0);
  std::map<uint64_t, uint32_t> seen;
  for (size_t i = 0; i < listed.size(); ++i) {
    if (i > 0 && listed[i] == listed[i - 1]) {
      info.error = "record " + std::to_string(listed[i]) + " is listed twice";
      return;
    }
    const TileMetadata &r = l.l2_table[listed[i]];
    if (r.region_m >= gm || r.region_n >= gn) {
      info.error = "record " + std::to_string(listed[i]) + " names tile (" + std::to_string(r.region_m) + ", " +
                   std::to_string(r.region_n) + ") outside the " + std::to_string(gm) + "x" + std::to_string(gn) + " grid";
      return;
    }
    const uint32_t k_end = std::min(r.k_end, l.k);
    if (r.k_start >= k_end) {
      info.error = "record " + std::to_string(listed[i]) + " has an empty k range [" + std::to_string(r.k_start) + ", " +
                   std::to_string(r.k_end) + ")";
      return;
    }
    info.k_gcd = std::gcd(info.k_gcd, k_end - r.k_start);
    info.start_gcd = std::gcd(info.start_gcd, r.k_start);
    uint32_t &n = seen[(uint64_t)r.region_m * gn + r.region_n];
    occurrence[listed[i]] = n++;
    info.slices = std::max(info.slices, n);
  }
  info.slice.resize(info.physical.size());
  for (size_t p = 0; p < info.physical.size(); ++p) info.slice[p] = occurrence[info.physical[p]];
  // Tiles that share records unevenly (a K range split for some tiles only, or a partial list with
  // shared tiles): the reduction then needs the count of every tile (0: unlisted, left untouched).
  if (info.slices > 1) {
    bool even = seen.size() == (size_t)gm * gn;
    for (const auto &kv : seen) even = even && kv.second == info.slices;
    if (!even) {
      info.counts.assign((size_t)gm * gn, 0u);
      for (const auto &kv : seen) info.counts[kv.first] = kv.second;
    }
  }
}

TraceaTtgLayout *finish(TileLayout &&l) {
  TraceaTtgLayout *h = new TraceaTtgLayout();
  h->layout = std::move(l);
  analyse(h);
  return h;
}

bool dims_ok(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt) {
  std::string err;
  if (TileLayout::check_dims(m, n, k, mt, nt, &err)) return true;
  fail(TRACEA_INVALID_PARAMS, "tile layout: %s", err.c_str());
  return false;
}

template <typename T>
uint32_t copy_out(const std::vector<T> &v, T *out, uint32_t cap) {
  if (out != nullptr) std::copy(v.begin(), v.begin() + std::min<size_t>(v.size(), cap), out);
  return (uint32_t)v.size();
}

TraceaStatus hip_fail(const char *what, hipError_t e) {
  return fail(TRACEA_UNKNOWN_ERROR, "%s: %s", what, hipGetErrorString(e));
}

// The tables of `h` on `device`: the caller's (upload_to) or, on first use, our own.
TraceaStatus device_tables(TraceaTtgLayout *h, int device, void *l1_dst, void *l2_dst, DeviceTileTables *out) {
  if (!h->info.error.empty()) return fail(TRACEA_INVALID_PARAMS, "tile layout: %s", h->info.error.c_str());
  std::lock_guard<std::mutex> lock(h->mu);
  auto it = h->copies.find(device);
  const bool replace = l1_dst != nullptr;
  if (it == h->copies.end() || replace) {
    int prev = 0;
    hipError_t e = hipGetDevice(&prev);
    if (e == hipSuccess) e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail("hipSetDevice", e);
    DeviceCopy copy = it == h->copies.end() ? DeviceCopy{} : it->second;
    const size_t n1 = h->info.physical.size() * 4, n2 = h->layout.l2_table.size() * sizeof(TileMetadata);
    if (replace) {
      if (copy.owns_tables) {
        (void)hipFree(copy.l1);
        (void)hipFree(copy.l2);
      }
      copy.l1 = l1_dst;
      copy.l2 = l2_dst;
      copy.owns_tables = false;
    } else {
      e = hipMalloc(&copy.l1, std::max<size_t>(n1, 4));
      if (e == hipSuccess) e = hipMalloc(&copy.l2, std::max<size_t>(n2, 4));
      copy.owns_tables = true;
    }
    if (e == hipSuccess && n1 > 0) e = hipMemcpy(copy.l1, h->info.physical.data(), n1, hipMemcpyHostToDevice);
    if (e == hipSuccess && n2 > 0) e = hipMemcpy(copy.l2, h->layout.l2_table.data(), n2, hipMemcpyHostToDevice);
    if (e == hipSuccess && h->info.slices > 1 && copy.slice == nullptr) {
      e = hipMalloc(&copy.slice, std::max<size_t>(n1, 4));
      if (e == hipSuccess && n1 > 0) e = hipMemcpy(copy.slice, h->info.slice.data(), n1, hipMemcpyHostToDevice);
    }
    if (e == hipSuccess && !h->info.counts.empty() && copy.counts == nullptr) {
      e = hipMalloc(&copy.counts, h->info.counts.size() * 4);
      if (e == hipSuccess) e = hipMemcpy(copy.counts, h->info.counts.data(), h->info.counts.size() * 4, hipMemcpyHostToDevice);
    }
    (void)hipSetDevice(prev);
    if (e != hipSuccess) {
      if (copy.owns_tables) {
        (void)hipFree(copy.l1);
        (void)hipFree(copy.l2);
      }
      (void)hipFree(copy.slice);
      (void)hipFree(copy.counts);
      h->copies.erase(device);
      return hip_fail("tile tables", e);
    }
    h->copies[device] = copy;
    it = h->copies.find(device);
  }
  if (out != nullptr) {
    out->l1 = (const unsigned *)it->second.l1;
    out->l2 = (const unsigned *)it->second.l2;
    out->slice = (const unsigned *)it->second.slice;
    out->counts = (const unsigned *)it->second.counts;
    out->count = (uint32_t)h->info.physical.size();
    out->slices = h->info.slices;
    out->k_gcd = h->info.k_gcd;
    out->start_gcd = h->info.start_gcd;
  }
  return TRACEA_SUCCESS;
}

TraceaStatus gemm_tiles(const TraceaTensorView &a, const TraceaTensorView &b, const TraceaTensorView *bias,
                        const TraceaTensorView *residual, TraceaTensorView *c, const TraceaGemmParams &params,
                        const TraceaEpilogueOp *ops, uint32_t n_ops, TraceaTtgLayout *h) {
  if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_gemm_ttg: tracea_init has not been called");
  if (h == nullptr || c == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_gemm_ttg: layout or output view is NULL");
  if (c->device_id < 0 || c->device_id >= runtime_device_count())
    return fail(TRACEA_INVALID_PARAMS, "tracea_gemm_ttg: device %d does not exist", c->device_id);
  DeviceTileTables tables;
  if (h->info.physical.empty()) {
    if (!h->info.error.empty()) return fail(TRACEA_INVALID_PARAMS, "tile layout: %s", h->info.error.c_str());
  } else {
    TraceaStatus st = device_tables(h, c->device_id, nullptr, nullptr, &tables);
    if (st != TRACEA_SUCCESS) return st;
  }
  return dispatch_gemm_tiles(a, b, bias, residual, c, params, ops, n_ops, h->layout, tables);
}

}  // namespace

#define TTG_GUARDED(fallback, body)                                    \
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

TraceaTtgLayout *tracea_ttg_from_dense(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    return finish(TileLayout::from_dense(m, n, k, mt, nt, kt));
  })
}

TraceaTtgLayout *tracea_ttg_from_dense_k_split(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt,
                                               uint32_t kt, uint32_t k_splits) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    if (k_splits == 0 || k_splits > k) {
      fail(TRACEA_INVALID_PARAMS, "tile layout: %u K splits of k = %u", k_splits, k);
      return nullptr;
    }
    return finish(TileLayout::from_dense_k_split(m, n, k, mt, nt, kt, k_splits));
  })
}

TraceaTtgLayout *tracea_ttg_from_mask(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                      const uint8_t *mask) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    if (mask == nullptr) {
      fail(TRACEA_INVALID_PARAMS, "tile layout: mask is NULL");
      return nullptr;
    }
    const uint32_t gn = (n + nt - 1) / nt;
    return finish(TileLayout::from_mask(m, n, k, mt, nt, kt,
                                        [&](uint32_t tm, uint32_t tn) { return mask[(size_t)tm * gn + tn] != 0; }));
  })
}

TraceaTtgLayout *tracea_ttg_from_diagonal(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    return finish(TileLayout::from_diagonal(m, n, k, mt, nt, kt));
  })
}

TraceaTtgLayout *tracea_ttg_from_random(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                        double density, uint64_t seed) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    if (!(density >= 0.0 && density <= 1.0)) {
      fail(TRACEA_INVALID_PARAMS, "tile layout: density %g is not a probability", density);
      return nullptr;
    }
    return finish(TileLayout::from_random(m, n, k, mt, nt, kt, density, seed));
  })
}

TraceaTtgLayout *tracea_ttg_from_low_rank(uint32_t m, uint32_t n, uint32_t k, uint32_t r, uint32_t mt, uint32_t nt,
                                          uint32_t kt) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    return finish(TileLayout::from_low_rank(m, n, k, r, mt, nt, kt));
  })
}

TraceaTtgLayout *tracea_ttg_from_tables(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                        const uint32_t *l1_map, uint32_t n_l1, const TraceaTileMetadata *l2_table,
                                        uint32_t n_l2) {
  TTG_GUARDED(nullptr, {
    if (!dims_ok(m, n, k, mt, nt)) return nullptr;
    TileLayout l;
    std::string err;
    if (!TileLayout::from_tables(m, n, k, mt, nt, kt, l1_map, n_l1, (const TileMetadata *)l2_table, n_l2, &l, &err)) {
      fail(TRACEA_INVALID_PARAMS, "tile layout: %s", err.c_str());
      return nullptr;
    }
    return finish(std::move(l));
  })
}

void tracea_ttg_destroy(TraceaTtgLayout *layout) {
  if (layout == nullptr) return;
  for (auto &kv : layout->copies) {
    int prev = 0;
    if (hipGetDevice(&prev) != hipSuccess || hipSetDevice(kv.first) != hipSuccess) continue;
    if (kv.second.owns_tables) {
      (void)hipFree(kv.second.l1);
      (void)hipFree(kv.second.l2);
    }
    (void)hipFree(kv.second.slice);
    (void)hipFree(kv.second.counts);
    (void)hipSetDevice(prev);
  }
  delete layout;
}

uint32_t tracea_ttg_num_active_tiles(const TraceaTtgLayout *layout) {
  return layout ? layout->layout.num_active_tiles : 0;
}
uint32_t tracea_ttg_num_records(const TraceaTtgLayout *layout) {
  return layout ? (uint32_t)layout->layout.l2_table.size() : 0;
}
uint32_t tracea_ttg_num_edges(const TraceaTtgLayout *layout) {
  return layout && layout->layout.has_topology ? (uint32_t)layout->layout.topology.edges.size() : 0;
}

uint32_t tracea_ttg_l1_map(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap) {
  TTG_GUARDED(0, { return layout ? copy_out(layout->layout.l1_map, out, cap) : 0; })
}
uint32_t tracea_ttg_l1_map_ordered(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap) {
  TTG_GUARDED(0, { return layout ? copy_out(layout->layout.l1_map_ordered(), out, cap) : 0; })
}
uint32_t tracea_ttg_l2_table(const TraceaTtgLayout *layout, TraceaTileMetadata *out, uint32_t cap) {
  TTG_GUARDED(0, { return layout ? copy_out(layout->layout.l2_table, (TileMetadata *)out, cap) : 0; })
}
uint32_t tracea_ttg_execution_order(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap) {
  TTG_GUARDED(0, { return layout ? copy_out(layout->layout.suggest_order(), out, cap) : 0; })
}
uint32_t tracea_ttg_edges(const TraceaTtgLayout *layout, TraceaTileEdge *out, uint32_t cap) {
  TTG_GUARDED(0, {
    if (layout == nullptr || !layout->layout.has_topology) return 0;
    return copy_out(layout->layout.topology.edges, (TileEdge *)out, cap);
  })
}
uint32_t tracea_ttg_reuse_hints(const TraceaTtgLayout *layout, uint32_t *reuse, uint32_t *reuse_source, uint32_t cap) {
  TTG_GUARDED(0, {
    if (layout == nullptr || !layout->layout.has_topology) return 0;
    const std::vector<TileNode> &nodes = layout->layout.topology.nodes;
    for (size_t i = 0; i < nodes.size() && i < cap; ++i) {
      if (reuse != nullptr) reuse[i] = nodes[i].reuse;
      if (reuse_source != nullptr) reuse_source[i] = nodes[i].reuse_source;
    }
    return (uint32_t)nodes.size();
  })
}
int32_t tracea_ttg_validate_order(const TraceaTtgLayout *layout, const uint32_t *order, uint32_t n) {
  TTG_GUARDED(0, {
    if (layout == nullptr || (order == nullptr && n > 0)) return 0;
    if (!layout->layout.has_topology) return 1;
    return layout->layout.topology.validate_order(std::vector<uint32_t>(order, order + n)) ? 1 : 0;
  })
}

TraceaStatus tracea_ttg_device_size(const TraceaTtgLayout *layout, size_t *l1_bytes, size_t *l2_bytes) {
  if (layout == nullptr || l1_bytes == nullptr || l2_bytes == nullptr)
    return fail(TRACEA_INVALID_PARAMS, "tracea_ttg_device_size: NULL argument");
  layout->layout.device_sizes(l1_bytes, l2_bytes);
  return TRACEA_SUCCESS;
}

TraceaStatus tracea_ttg_upload_to(TraceaTtgLayout *layout, int32_t device_id, void *l1_dst, void *l2_dst) {
  TTG_GUARDED(TRACEA_UNKNOWN_ERROR, {
    if (!runtime_ready()) return fail(TRACEA_UNKNOWN_ERROR, "tracea_ttg_upload_to: tracea_init has not been called");
    if (layout == nullptr || l1_dst == nullptr || l2_dst == nullptr)
      return fail(TRACEA_INVALID_PARAMS, "tracea_ttg_upload_to: NULL argument");
    if (device_id < 0 || device_id >= runtime_device_count())
      return fail(TRACEA_INVALID_PARAMS, "tracea_ttg_upload_to: device %d does not exist", device_id);
    return device_tables(layout, device_id, l1_dst, l2_dst, nullptr);
  })
}

TraceaStatus tracea_gemm_ttg(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                             const TraceaTensorView *residual, TraceaTensorView *c, TraceaGemmParams params,
                             TraceaTtgLayout *layout) {
  TTG_GUARDED(TRACEA_UNKNOWN_ERROR, { return gemm_tiles(a, b, bias, residual, c, params, nullptr, 0, layout); })
}

TraceaStatus tracea_gemm_ttg_ex(TraceaTensorView a, TraceaTensorView b, TraceaTensorView *c, TraceaGemmParams params,
                                const TraceaEpilogueOp *ops, uint32_t n_ops, TraceaTtgLayout *layout) {
  TTG_GUARDED(TRACEA_UNKNOWN_ERROR, {
    static const TraceaEpilogueOp none{};
    return gemm_tiles(a, b, nullptr, nullptr, c, params, ops != nullptr ? ops : &none, ops != nullptr ? n_ops : 0,
                      layout);
  })
}

}  // extern "C"
#pragma GCC visibility pop
