#include "tile_graph.hpp"

#include <algorithm>
#include <numeric>

namespace tracea_amd {
namespace {

uint32_t boundary_role(uint32_t tm, uint32_t tn, uint32_t mt, uint32_t nt, uint32_t m, uint32_t n) {
  return ((uint64_t)(tm + 1) * mt > m || (uint64_t)(tn + 1) * nt > n) ? 1u : 0u;
}

uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

}  // namespace

// ---- topology (src/core/ttg.rs:74-300) ---------------------------------------------

TileTopology TileTopology::from_grid(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m,
                                     uint32_t n, uint32_t k) {
  TileTopology t;
  t.grid_m = grid_m;
  t.grid_n = grid_n;
  t.nodes.reserve((size_t)grid_m * grid_n);
  for (uint32_t tm = 0; tm < grid_m; ++tm)
    for (uint32_t tn = 0; tn < grid_n; ++tn) {
      const uint32_t id = tm * grid_n + tn;
      t.nodes.push_back({id, {tm, tn, 0, k, boundary_role(tm, tn, mt, nt, m, n)}, kReuseNone, 0});
      if (tn > 0) t.edges.push_back({id - 1, id, kEdgeRowAdjacent});
      if (tm > 0) t.edges.push_back({id - grid_n, id, kEdgeColAdjacent});
    }
  t.compute_reuse_hints();
  return t;
}

TileTopology TileTopology::from_grid_k_split(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m,
                                             uint32_t n, uint32_t k, uint32_t k_splits) {
  TileTopology t;
  t.grid_m = grid_m;
  t.grid_n = grid_n;
  t.k_splits = k_splits;
  const uint32_t per = k / std::max(k_splits, 1u);
  uint32_t id = 0;
  for (uint32_t tm = 0; tm < grid_m; ++tm)
    for (uint32_t tn = 0; tn < grid_n; ++tn)
      for (uint32_t ks = 0; ks < k_splits; ++ks, ++id) {
        const uint32_t k_end = ks + 1 == k_splits ? k : (ks + 1) * per;
        t.nodes.push_back({id, {tm, tn, ks * per, k_end, boundary_role(tm, tn, mt, nt, m, n)}, kReuseNone, 0});
        // a K stage follows the previous stage of its tile; the first stage of a tile
        // hangs on the first stages of its left and upper neighbours
        if (ks > 0) t.edges.push_back({id - 1, id, kEdgeKPipeline});
        if (tn > 0 && ks == 0) t.edges.push_back({(tm * grid_n + tn - 1) * k_splits, id, kEdgeRowAdjacent});
        if (tm > 0 && ks == 0) t.edges.push_back({((tm - 1) * grid_n + tn) * k_splits, id, kEdgeColAdjacent});
      }
  t.compute_reuse_hints();
  return t;
}

TileTopology TileTopology::from_mask(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m, uint32_t n,
                                     uint32_t k, const std::function<bool(uint32_t, uint32_t)> &include) {
  TileTopology t;
  t.grid_m = grid_m;
  t.grid_n = grid_n;
  const uint32_t none = UINT32_MAX;
  std::vector<uint32_t> id_of((size_t)grid_m * grid_n, none);
  for (uint32_t tm = 0; tm < grid_m; ++tm)
    for (uint32_t tn = 0; tn < grid_n; ++tn) {
      if (!include(tm, tn)) continue;
      const uint32_t id = (uint32_t)t.nodes.size();
      id_of[(size_t)tm * grid_n + tn] = id;
      t.nodes.push_back({id, {tm, tn, 0, k, boundary_role(tm, tn, mt, nt, m, n)}, kReuseNone, 0});
    }
  for (uint32_t tm = 0; tm < grid_m; ++tm)
    for (uint32_t tn = 0; tn < grid_n; ++tn) {
      const uint32_t id = id_of[(size_t)tm * grid_n + tn];
      if (id == none) continue;
      if (tn > 0 && id_of[(size_t)tm * grid_n + tn - 1] != none)
        t.edges.push_back({id_of[(size_t)tm * grid_n + tn - 1], id, kEdgeRowAdjacent});
      if (tm > 0 && id_of[(size_t)(tm - 1) * grid_n + tn] != none)
        t.edges.push_back({id_of[(size_t)(tm - 1) * grid_n + tn], id, kEdgeColAdjacent});
    }
  t.compute_reuse_hints();
  return t;
}

// The reference names the neighbour by its position in the full grid (tm*grid_n + tn -+ 1)
// and accepts it when that number is below the node count, for sparse and K-split node
// lists as well (src/core/ttg.rs:208-237); a row neighbour wins over a column neighbour.
void TileTopology::compute_reuse_hints() {
  const uint32_t count = (uint32_t)nodes.size();
  for (TileNode &node : nodes) {
    const uint32_t tm = node.meta.region_m, tn = node.meta.region_n;
    node.reuse = kReuseNone;
    node.reuse_source = 0;
    if (tn > 0 && tm * grid_n + tn - 1 < count) {
      node.reuse = kReuseA;
      node.reuse_source = tm * grid_n + tn - 1;
    } else if (tm > 0 && (tm - 1) * grid_n + tn < count) {
      node.reuse = kReuseB;
      node.reuse_source = (tm - 1) * grid_n + tn;
    }
  }
}

bool TileTopology::topological_sort(std::vector<uint32_t> *order) const {
  const size_t count = nodes.size();
  std::vector<uint32_t> in_degree(count, 0);
  std::vector<std::vector<uint32_t>> next(count);
  for (const TileEdge &e : edges)
    if (e.from < count && e.to < count) {
      next[e.from].push_back(e.to);
      ++in_degree[e.to];
    }
  std::vector<uint32_t> ready;
  for (uint32_t i = 0; i < count; ++i)
    if (in_degree[i] == 0) ready.push_back(i);
  order->clear();
  order->reserve(count);
  while (!ready.empty()) {
    const uint32_t node = ready.back();
    ready.pop_back();
    order->push_back(node);
    for (uint32_t to : next[node])
      if (--in_degree[to] == 0) ready.push_back(to);
  }
  return order->size() == count;
}

std::vector<uint32_t> TileTopology::execution_order() const {
  std::vector<uint32_t> order(nodes.size());
  std::iota(order.begin(), order.end(), 0u);
  if (k_splits > 0 || nodes.size() < (size_t)grid_m * grid_n) {
    std::vector<uint32_t> sorted;
    if (topological_sort(&sorted)) return sorted;
    return order;
  }
  // dense grid: rows of tiles one after the other (the A rows stay hot)
  std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
    return (a / grid_n) * (grid_n + 1) + a % grid_n < (b / grid_n) * (grid_n + 1) + b % grid_n;
  });
  return order;
}

std::vector<std::pair<uint32_t, uint32_t>> TileTopology::fusion_candidates() const {
  std::vector<std::pair<uint32_t, uint32_t>> out;
  for (const TileEdge &e : edges)
    if (e.kind == kEdgeRowAdjacent) out.push_back({e.from, e.to});
  return out;
}

bool TileTopology::validate_order(const std::vector<uint32_t> &order) const {
  std::vector<int64_t> pos(nodes.size(), -1);
  for (size_t i = 0; i < order.size(); ++i)
    if (order[i] < pos.size()) pos[order[i]] = (int64_t)i;
  for (const TileEdge &e : edges)
    if (e.from < pos.size() && e.to < pos.size() && pos[e.from] >= 0 && pos[e.to] >= 0 && pos[e.from] > pos[e.to])
      return false;
  return true;
}

// ---- layouts (src/runtime/ttg_builder.rs:140-296, 454-464) ---------------------------

bool TileLayout::check_dims(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, std::string *err) {
  if (mt == 0 || nt == 0) {
    *err = "tile extents must be positive";
    return false;
  }
  if (m == 0 || n == 0 || k == 0) {
    *err = "problem extents must be positive";
    return false;
  }
  if ((uint64_t)((m + mt - 1) / mt) * ((n + nt - 1) / nt) > (1u << 26)) {
    *err = "more than 2^26 tiles";
    return false;
  }
  return true;
}

namespace {
TileLayout base(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt) {
  TileLayout l;
  l.m = m; l.n = n; l.k = k; l.mt = mt; l.nt = nt; l.kt = kt;
  return l;
}
}  // namespace

TileLayout TileLayout::from_dense(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  for (uint32_t i = 0; i < gm * gn; ++i) {
    l.l1_map.push_back(i);
    l.l2_table.push_back({i / gn, i % gn, 0, k, boundary_role(i / gn, i % gn, mt, nt, m, n)});
  }
  l.num_active_tiles = gm * gn;
  l.has_topology = true;
  l.topology = TileTopology::from_grid(gm, gn, mt, nt, m, n, k);
  return l;
}

TileLayout TileLayout::from_dense_k_split(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                          uint32_t k_splits) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  const uint32_t per = k / std::max(k_splits, 1u);
  uint32_t id = 0;
  for (uint32_t tm = 0; tm < gm; ++tm)
    for (uint32_t tn = 0; tn < gn; ++tn)
      for (uint32_t ks = 0; ks < k_splits; ++ks, ++id) {
        l.l1_map.push_back(id);
        l.l2_table.push_back({tm, tn, ks * per, ks + 1 == k_splits ? k : (ks + 1) * per,
                              boundary_role(tm, tn, mt, nt, m, n)});
      }
  l.num_active_tiles = id;
  l.has_topology = true;
  l.topology = TileTopology::from_grid_k_split(gm, gn, mt, nt, m, n, k, k_splits);
  return l;
}

TileLayout TileLayout::from_mask(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                 const std::function<bool(uint32_t, uint32_t)> &include) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  for (uint32_t tm = 0; tm < gm; ++tm)
    for (uint32_t tn = 0; tn < gn; ++tn) {
      if (!include(tm, tn)) continue;
      l.l1_map.push_back((uint32_t)l.l2_table.size());
      l.l2_table.push_back({tm, tn, 0, k, 0});  // the reference leaves the role of masked layouts at 0
    }
  l.num_active_tiles = (uint32_t)l.l2_table.size();
  l.has_topology = true;
  l.topology = TileTopology::from_mask(gm, gn, mt, nt, m, n, k, include);
  return l;
}

TileLayout TileLayout::from_diagonal(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  for (uint32_t t = 0; t < std::min(gm, gn); ++t) {
    l.l1_map.push_back((uint32_t)l.l2_table.size());
    l.l2_table.push_back({t, t, 0, k, boundary_role(t, t, mt, nt, m, n)});
  }
  l.num_active_tiles = (uint32_t)l.l2_table.size();
  return l;
}

TileLayout TileLayout::from_random(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                   double density, uint64_t seed) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  const uint32_t gm = l.grid_m(), gn = l.grid_n();
  for (uint32_t tm = 0; tm < gm; ++tm)
    for (uint32_t tn = 0; tn < gn; ++tn) {
      const double u = (double)(splitmix64(seed ^ splitmix64((uint64_t)tm * gn + tn)) >> 11) * (1.0 / 9007199254740992.0);
      if (!(u < density)) continue;
      l.l1_map.push_back((uint32_t)l.l2_table.size());
      l.l2_table.push_back({tm, tn, 0, k, boundary_role(tm, tn, mt, nt, m, n)});
    }
  l.num_active_tiles = (uint32_t)l.l2_table.size();
  return l;
}

TileLayout TileLayout::from_low_rank(uint32_t m, uint32_t n, uint32_t k, uint32_t /*r*/, uint32_t mt, uint32_t nt,
                                     uint32_t kt) {
  TileLayout l = from_dense(m, n, k, mt, nt, kt);
  for (TileMetadata &meta : l.l2_table) meta.role |= 0x2;
  return l;
}

bool TileLayout::from_tables(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                             const uint32_t *l1, uint32_t n_l1, const TileMetadata *l2, uint32_t n_l2, TileLayout *out,
                             std::string *err) {
  TileLayout l = base(m, n, k, mt, nt, kt);
  if ((n_l1 > 0 && l1 == nullptr) || (n_l2 > 0 && l2 == nullptr)) {
    *err = "table pointer is NULL";
    return false;
  }
  for (uint32_t i = 0; i < n_l1; ++i)
    if (l1[i] >= n_l2) {
      *err = "level-1 entry " + std::to_string(i) + " names record " + std::to_string(l1[i]) + " of " +
             std::to_string(n_l2);
      return false;
    }
  l.l1_map.assign(l1, l1 + n_l1);
  l.l2_table.assign(l2, l2 + n_l2);
  l.num_active_tiles = n_l1;
  *out = std::move(l);
  return true;
}

std::vector<uint32_t> TileLayout::suggest_order() const {
  if (has_topology) return topology.execution_order();
  std::vector<uint32_t> order(num_active_tiles);
  std::iota(order.begin(), order.end(), 0u);
  return order;
}

std::vector<uint32_t> TileLayout::l1_map_ordered() const {
  if (!has_topology) return l1_map;
  const std::vector<uint32_t> order = suggest_order();
  std::vector<uint32_t> ordered(num_active_tiles, 0);
  for (size_t pos = 0; pos < order.size() && pos < ordered.size(); ++pos)
    if (order[pos] < l1_map.size()) ordered[pos] = l1_map[order[pos]];
  return ordered;
}

void TileLayout::device_sizes(size_t *l1_bytes, size_t *l2_bytes) const {
  *l1_bytes = (l1_map.size() * 4 + 255) & ~(size_t)255;
  *l2_bytes = (l2_table.size() * sizeof(TileMetadata) + 255) & ~(size_t)255;
}

}  // namespace tracea_amd
