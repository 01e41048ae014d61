// Tile lists for GEMM over part of the output grid: which tiles run, over which K
// range, and in which order.
//
// Counterpart of the reference's tile task graph: the two-level table a kernel
// reads (src/core/ttg.rs:3-11, 305-340: level 1 maps a workgroup to a record,
// level 2 holds {region_m, region_n, k_start, k_end, role} per record), the
// topology that orders records for operand reuse (src/core/ttg.rs:56-300) and
// the builders of src/runtime/ttg_builder.rs:140-296, 454-464 (dense, dense with
// K split, mask, diagonal, random, low-rank).  Host-only; dispatch.cpp uploads
// the tables and launches the contraction kernel over them.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <string>
#include <vector>

namespace tracea_amd {

struct TileMetadata {  // 20 bytes, the device record
  uint32_t region_m, region_n, k_start, k_end, role;  // role: 0 main, 1 boundary; bit 1 marks a low-rank layout
};
static_assert(sizeof(TileMetadata) == 20, "device record layout");

enum TileEdgeKind : uint32_t { kEdgeDataDep = 0, kEdgeRowAdjacent = 1, kEdgeColAdjacent = 2, kEdgeKPipeline = 3 };
struct TileEdge {
  uint32_t from, to, kind;
};
enum TileReuse : uint32_t { kReuseNone = 0, kReuseA = 1, kReuseB = 2 };
struct TileNode {
  uint32_t tile_id;
  TileMetadata meta;
  uint32_t reuse;         // TileReuse
  uint32_t reuse_source;  // the node whose A rows / B columns this one shares
};

struct TileTopology {
  std::vector<TileNode> nodes;
  std::vector<TileEdge> edges;
  uint32_t grid_m = 0, grid_n = 0, k_splits = 0;

  static TileTopology from_grid(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m, uint32_t n,
                                uint32_t k);
  static TileTopology from_grid_k_split(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m,
                                        uint32_t n, uint32_t k, uint32_t k_splits);
  static TileTopology from_mask(uint32_t grid_m, uint32_t grid_n, uint32_t mt, uint32_t nt, uint32_t m, uint32_t n,
                                uint32_t k, const std::function<bool(uint32_t, uint32_t)> &include);
  // Kahn's algorithm with a last-in-first-out work list; false on a cycle.
  bool topological_sort(std::vector<uint32_t> *order) const;
  std::vector<uint32_t> execution_order() const;
  std::vector<std::pair<uint32_t, uint32_t>> fusion_candidates() const;  // row-adjacent pairs
  bool validate_order(const std::vector<uint32_t> &order) const;

 private:
  void compute_reuse_hints();
};

struct TileLayout {
  uint32_t m = 0, n = 0, k = 0, mt = 0, nt = 0, kt = 0;
  std::vector<uint32_t> l1_map;        // workgroup -> record
  std::vector<TileMetadata> l2_table;  // records
  uint32_t num_active_tiles = 0;
  bool has_topology = false;
  TileTopology topology;

  static bool check_dims(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, std::string *err);
  static TileLayout from_dense(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt);
  static TileLayout from_dense_k_split(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                       uint32_t k_splits);
  static TileLayout from_mask(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                              const std::function<bool(uint32_t, uint32_t)> &include);
  static TileLayout from_diagonal(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt);
  // Every tile kept with probability `density`; the reference draws from an unseeded
  // generator, here the draw is a function of (seed, tile index).
  static TileLayout from_random(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                double density, uint64_t seed);
  static TileLayout from_low_rank(uint32_t m, uint32_t n, uint32_t k, uint32_t r, uint32_t mt, uint32_t nt,
                                  uint32_t kt);
  // Caller-built tables in the device format.
  static bool from_tables(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                          const uint32_t *l1, uint32_t n_l1, const TileMetadata *l2, uint32_t n_l2, TileLayout *out,
                          std::string *err);

  uint32_t grid_m() const { return (m + mt - 1) / mt; }
  uint32_t grid_n() const { return (n + nt - 1) / nt; }
  std::vector<uint32_t> suggest_order() const;
  std::vector<uint32_t> l1_map_ordered() const;
  // Bytes of the level-1 and level-2 tables on the device, each rounded up to 256.
  void device_sizes(size_t *l1_bytes, size_t *l2_bytes) const;
};

}  // namespace tracea_amd
