/* Tile lists for libtracea.so: GEMM over a chosen subset of the output tiles, each
 * over its own K range -- block-sparse, diagonal, masked, windowed or K-split
 * products with the dense kernels.
 *
 * Counterpart of the reference's tile task graph: TTGLayout / TileMetadata /
 * TileTopology (src/core/ttg.rs:3-11, 56-71, 305-340), the builders of TTGBuilder
 * (src/runtime/ttg_builder.rs:140-296, 454-464), the device tables of DeviceTTG
 * (src/runtime/ttg.rs:4-92) and RuntimeManager::launch_ttg
 * (src/runtime/manager/launcher.rs:225-241), which appends the two tables to a
 * kernel's arguments and launches one workgroup per active tile.
 *
 * Device format, as in the reference: a level-1 map of uint32 (workgroup ->
 * record) and a level-2 table of 20-byte records {region_m, region_n, k_start,
 * k_end, role}.  Workgroup p computes rows [region_m*mt, +mt) x columns
 * [region_n*nt, +nt) of C = chain(A[:, k_start:k_end] * B[k_start:k_end, :]);
 * tiles of C that no listed record names are NOT written.  role is carried, not
 * interpreted, by the kernel (0 main, 1 boundary; bit 1 marks a low-rank layout). */
#ifndef TRACEA_TTG_H
#define TRACEA_TTG_H

#include "tracea.h"

#ifdef __cplusplus
extern "C" {
#endif

/* TileMetadata (src/core/ttg.rs:3-11). */
typedef struct TraceaTileMetadata {
  uint32_t region_m, region_n, k_start, k_end, role;
} TraceaTileMetadata;

/* TileEdge (src/core/ttg.rs:15-33): kind 0 data dependency, 1 row-adjacent, 2 column-adjacent, 3 K pipeline. */
typedef struct TraceaTileEdge {
  uint32_t from, to, kind;
} TraceaTileEdge;

typedef struct TraceaTtgLayout TraceaTtgLayout;

/* Builders (TTGBuilder::from_dense, from_dense_k_split, from_mask, from_diagonal, from_random,
 * from_low_rank).  m, n, k: the GEMM; mt, nt, kt: tile extents (kt is carried only, as in the
 * reference).  Each returns NULL with the reason in tracea_get_last_error.
 * from_mask: mask[tm * grid_n + tn] != 0 keeps tile (tm, tn), grid_n = ceil(n / nt).
 * from_random: the reference draws from an unseeded generator; here the draw is a function
 * of (seed, tile), so that a layout can be rebuilt. */
TraceaTtgLayout *tracea_ttg_from_dense(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt);
TraceaTtgLayout *tracea_ttg_from_dense_k_split(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt,
                                               uint32_t kt, uint32_t k_splits);
TraceaTtgLayout *tracea_ttg_from_mask(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                      const uint8_t *mask);
TraceaTtgLayout *tracea_ttg_from_diagonal(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt);
TraceaTtgLayout *tracea_ttg_from_random(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                        double density, uint64_t seed);
TraceaTtgLayout *tracea_ttg_from_low_rank(uint32_t m, uint32_t n, uint32_t k, uint32_t r, uint32_t mt, uint32_t nt,
                                          uint32_t kt);
/* Tables built by the caller, in the device format (windowed K ranges, any subset, any order). */
TraceaTtgLayout *tracea_ttg_from_tables(uint32_t m, uint32_t n, uint32_t k, uint32_t mt, uint32_t nt, uint32_t kt,
                                        const uint32_t *l1_map, uint32_t n_l1, const TraceaTileMetadata *l2_table,
                                        uint32_t n_l2);
/* Frees the layout and the device tables the library allocated for it (not caller memory given to
 * tracea_ttg_upload_to).  Launches that use the layout must have completed. */
void tracea_ttg_destroy(TraceaTtgLayout *layout);

/* TTGLayout::num_active_tiles, and the sizes of its tables and of its topology (0 edges: none). */
uint32_t tracea_ttg_num_active_tiles(const TraceaTtgLayout *layout);
uint32_t tracea_ttg_num_records(const TraceaTtgLayout *layout);
uint32_t tracea_ttg_num_edges(const TraceaTtgLayout *layout);
/* Copies of the host tables; each returns the number of entries the layout holds and writes
 * min(that, cap) of them (out may be NULL with cap 0).
 * l1_map: TTGLayout::l1_map; l1_map_ordered: TTGLayout::l1_map_ordered (ttg.rs:322-335), the order
 * workgroups are given; execution_order: TTGLayout::suggest_order; reuse: per topology node,
 * 0 none / 1 shares A rows / 2 shares B columns with node reuse_source[i]. */
uint32_t tracea_ttg_l1_map(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap);
uint32_t tracea_ttg_l1_map_ordered(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap);
uint32_t tracea_ttg_l2_table(const TraceaTtgLayout *layout, TraceaTileMetadata *out, uint32_t cap);
uint32_t tracea_ttg_execution_order(const TraceaTtgLayout *layout, uint32_t *out, uint32_t cap);
uint32_t tracea_ttg_edges(const TraceaTtgLayout *layout, TraceaTileEdge *out, uint32_t cap);
uint32_t tracea_ttg_reuse_hints(const TraceaTtgLayout *layout, uint32_t *reuse, uint32_t *reuse_source, uint32_t cap);
/* TileTopology::validate_order (ttg.rs:281-291): 1 if no edge of the topology runs backwards in
 * `order`, 1 for a layout without topology. */
int32_t tracea_ttg_validate_order(const TraceaTtgLayout *layout, const uint32_t *order, uint32_t n);

/* DeviceTTG::calculate_size (src/runtime/ttg.rs:15-23): bytes of the two device tables, each
 * rounded up to 256. */
TraceaStatus tracea_ttg_device_size(const TraceaTtgLayout *layout, size_t *l1_bytes, size_t *l2_bytes);
/* DeviceTTG::new_from_arena (ttg.rs:26-61): writes the tables into caller-owned device memory
 * (level 1 in launch order) with synchronous copies and makes later launches on that device read
 * them there; the memory must outlive the layout's launches.  Without this call the first
 * tracea_gemm_ttg on a device allocates and fills the tables itself (DeviceTTG::new). */
TraceaStatus tracea_ttg_upload_to(TraceaTtgLayout *layout, int32_t device_id, void *l1_dst, void *l2_dst);

/* tracea_gemm / tracea_gemm_ex restricted to the layout's records (launch_ttg).  The layout's
 * (mt, nt) must be the macro-tile of a compiled kernel (64x64, 128x64, 128x128, 256x64, 256x128,
 * 256x256), its (m, n, k) the operands' extents; operands are fp16 or bf16 as for the fast path
 * of tracea_gemm; every k_start and k range length must be a multiple of 8, k_start < k_end
 * (k_end is clipped to K).  Records that share a tile (from_dense_k_split) are summed in fp32,
 * provided every tile of the grid has the same number of them; otherwise a shared tile is
 * TRACEA_UNSUPPORTED_CONFIG.  Must not be the first use of a layout on a device while the
 * stream is being captured (the first use copies the tables). */
TraceaStatus tracea_gemm_ttg(TraceaTensorView a, TraceaTensorView b, const TraceaTensorView *bias,
                             const TraceaTensorView *residual, TraceaTensorView *c, TraceaGemmParams params,
                             TraceaTtgLayout *layout);
TraceaStatus tracea_gemm_ttg_ex(TraceaTensorView a, TraceaTensorView b, TraceaTensorView *c, TraceaGemmParams params,
                                const TraceaEpilogueOp *ops, uint32_t n_ops, TraceaTtgLayout *layout);

#ifdef __cplusplus
}
#endif
#endif /* TRACEA_TTG_H */
