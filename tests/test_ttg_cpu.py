"""Tile lists on the host: the reference's own unit tests for its tile task graph
(src/core/ttg.rs:389-461, src/runtime/ttg_builder.rs:467-604) restated on the C ABI,
plus brute-force checks of every builder and of the orders they produce."""
import itertools

import numpy as np
import pytest

from tracea_amd import capi
from tracea_amd.ttg import (EDGE_COL_ADJACENT, EDGE_K_PIPELINE, EDGE_ROW_ADJACENT, REUSE_A, REUSE_B, REUSE_NONE,
                            TILE_DTYPE, TileLayout)


def records(layout):
    return [tuple(int(x) for x in r) for r in layout.l2_table]


def edge_list(layout):
    return [tuple(int(x) for x in e) for e in layout.edges]


# ---- src/core/ttg.rs:389-461 ----

def test_topology_row_adjacency():
    # 3x3 grid: the centre tile touches four edges (ttg.rs:392-397)
    lay = TileLayout.from_dense(96, 96, 128, 32, 32)
    assert lay.num_active_tiles == 9
    assert sum(1 for f, t, _ in edge_list(lay) if f == 4 or t == 4) == 4


def test_topology_execution_order_row_major():
    # ttg.rs:400-403
    lay = TileLayout.from_dense(64, 96, 128, 32, 32)
    assert lay.execution_order().tolist() == [0, 1, 2, 3, 4, 5]
    assert lay.l1_map_ordered.tolist() == [0, 1, 2, 3, 4, 5]


def test_topology_k_split_execution_order():
    # ttg.rs:406-418: 2x2 grid, 2 K stages: 8 nodes, the order respects every edge,
    # and stage 0 of a tile comes before its stage 1
    lay = TileLayout.from_dense_k_split(64, 64, 128, 32, 32, 32, 2)
    order = lay.execution_order().tolist()
    assert sorted(order) == list(range(8))
    assert lay.validate_order(order)
    assert order.index(0) < order.index(1)
    kinds = edge_list(lay)
    assert (0, 1, EDGE_K_PIPELINE) in kinds and (2, 3, EDGE_K_PIPELINE) in kinds
    assert (0, 2, EDGE_ROW_ADJACENT) in kinds and (4, 6, EDGE_ROW_ADJACENT) in kinds
    assert (0, 4, EDGE_COL_ADJACENT) in kinds and (2, 6, EDGE_COL_ADJACENT) in kinds
    assert len(kinds) == 8
    assert not lay.validate_order(order[::-1])


def test_topology_sparse_mask():
    # ttg.rs:421-431: only the diagonal of a 3x3 grid: 3 nodes, no adjacency between them
    lay = TileLayout.from_mask(96, 96, 128, 32, 32, 32, lambda tm, tn: tm == tn)
    assert lay.num_active_tiles == 3
    assert len(lay.edges) == 0
    assert len(lay.execution_order()) == 3


def test_topology_fusion_candidates():
    # ttg.rs:434-441
    lay = TileLayout.from_dense(64, 96, 128, 32, 32)
    fusions = lay.fusion_candidates()
    assert len(fusions) == 4
    assert (0, 1) in fusions and (3, 4) in fusions and (1, 2) in fusions and (4, 5) in fusions


def test_topology_reuse_hints():
    # ttg.rs:444-451: tile (0,1) shares the A rows of tile 0; a first-column tile shares B with the tile above
    lay = TileLayout.from_dense(64, 96, 128, 32, 32)
    kind, source = lay.reuse_hints()
    assert (kind[1], source[1]) == (REUSE_A, 0)
    assert kind[0] == REUSE_NONE
    assert (kind[3], source[3]) == (REUSE_B, 0)
    assert (kind[5], source[5]) == (REUSE_A, 4)


def test_topological_sort_respects_edges():
    # ttg.rs:454-460: one tile in three K stages runs 0, 1, 2
    lay = TileLayout.from_dense_k_split(32, 32, 64, 32, 32, 32, 3)
    assert lay.execution_order().tolist() == [0, 1, 2]
    assert [(r[2], r[3]) for r in records(lay)] == [(0, 21), (21, 42), (42, 64)]  # the last stage takes the rest


# ---- src/runtime/ttg_builder.rs:467-604 ----

def test_ttg_low_rank():
    # ttg_builder.rs:471-477
    lay = TileLayout.from_low_rank(256, 256, 256, 64, 64, 64, 32)
    assert lay.num_active_tiles == 16
    assert all(r[4] & 0x2 for r in records(lay))


def test_ttg_dense_and_diagonal():
    # ttg_builder.rs:538-581 (through from_policy in the reference): 128x128 in 64x64 tiles
    dense = TileLayout.from_dense(128, 128, 64, 64, 64, 32)
    assert dense.num_active_tiles == 4 and len(dense.l1_map) == 4 and len(dense.l2_table) == 4
    diag = TileLayout.from_diagonal(128, 128, 64, 64, 64, 32)
    assert diag.num_active_tiles == 2 and len(diag.l1_map) == 2
    assert all(r[0] == r[1] for r in records(diag))


# ---- builders against brute force ----

@pytest.mark.parametrize("m,n,k,mt,nt", [(256, 256, 256, 64, 64), (300, 200, 96, 128, 64), (64, 1000, 40, 256, 256)])
def test_from_dense_tables(m, n, k, mt, nt):
    lay = TileLayout.from_dense(m, n, k, mt, nt)
    gm, gn = -(-m // mt), -(-n // nt)
    want = [(tm, tn, 0, k, int((tm + 1) * mt > m or (tn + 1) * nt > n)) for tm in range(gm) for tn in range(gn)]
    assert records(lay) == want
    assert lay.l1_map.tolist() == list(range(gm * gn))
    # edges: one per horizontally and per vertically adjacent pair
    assert len(lay.edges) == gm * (gn - 1) + (gm - 1) * gn
    assert lay.validate_order(lay.execution_order())


def test_from_dense_k_split_tables():
    m, n, k, mt, nt, s = 128, 192, 200, 64, 64, 3
    lay = TileLayout.from_dense_k_split(m, n, k, mt, nt, 32, s)
    per = k // s
    want = [(tm, tn, ks * per, k if ks == s - 1 else (ks + 1) * per, 0)
            for tm in range(2) for tn in range(3) for ks in range(s)]
    assert records(lay) == want
    assert lay.num_active_tiles == 18
    order = lay.execution_order().tolist()
    assert sorted(order) == list(range(18)) and lay.validate_order(order)
    # the map workgroups are given follows that order
    assert lay.l1_map_ordered.tolist() == order


def test_from_mask_keeps_role_zero_and_connects_active_neighbours():
    # lower triangle of a 3x3 grid with a ragged edge: the reference leaves role at 0 for masked layouts
    lay = TileLayout.from_mask(150, 150, 64, 64, 64, 32, lambda tm, tn: tn <= tm)
    assert [r[:2] for r in records(lay)] == [(0, 0), (1, 0), (1, 1), (2, 0), (2, 1), (2, 2)]
    assert all(r[4] == 0 for r in records(lay))
    e = edge_list(lay)
    assert (1, 2, EDGE_ROW_ADJACENT) in e and (0, 1, EDGE_COL_ADJACENT) in e and (2, 4, EDGE_COL_ADJACENT) in e
    assert len(e) == 6  # rows: (1,2) (3,4) (4,5); columns: (0,1) (1,3) (2,4)
    order = lay.execution_order().tolist()
    assert sorted(order) == list(range(6)) and lay.validate_order(order)
    # an array works like the callable
    arr = np.tril(np.ones((3, 3), dtype=np.uint8))
    assert records(TileLayout.from_mask(150, 150, 64, 64, 64, 32, arr)) == records(lay)


def test_from_diagonal_marks_the_ragged_corner():
    lay = TileLayout.from_diagonal(150, 300, 64, 64, 64)
    assert records(lay) == [(0, 0, 0, 64, 0), (1, 1, 0, 64, 0), (2, 2, 0, 64, 1)]
    assert len(lay.edges) == 0 and lay.execution_order().tolist() == [0, 1, 2]


def test_from_random_density_and_seed():
    m = n = 64 * 40
    full = TileLayout.from_random(m, n, 64, 64, 64, 32, 1.0, seed=1)
    none = TileLayout.from_random(m, n, 64, 64, 64, 32, 0.0, seed=1)
    half = TileLayout.from_random(m, n, 64, 64, 64, 32, 0.5, seed=1)
    again = TileLayout.from_random(m, n, 64, 64, 64, 32, 0.5, seed=1)
    other = TileLayout.from_random(m, n, 64, 64, 64, 32, 0.5, seed=2)
    assert full.num_active_tiles == 1600 and none.num_active_tiles == 0
    assert abs(half.num_active_tiles - 800) < 5 * 20  # five standard deviations of Binomial(1600, 1/2)
    assert records(half) == records(again) and records(half) != records(other)
    # kept tiles appear in row-major order, each once
    tiles = [r[:2] for r in records(half)]
    assert tiles == sorted(set(tiles))


def test_from_tables_round_trip_and_checks():
    l2 = np.array([(0, 1, 0, 64, 0), (1, 0, 64, 128, 0), (1, 1, 32, 96, 1)], dtype=TILE_DTYPE)
    lay = TileLayout.from_tables(128, 128, 128, 64, 64, 32, [2, 0], l2)
    assert lay.num_active_tiles == 2
    assert lay.l1_map.tolist() == [2, 0] and lay.l1_map_ordered.tolist() == [2, 0]
    assert records(lay) == [tuple(int(x) for x in r) for r in l2]
    assert lay.execution_order().tolist() == [0, 1] and lay.validate_order([1, 0])
    with pytest.raises(ValueError, match="names record 3"):
        TileLayout.from_tables(128, 128, 128, 64, 64, 32, [3], l2)


def test_bad_dimensions_are_rejected():
    with pytest.raises(ValueError, match="tile extents"):
        TileLayout.from_dense(128, 128, 128, 0, 64)
    with pytest.raises(ValueError, match="problem extents"):
        TileLayout.from_dense(0, 128, 128, 64, 64)
    with pytest.raises(ValueError, match="K splits"):
        TileLayout.from_dense_k_split(128, 128, 128, 64, 64, 32, 0)
    with pytest.raises(ValueError, match="probability"):
        TileLayout.from_random(128, 128, 128, 64, 64, 32, 1.5)


def test_device_sizes_are_rounded_to_256():
    # src/runtime/ttg.rs:15-23: 4 bytes per level-1 entry, 20 per record
    lay = TileLayout.from_dense(64 * 9, 64 * 9, 64, 64, 64)   # 81 tiles: 324 and 1620 bytes
    assert lay.device_size() == (512, 1792)
    one = TileLayout.from_dense(64, 64, 64, 64, 64)
    assert one.device_size() == (256, 256)


def test_topological_order_is_the_lifo_kahn_order():
    # an independent Kahn's algorithm with a stack, on the mask layout's edges
    lay = TileLayout.from_mask(64 * 4, 64 * 4, 64, 64, 64, 32, lambda tm, tn: (tm + tn) % 3 != 1)
    n = lay.num_active_tiles
    nxt, indeg = {i: [] for i in range(n)}, [0] * n
    for f, t, _ in edge_list(lay):
        nxt[f].append(t)
        indeg[t] += 1
    stack, want = [i for i in range(n) if indeg[i] == 0], []
    while stack:
        v = stack.pop()
        want.append(v)
        for t in nxt[v]:
            indeg[t] -= 1
            if indeg[t] == 0:
                stack.append(t)
    assert lay.execution_order().tolist() == want
