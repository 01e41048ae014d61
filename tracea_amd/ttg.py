"""Tile lists: GEMM over a chosen subset of output tiles, each over its own K range.

Python face of ``include/tracea_ttg.h``, following the reference's
``TTGBuilder`` (src/runtime/ttg_builder.rs:140-296, 454-464), ``TTGLayout``
(src/core/ttg.rs:305-340) and ``RuntimeManager::launch_ttg``
(src/runtime/manager/launcher.rs:225-241).  The tables are numpy arrays in the
device format: a uint32 level-1 map and 20-byte level-2 records
``(region_m, region_n, k_start, k_end, role)``.
"""
import ctypes as C

import numpy as np

from . import capi

TILE_DTYPE = np.dtype([("region_m", "<u4"), ("region_n", "<u4"), ("k_start", "<u4"), ("k_end", "<u4"),
                       ("role", "<u4")])
EDGE_DTYPE = np.dtype([("from", "<u4"), ("to", "<u4"), ("kind", "<u4")])
EDGE_DATA_DEP, EDGE_ROW_ADJACENT, EDGE_COL_ADJACENT, EDGE_K_PIPELINE = range(4)
REUSE_NONE, REUSE_A, REUSE_B = range(3)


class TileLayout:
    """Owns a ``TraceaTtgLayout``.  Build with the ``from_*`` class methods."""

    def __init__(self, handle, dims):
        if not handle:
            raise ValueError("tile layout: " + capi.last_error())
        self._h = C.c_void_p(handle)
        self.m, self.n, self.k, self.mt, self.nt, self.kt = dims
        self._keep = []

    # ---- builders ----
    @classmethod
    def from_dense(cls, m, n, k, mt, nt, kt=32):
        return cls(capi.lib().tracea_ttg_from_dense(m, n, k, mt, nt, kt), (m, n, k, mt, nt, kt))

    @classmethod
    def from_dense_k_split(cls, m, n, k, mt, nt, kt, k_splits):
        return cls(capi.lib().tracea_ttg_from_dense_k_split(m, n, k, mt, nt, kt, k_splits), (m, n, k, mt, nt, kt))

    @classmethod
    def from_mask(cls, m, n, k, mt, nt, kt, include):
        """``include``: a callable (tm, tn) -> bool, as in the reference, or a [grid_m, grid_n] array."""
        gm, gn = -(-m // mt), -(-n // nt)
        if callable(include):
            mask = np.array([[bool(include(tm, tn)) for tn in range(gn)] for tm in range(gm)], dtype=np.uint8)
        else:
            mask = np.ascontiguousarray(np.asarray(include) != 0, dtype=np.uint8)
        if mask.shape != (gm, gn):
            raise ValueError("mask shape %s, grid is %s" % (mask.shape, (gm, gn)))
        return cls(capi.lib().tracea_ttg_from_mask(m, n, k, mt, nt, kt, mask.ctypes.data), (m, n, k, mt, nt, kt))

    @classmethod
    def from_diagonal(cls, m, n, k, mt, nt, kt=32):
        return cls(capi.lib().tracea_ttg_from_diagonal(m, n, k, mt, nt, kt), (m, n, k, mt, nt, kt))

    @classmethod
    def from_random(cls, m, n, k, mt, nt, kt, density, seed=0):
        return cls(capi.lib().tracea_ttg_from_random(m, n, k, mt, nt, kt, float(density), int(seed)),
                   (m, n, k, mt, nt, kt))

    @classmethod
    def from_low_rank(cls, m, n, k, r, mt, nt, kt=32):
        return cls(capi.lib().tracea_ttg_from_low_rank(m, n, k, r, mt, nt, kt), (m, n, k, mt, nt, kt))

    @classmethod
    def from_tables(cls, m, n, k, mt, nt, kt, l1_map, l2_table):
        l1 = np.ascontiguousarray(l1_map, dtype=np.uint32)
        l2 = np.ascontiguousarray(l2_table, dtype=TILE_DTYPE)
        return cls(capi.lib().tracea_ttg_from_tables(m, n, k, mt, nt, kt, l1.ctypes.data, len(l1),
                                                     l2.ctypes.data, len(l2)), (m, n, k, mt, nt, kt))

    def close(self):
        if getattr(self, "_h", None):
            capi.lib().tracea_ttg_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- host tables ----
    @property
    def num_active_tiles(self):
        return int(capi.lib().tracea_ttg_num_active_tiles(self._h))

    def _array(self, fn, dtype):
        n = fn(self._h, None, 0)
        out = np.zeros(n, dtype=dtype)
        if n:
            fn(self._h, out.ctypes.data, n)
        return out

    @property
    def l1_map(self):
        return self._array(capi.lib().tracea_ttg_l1_map, np.uint32)

    @property
    def l1_map_ordered(self):
        return self._array(capi.lib().tracea_ttg_l1_map_ordered, np.uint32)

    @property
    def l2_table(self):
        return self._array(capi.lib().tracea_ttg_l2_table, TILE_DTYPE)

    @property
    def edges(self):
        return self._array(capi.lib().tracea_ttg_edges, EDGE_DTYPE)

    def execution_order(self):
        return self._array(capi.lib().tracea_ttg_execution_order, np.uint32)

    def reuse_hints(self):
        n = capi.lib().tracea_ttg_reuse_hints(self._h, None, None, 0)
        kind, source = np.zeros(n, dtype=np.uint32), np.zeros(n, dtype=np.uint32)
        if n:
            capi.lib().tracea_ttg_reuse_hints(self._h, kind.ctypes.data, source.ctypes.data, n)
        return kind, source

    def fusion_candidates(self):
        e = self.edges
        return [(int(a), int(b)) for a, b, kind in e if kind == EDGE_ROW_ADJACENT]

    def validate_order(self, order):
        o = np.ascontiguousarray(order, dtype=np.uint32)
        return bool(capi.lib().tracea_ttg_validate_order(self._h, o.ctypes.data, len(o)))

    def device_size(self):
        a, b = C.c_size_t(0), C.c_size_t(0)
        capi.check("tracea_ttg_device_size", capi.lib().tracea_ttg_device_size(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def upload_to(self, arena, l1_offset, l2_offset):
        """Places the device tables inside ``arena`` (a uint8 torch tensor on the GPU)."""
        base = arena.data_ptr()
        self._keep.append(arena)
        st = capi.lib().tracea_ttg_upload_to(self._h, arena.device.index or 0, base + l1_offset, base + l2_offset)
        capi.check("tracea_ttg_upload_to", st)


def gemm_ttg(a, b, layout, out, bias=None, residual=None, epilogue="none", ops=None):
    """Writes epilogue(a[:, k0:k1] @ b[k0:k1, :]) into the tiles of ``out`` that ``layout`` lists;
    the other tiles of ``out`` keep their contents.  ``ops``: an operator chain as for
    ``ops.gemm_ex`` instead of (bias, residual, epilogue)."""
    from . import ops as _ops
    va, vb, vc = _ops._view(a), _ops._view(b), _ops._view(out)
    params = capi.GemmParams(0 if ops is not None else _ops.parse_epilogue(epilogue), _ops._stream(a))
    if ops is not None:
        arr, keep = _ops._ops_array(ops)
        st = capi.lib().tracea_gemm_ttg_ex(va.c, vb.c, C.byref(vc.c), params, arr, len(ops), layout._h)
    else:
        vbias = _ops._view(bias) if bias is not None else None
        vres = _ops._view(residual) if residual is not None else None
        st = capi.lib().tracea_gemm_ttg(va.c, vb.c, C.byref(vbias.c) if vbias else None,
                                        C.byref(vres.c) if vres else None, C.byref(vc.c), params, layout._h)
    capi.check("tracea_gemm_ttg", st)
    return out
