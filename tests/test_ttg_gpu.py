"""GEMM over tile lists on the GPU, through the C ABI, against the CPU oracle applied tile by
tile: listed tiles hold chain(A[:, k0:k1] @ B[k0:k1, :]) within the half-precision tolerance of the
dense tests (2e-2*sqrt(K)/sqrt(1024) scaled by max(1,|ref|), plus the output rounding), tiles
that are not listed keep the bytes they held (compared exactly)."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_bf16, round_f16, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tracea_amd import capi  # noqa: E402
from tracea_amd.ttg import TILE_DTYPE, TileLayout, gemm_ttg  # noqa: E402

SENTINEL = -7.0


def _dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda().to(dtype)


def _operands(m, n, k, dtype, seed, b_layout="kn"):
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    rng = np.random.default_rng(seed)
    a = rnd(rng.standard_normal((m, k)) / np.sqrt(k))
    b = rnd(rng.standard_normal((k, n)))
    da = _dev(a, tdt)
    db = _dev(b, tdt) if b_layout == "kn" else _dev(b.T, tdt).t()  # "nk": column-major B
    return a, b, da, db, tdt


def _expected(a, b, layout, start, chain=lambda x, rows, cols: x):
    """start with the listed tiles replaced by the oracle's product over each record's K range
    (records that share a tile summed), rounded like the output."""
    want = start.copy()
    m, n = start.shape
    l1, l2 = layout.l1_map, layout.l2_table
    acc = {}
    for rec in l1:
        tm, tn, k0, k1, _ = (int(x) for x in l2[rec])
        k1 = min(k1, a.shape[1])
        rows = slice(tm * layout.mt, min((tm + 1) * layout.mt, m))
        cols = slice(tn * layout.nt, min((tn + 1) * layout.nt, n))
        part = oracle.gemm_f64(a[rows, k0:k1], b[k0:k1, cols])
        acc[(tm, tn)] = acc.get((tm, tn), 0.0) + part
    for (tm, tn), v in acc.items():
        rows = slice(tm * layout.mt, min((tm + 1) * layout.mt, m))
        cols = slice(tn * layout.nt, min((tn + 1) * layout.nt, n))
        want[rows, cols] = chain(v, rows, cols)
    listed = np.zeros((m, n), dtype=bool)
    for (tm, tn) in acc:
        listed[tm * layout.mt:(tm + 1) * layout.mt, tn * layout.nt:(tn + 1) * layout.nt] = True
    return want, listed


def _check(got, want, listed, k, dtype, what):
    got = got.float().cpu().numpy()
    np.testing.assert_array_equal(got[~listed], want[~listed], err_msg=what + ": a tile that is not listed changed")
    if listed.any():
        assert_close_scaled(got[listed], want[listed], tol_half(k, dtype), what)


TILES = [(64, 64), (128, 64), (128, 128), (256, 64), (256, 128), (256, 256)]


@pytest.mark.parametrize("mt,nt", TILES)
def test_dense_layout_equals_the_plain_gemm_bit_for_bit(tracea_gpu, mt, nt):
    # every tile listed over all of K: the same kernel work as tracea_gemm on that variant
    m, n, k = 512 + 40, 512 + 24, 256
    a, b, da, db, tdt = _operands(m, n, k, "f16", 1)
    lay = TileLayout.from_dense(m, n, k, mt, nt)
    out = torch.full((m, n), SENTINEL, dtype=tdt, device="cuda")
    gemm_ttg(da, db, lay, out)
    ran = capi.last_variant("gemm")
    assert "%dx%d" % (mt, nt) in ran
    capi.force_variant("gemm", capi.variants("gemm").index(ran))
    try:
        plain = tracea_gpu.gemm(da, db)
    finally:
        capi.force_variant("gemm", -1)
    assert torch.equal(out, plain)
    want, listed = _expected(a, b, lay, np.full((m, n), SENTINEL, np.float32))
    assert listed.all()
    _check(out, want, listed, k, "f16", "dense %dx%d" % (mt, nt))


def test_reference_experiment_ones_diagonal_and_random(tracea_gpu):
    # examples/ttg_sparse_experiment.rs: A = B = 1, 256^3, 64x64 tiles, C cleared first: listed tiles
    # hold K, the others stay 0 (dense / diagonal / random half)
    m = n = k = 256
    ones = torch.ones(m, k, dtype=torch.float16, device="cuda")
    for lay in (TileLayout.from_dense(m, n, k, 64, 64), TileLayout.from_diagonal(m, n, k, 64, 64),
                TileLayout.from_random(m, n, k, 64, 64, 32, 0.5, seed=7)):
        c = torch.zeros(m, n, dtype=torch.float16, device="cuda")
        gemm_ttg(ones, ones, lay, c)
        want = np.zeros((m, n), np.float32)
        for tm, tn, *_ in lay.l2_table[lay.l1_map]:
            want[tm * 64:(tm + 1) * 64, tn * 64:(tn + 1) * 64] = k
        np.testing.assert_array_equal(c.float().cpu().numpy(), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("b_layout", ["kn", "nk"])
@pytest.mark.parametrize("mt,nt", [(64, 64), (128, 128), (256, 256), (256, 64)])
def test_masked_layout_ragged_edges(tracea_gpu, dtype, b_layout, mt, nt):
    m, n, k = 3 * mt + 17, 3 * nt + 8, 320
    a, b, da, db, tdt = _operands(m, n, k, dtype, mt + nt, b_layout)
    lay = TileLayout.from_mask(m, n, k, mt, nt, 32, lambda tm, tn: (tm + 2 * tn) % 3 != 0)
    start = np.full((m, n), SENTINEL, np.float32)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out)
    want, listed = _expected(a, b, lay, start)
    assert listed.any() and not listed.all()
    _check(out, want, listed, k, dtype, "mask %dx%d %s %s" % (mt, nt, dtype, b_layout))


def test_windowed_k_ranges_from_caller_tables(tracea_gpu):
    # each listed tile multiplies its own window of K (a band: tile (i, j) sees k in [64 j, 64 j + 128));
    # the level-1 map lists a subset of the records in its own order
    m = n = 384
    k = 512
    mt = nt = 128
    a, b, da, db, tdt = _operands(m, n, k, "f16", 5)
    recs = [(i, j, 64 * j, 64 * j + 128, 0) for i in range(3) for j in range(3)]
    recs.append((2, 2, 448, 4096, 0))  # k_end past K is clipped
    l2 = np.array(recs, dtype=TILE_DTYPE)
    l1 = [9, 0, 4, 7, 2]
    lay = TileLayout.from_tables(m, n, k, mt, nt, 32, l1, l2)
    start = np.full((m, n), SENTINEL, np.float32)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out)
    want, listed = _expected(a, b, lay, start)
    assert listed.sum() == 5 * mt * nt
    _check(out, want, listed, 128, "f16", "windowed")
    # a range that is a multiple of 8 but not of the K tile goes through the masked kernel
    l2b = np.array([(0, 0, 8, 104, 0), (1, 2, 40, 48, 0)], dtype=TILE_DTYPE)
    lay = TileLayout.from_tables(m, n, k, mt, nt, 32, [0, 1], l2b)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out)
    want, listed = _expected(a, b, lay, start)
    _check(out, want, listed, 96, "f16", "windowed, partial K tiles")


def test_k_split_layout_sums_the_stages(tracea_gpu):
    # from_dense_k_split: every tile in 3 records over consecutive K ranges; the result is the full product
    m, n, k = 256 + 32, 256, 768
    a, b, da, db, tdt = _operands(m, n, k, "bf16", 9)
    lay = TileLayout.from_dense_k_split(m, n, k, 128, 128, 32, 3)
    bias = torch.linspace(-1, 1, n, device="cuda")
    out = torch.full((m, n), SENTINEL, dtype=tdt, device="cuda")
    gemm_ttg(da, db, lay, out, bias=bias, epilogue="bias+relu")
    assert capi.lib().tracea_last_split_k() == 3
    ref = np.maximum(oracle.gemm_f64(a, b) + bias.cpu().numpy()[None, :].astype(np.float64), 0.0)
    assert_close_scaled(out.float().cpu().numpy(), ref, tol_half(k, "bf16"), "k-split layout")


def test_epilogue_chain_on_listed_tiles_only(tracea_gpu):
    m, n, k = 512, 384, 256
    a, b, da, db, tdt = _operands(m, n, k, "f16", 13)
    lay = TileLayout.from_mask(m, n, k, 128, 128, 32, lambda tm, tn: tm >= tn)
    rng = np.random.default_rng(3)
    bias = rng.standard_normal(n).astype(np.float32)
    res = round_f16(rng.standard_normal((m, n)))
    start = np.full((m, n), SENTINEL, np.float32)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out, ops=[(capi.OP_BIAS_ADD, torch.from_numpy(bias).cuda()),
                                    (capi.OP_RESIDUAL_ADD, _dev(res, tdt)), (capi.OP_RELU,)])
    want, listed = _expected(a, b, lay, start,
                             chain=lambda v, rows, cols: np.maximum(v + bias[None, cols] + res[rows, cols], 0.0))
    _check(out, want, listed, k, "f16", "chain on a lower-triangular layout")


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_unevenly_shared_tiles_are_summed_and_unlisted_ones_left_alone(tracea_gpu, dtype):
    # Tiles with different numbers of records (src/runtime/ttg_builder.rs:140-296 builds such lists when only
    # some tiles split their K range): every listed tile is the sum of its own records, a tile without a
    # record keeps its contents.  Ragged edges, an operator chain, records of one tile far apart in the list.
    m, n, k = 320, 200, 384
    a, b, da, db, tdt = _operands(m, n, k, dtype, 31)
    recs = [(0, 0, 0, 128, 0), (1, 1, 0, 384, 0), (0, 0, 128, 256, 0), (2, 3, 64, 320, 0), (0, 0, 256, 384, 0),
            (4, 0, 0, 192, 0), (4, 0, 192, 384, 0), (3, 2, 0, 384, 0)]
    table = np.array(recs, dtype=TILE_DTYPE)
    lay = TileLayout.from_tables(m, n, k, 64, 64, 32, list(range(len(recs))), table)
    rng = np.random.default_rng(8)
    bias = rng.standard_normal(n).astype(np.float32)
    start = np.full((m, n), SENTINEL, np.float32)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out, ops=[(capi.OP_BIAS_ADD, torch.from_numpy(bias).cuda()), (capi.OP_RELU,)])
    assert capi.lib().tracea_last_split_k() == 3
    want, listed = _expected(a, b, lay, start, chain=lambda v, rows, cols: np.maximum(v + bias[None, cols], 0.0))
    assert listed.sum() > 0 and (~listed).sum() > 0
    _check(out, want, listed, k, dtype, "uneven sharing")
    # the same list with every tile's records merged into one gives the same tiles (accumulation order aside)
    merged = np.array([(0, 0, 0, 384, 0), (1, 1, 0, 384, 0), (2, 3, 64, 320, 0), (4, 0, 0, 384, 0), (3, 2, 0, 384, 0)],
                      dtype=TILE_DTYPE)
    out2 = _dev(start, tdt)
    gemm_ttg(da, db, TileLayout.from_tables(m, n, k, 64, 64, 32, list(range(5)), merged), out2,
             ops=[(capi.OP_BIAS_ADD, torch.from_numpy(bias).cuda()), (capi.OP_RELU,)])
    _check(out2, want, listed, k, dtype, "merged records")


def test_tables_in_a_caller_arena(tracea_gpu):
    # DeviceTTG::new_from_arena (src/runtime/ttg.rs:26-61): both tables inside one caller buffer
    m = n = 512
    k = 128
    a, b, da, db, tdt = _operands(m, n, k, "f16", 21)
    lay = TileLayout.from_diagonal(m, n, k, 128, 128)
    l1_bytes, l2_bytes = lay.device_size()
    arena = torch.zeros(1024 + l1_bytes + l2_bytes, dtype=torch.uint8, device="cuda")
    lay.upload_to(arena, 1024, 1024 + l1_bytes)
    torch.cuda.synchronize()
    host = arena.cpu().numpy()
    assert sorted(host[1024:1024 + 16].view(np.uint32).tolist()) == [0, 1, 2, 3]
    np.testing.assert_array_equal(host[1024 + l1_bytes:1024 + l1_bytes + 80].view(TILE_DTYPE), lay.l2_table)
    start = np.full((m, n), SENTINEL, np.float32)
    out = _dev(start, tdt)
    gemm_ttg(da, db, lay, out)
    want, listed = _expected(a, b, lay, start)
    _check(out, want, listed, k, "f16", "arena tables")


def test_empty_list_writes_nothing_and_bad_layouts_are_refused(tracea_gpu):
    m = n = k = 256
    a, b, da, db, tdt = _operands(m, n, k, "f16", 2)
    out = torch.full((m, n), SENTINEL, dtype=tdt, device="cuda")
    gemm_ttg(da, db, TileLayout.from_random(m, n, k, 64, 64, 32, 0.0), out)
    assert (out == SENTINEL).all().item()
    with pytest.raises(capi.TraceaError, match="macro-tile"):
        gemm_ttg(da, db, TileLayout.from_dense(m, n, k, 32, 32), out)
    with pytest.raises(capi.TraceaError, match="built for"):
        gemm_ttg(da, db, TileLayout.from_dense(m, n, 128, 64, 64), out)
    bad = np.array([(0, 0, 4, 68, 0)], dtype=TILE_DTYPE)
    with pytest.raises(capi.TraceaError, match="multiple of 8"):
        gemm_ttg(da, db, TileLayout.from_tables(m, n, k, 64, 64, 32, [0], bad), out)
    outside = np.array([(9, 0, 0, 64, 0)], dtype=TILE_DTYPE)
    with pytest.raises(capi.TraceaError, match="outside"):
        gemm_ttg(da, db, TileLayout.from_tables(m, n, k, 64, 64, 32, [0], outside), out)
    empty = np.array([(0, 0, 64, 64, 0)], dtype=TILE_DTYPE)
    with pytest.raises(capi.TraceaError, match="empty k range"):
        gemm_ttg(da, db, TileLayout.from_tables(m, n, k, 64, 64, 32, [0], empty), out)
    f32 = torch.zeros(m, k, device="cuda")
    with pytest.raises(capi.TraceaError, match="fp16 or bf16"):
        gemm_ttg(f32, f32, TileLayout.from_dense(m, n, k, 64, 64), torch.zeros(m, n, device="cuda"))
    assert (out == SENTINEL).all().item()


def test_large_block_sparse_size_independent_property(tracea_gpu):
    # 4096^3 with a random half of the 256x256 tiles: listed tiles equal the dense product of the same
    # kernel bit for bit, the rest are untouched
    m = n = k = 4096
    g = torch.Generator(device="cuda").manual_seed(4)
    da = (torch.randn(m, k, device="cuda", generator=g) / 64).half()
    dbt = torch.randn(n, k, device="cuda", generator=g).half()
    lay = TileLayout.from_random(m, n, k, 256, 256, 64, 0.5, seed=11)
    out = torch.full((m, n), SENTINEL, dtype=torch.float16, device="cuda")
    gemm_ttg(da, dbt.t(), lay, out)
    ran = capi.last_variant("gemm")
    capi.force_variant("gemm", capi.variants("gemm").index(ran))
    try:
        dense = tracea_gpu.gemm(da, dbt.t())
    finally:
        capi.force_variant("gemm", -1)
    listed = torch.zeros(16, 16, dtype=torch.bool)
    for tm, tn, *_ in lay.l2_table[lay.l1_map]:
        listed[int(tm), int(tn)] = True
    mask = listed.repeat_interleave(256, 0).repeat_interleave(256, 1).cuda()
    assert 0 < int(listed.sum()) < 256
    assert torch.equal(out[mask], dense[mask])
    assert (out[~mask] == SENTINEL).all().item()


# ---- low-rank MLP: C = (X A) B, the operator the reference's low-rank tile layout serves ----

def test_low_rank_mlp_ones_closed_form(tracea_gpu):
    # examples/low_rank_mlp_test.rs:16-30, 96-98: m = n = k = 256, r = 64, all ones: every entry is k*r
    ones = lambda r, c: torch.ones(r, c, dtype=torch.float16, device="cuda")
    c = tracea_gpu.low_rank_mlp(ones(256, 256), ones(256, 64), ones(64, 256))
    assert (c == 256 * 64).all().item()


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("shape", [(256, 256, 256, 64), (300, 136, 520, 24), (64, 1000, 72, 5)])
def test_low_rank_mlp_against_the_two_step_oracle(tracea_gpu, dtype, shape):
    m, n, k, r = shape
    tdt, rnd = {"f16": (torch.float16, round_f16), "bf16": (torch.bfloat16, round_bf16),
                "f32": (torch.float32, lambda v: np.asarray(v, dtype=np.float32))}[dtype]
    rng = np.random.default_rng(m + n + k + r)
    x = rnd(rng.standard_normal((m, k)) / np.sqrt(k))
    a = rnd(rng.standard_normal((k, r)))
    b = rnd(rng.standard_normal((r, n)) / np.sqrt(r))
    bias = rng.standard_normal(n).astype(np.float32)
    got = tracea_gpu.low_rank_mlp(_dev(x, tdt), _dev(a, tdt), _dev(b, tdt), bias=torch.from_numpy(bias).cuda(),
                                  epilogue="bias+relu")
    t = rnd(oracle.gemm_f64(x, a))                       # the rank-r product, rounded as the kernel stores it
    ref = np.maximum(oracle.gemm_f64(t, b) + bias[None, :], 0.0)
    if dtype == "f32":
        assert np.abs(got.cpu().numpy() - ref).max() <= 2e-4 * max(1.0, np.abs(ref).max())
    else:
        # one rounding step of T (relative 2^-11 / 2^-8) may flip against the oracle's: allow it through B
        slack = (2.0 ** -8 if dtype == "bf16" else 2.0 ** -11) * np.sqrt(r)
        assert_close_scaled(got.float().cpu().numpy(), ref, tol_half(max(k, r), dtype) + slack, "low-rank mlp")


def test_low_rank_mlp_rejects_bad_arguments(tracea_gpu):
    h = lambda r, c: torch.zeros(r, c, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.TraceaError, match="do not agree"):
        tracea_gpu.low_rank_mlp(h(64, 64), h(32, 8), h(8, 64))
    with pytest.raises(capi.TraceaError, match="share one floating type"):
        tracea_gpu.low_rank_mlp(h(64, 64), h(64, 8).float(), h(8, 64))
