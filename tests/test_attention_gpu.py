"""FlashAttention-2 forward parity on the GPU, through the C ABI, against the CPU
oracle (naive softmax(QK^T)V in float64 on the bf16/f16-rounded inputs)."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_bf16, round_f16, tol_for_k

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda().to(dtype)


def _inputs(b, h, s, d, seed, rnd):
    rng = np.random.default_rng(seed)
    return [rnd(rng.standard_normal((b, h, s, d))) for _ in range(3)]


# output is a convex combination of V rows (|o| <= max|v| ~ 4): bf16 rounding of o alone is up
# to 2^-8 * |o|.  Gate: tolerance with K = D for the half-precision products plus that rounding.
def _tol(d, dtype):
    return tol_for_k(d) + (2.0 ** -8 if dtype == "bf16" else 2.0 ** -11) * 2


# members of the kernel family: (queries per workgroup, form); w4 = four waves of 64 queries, otherwise
# 32 queries per wave; a member that a head dimension does not have (3-stage rings at D = 128) is skipped
FAMILY = [("q128", "pipe"), ("q128", "pipe2"), ("q128", "tr"), ("q128", "u16"), ("q256", "s2_pipe2"),
          ("q256", "s3_pipe2"), ("q128", "s3_pipe2"), ("q256", "w4_pipe2"), ("q128", "m16"), ("q256", "s2_m16"),
          ("q128", "pipe2_x2"), ("q256", "s2_pipe2_x2"), ("q256", "s2_pp"), ("q256", "s4_pipe2"), ("q128", "s4_pipe2")]


def _member(capi, variant, d):
    name = "fa2_%s_kv64_d%d_%s" % (variant[0], d, variant[1])
    if name not in capi.variants("attention"):
        pytest.skip("the family has no member %s" % name)
    return name


@pytest.mark.parametrize("variant", FAMILY, ids=lambda v: "_".join(v))
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_small_and_edge_lengths(tracea_gpu, variant, d, dtype):
    from tracea_amd import capi
    tdt, rnd = (torch.bfloat16, round_bf16) if dtype == "bf16" else (torch.float16, round_f16)
    name = _member(capi, variant, d)
    capi.force_variant("attention", name)
    try:
        # S in {16,77,123,1025}: tests/python/edge_case_fa2.py:56-71; 128/256: tile multiples
        for (b, h, s) in [(1, 2, 16), (1, 2, 77), (2, 1, 123), (1, 2, 128), (2, 3, 256), (1, 2, 300), (1, 1, 1025)]:
            q, k, v = _inputs(b, h, s, d, 31 * s + d, rnd)
            for causal in (False, True):
                want = oracle.attention_bhsd(q, k, v, 1.0 / np.sqrt(d), causal)
                got = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=causal)
                assert_close_scaled(got.float().cpu().numpy(), want, _tol(d, dtype),
                                    "%s S=%d causal=%s %s" % (name, s, causal, dtype))
    finally:
        capi.force_variant("attention", -1)


@pytest.mark.parametrize("variant", FAMILY, ids=lambda v: "_".join(v))
@pytest.mark.parametrize("dom_mod8", [1, 5])
def test_dominant_key_needs_the_true_running_maximum(tracea_gpu, variant, dom_mod8):
    """One key scores about 2^250 times the others for every query row that can see it; the exact output is that
    key's V row.
    In the kernels a query's keys are split between lanes l and l+32 (keys with kv % 8 in 0..3 and in
    4..7); a running maximum that is consistent between the two but not the true one cancels out of an
    ordinary softmax and passes every comparison with the oracle, yet here exp2 of (score - too small a
    maximum) overflows.  The dominant key is placed once in each half."""
    from tracea_amd import capi
    b, h, s, d = 1, 2, 384, 128
    rng = np.random.default_rng(77 + dom_mod8)
    q = np.zeros((b, h, s, d), np.float32)
    k = round_bf16(rng.standard_normal((b, h, s, d)) * 0.05)
    v = round_bf16(rng.standard_normal((b, h, s, d)))
    q[...] = 4.0
    # a single dominant key per run, visible to every row (under the causal mask: to the rows at or after it)
    gk = 64 * 2 + 8 * 3 + dom_mod8          # tile 2, lane-half chosen by dom_mod8
    k[:, :, gk, :] = 4.0                    # q.k = 128 * 16 = 2048; others ~ N(0, (4*0.05)^2 * 128) ~ +-2.3
    name = _member(capi, variant, d)
    capi.force_variant("attention", name)
    try:
        for causal in (False, True):
            got = tracea_gpu.attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16),
                                       causal=causal).float().cpu().numpy()
            assert np.isfinite(got).all(), "%s causal=%s: non-finite output" % (name, causal)
            rows = slice(gk, s) if causal else slice(0, s)   # causal rows before gk cannot see it
            expect = np.broadcast_to(v[:, :, gk:gk + 1, :], got[:, :, rows, :].shape)
            # softmax weight of the dominant key is 1 - O(2^-250): the output is its V row up to bf16 rounding
            assert np.abs(got[:, :, rows, :] - expect).max() <= 2.0 ** -7 * np.abs(v).max(), (name, causal)
            if causal:  # the rows that cannot see it still match the oracle
                ref = oracle.attention_bhsd(q, k, v, 1.0 / np.sqrt(d), True)
                assert_close_scaled(got[:, :, :gk, :], ref[:, :, :gk, :], _tol(d, "bf16"), name + " before the dominant key")
    finally:
        capi.force_variant("attention", -1)


@pytest.mark.parametrize("variant", [("q128", "pipe2"), ("q128", "m16"), ("q256", "s2_pipe2"), ("q128", "pipe")], ids=lambda v: "_".join(v))
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("step", [0.05, 0.11, 0.3])
def test_scores_that_climb_along_the_sequence(tracea_gpu, variant, dtype, step):
    """The kernels' reference value for the softmax moves only when a tile's maximum is more than 2^8 above
    it.  Here every query's score grows linearly with the key index, by step * 64 per tile in the exponent's
    log2 units (3.2, 7, 19): below the threshold (the reference lags by several tiles and probabilities
    reach 2^8), just under it, and above it (it moves at every tile).  The output must be the oracle's in all
    three regimes, dense and causal, and at a sequence end inside a tile."""
    from tracea_amd import capi
    tdt, rnd = (torch.bfloat16, round_bf16) if dtype == "bf16" else (torch.float16, round_f16)
    b, h, s, d = 1, 2, 600, 128
    rng = np.random.default_rng(int(step * 100))
    # q = (c, 0, 0, ...) + noise, k_j = (j * u, ...) + noise: q.k_j / sqrt(d) * log2(e) = step * j + O(1)
    c = 8.0
    u = step * np.sqrt(d) / (c * np.log2(np.e))
    q = rng.standard_normal((b, h, s, d)) * 0.3
    k = rng.standard_normal((b, h, s, d)) * 0.3
    q[..., 0] = c
    k[..., 0] = np.arange(s) * u
    v = rng.standard_normal((b, h, s, d))
    q, k, v = rnd(q), rnd(k), rnd(v)
    name = _member(capi, variant, d)
    capi.force_variant("attention", name)
    try:
        for causal in (False, True):
            ref = oracle.attention_bhsd(q, k, v, 1.0 / np.sqrt(d), causal)
            got = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=causal).float().cpu().numpy()
            assert np.isfinite(got).all()
            assert_close_scaled(got, ref, _tol(d, dtype), "%s step %.2f causal=%s" % (name, step, causal))
    finally:
        capi.force_variant("attention", -1)


@pytest.mark.parametrize("variant", [("q128", "pipe2"), ("q256", "s2_pipe2")], ids=lambda v: "_".join(v))
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_two_query_blocks_per_workgroup(tracea_gpu, variant, d, dtype):
    """The _x2 members give a workgroup two query blocks (a heavy and a light one under a causal mask), the
    second on K/V tiles and queries requested during the first.  Every query still sees its keys in the same
    order with the same arithmetic (both fold the softmax shift into the score product; at head dimension 128
    the paired member parks half of the second block's queries in LDS to have the registers for it): the output
    must equal the one-block member's bit for bit, on lengths that end inside a tile, on scores that climb along
    the sequence and with a dominant key; the one-block member is checked against the oracle on the same inputs.
    A length with an odd number of blocks has no pairs: a forced _x2 member is then not the one that runs."""
    from tracea_amd import capi
    tdt, rnd = (torch.bfloat16, round_bf16) if dtype == "bf16" else (torch.float16, round_f16)
    bq = int(variant[0][1:])
    single, paired = _member(capi, variant, d), _member(capi, (variant[0], variant[1] + "_x2"), d)
    try:
        for (b, h, s) in [(1, 2, 2 * bq), (2, 3, 4 * bq - 37), (1, 2, 8 * bq), (1, 1, 6 * bq - bq // 2 - 1)]:
            rng = np.random.default_rng(s + d)
            q, k, v = [rng.standard_normal((b, h, s, d)) * 0.5 for _ in range(3)]
            q[..., 0] = 6.0
            k[0, 0, :, 0] = np.arange(s) * (0.11 * np.sqrt(d) / (6.0 * np.log2(np.e)))  # climbing scores in one head
            k[0, -1, s // 3, :] = 3.0                                                     # a dominant key in another
            q, k, v = rnd(q), rnd(k), rnd(v)
            for causal in (False, True):
                capi.force_variant("attention", single)
                one = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=causal)
                assert capi.last_variant("attention") == single
                capi.force_variant("attention", paired)
                two = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=causal)
                assert capi.last_variant("attention") == paired, (s, causal)
                want = oracle.attention_bhsd(q, k, v, 1.0 / np.sqrt(d), causal)
                assert torch.equal(one, two), "%s S=%d causal=%s: differs from %s" % (paired, s, causal, single)
                assert_close_scaled(one.float().cpu().numpy(), want, _tol(d, dtype), "%s S=%d causal=%s" % (single, s, causal))
        q, k, v = [_dev(rnd(np.random.default_rng(3).standard_normal((1, 2, 3 * bq, d))), tdt) for _ in range(3)]
        capi.force_variant("attention", paired)
        tracea_gpu.attention(q, k, v, causal=True)
        assert capi.last_variant("attention") != paired
    finally:
        capi.force_variant("attention", -1)


def test_reference_gpu_check_shape(tracea_gpu):
    # examples/verify_fa2_gpu.rs:67-162: B1 H4 S512 D64 causal, inputs U[0,0.2), tolerance 2e-3
    rng = np.random.default_rng(42)
    q, k, v = [round_f16(rng.uniform(0, 0.2, (1, 4, 512, 64))) for _ in range(3)]
    want = oracle.attention_bhsd(q, k, v, 1.0 / 8.0, True)
    got = tracea_gpu.attention(_dev(q, torch.float16), _dev(k, torch.float16), _dev(v, torch.float16), causal=True)
    assert np.abs(got.float().cpu().numpy() - want).max() < 2e-3


def test_invariants_on_device(tracea_gpu):
    b, h, s, d = 1, 2, 320, 128
    q, k, _ = _inputs(b, h, s, d, 5, round_bf16)
    v = round_bf16(np.tile(np.linspace(-1, 1, d, dtype=np.float32), (b, h, s, 1)))
    dq, dk, dv = [_dev(t, torch.bfloat16) for t in (q, k, v)]
    for causal in (False, True):
        o = tracea_gpu.attention(dq, dk, dv, causal=causal).float().cpu().numpy()
        assert np.abs(o - v).max() <= 2.0 ** -8  # rows of P sum to one
    q, k, v = _inputs(b, h, s, d, 6, round_bf16)
    o = tracea_gpu.attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16), causal=True)
    assert np.abs(o[0, :, 0].float().cpu().numpy() - v[0, :, 0]).max() <= 2.0 ** -7  # causal row 0 = V[0]
    # explicit scale equals the default 1/sqrt(D)
    o2 = tracea_gpu.attention(_dev(q, torch.bfloat16), _dev(k, torch.bfloat16), _dev(v, torch.bfloat16), causal=True,
                              scale=1.0 / np.sqrt(d))
    assert torch.equal(o, o2)


@pytest.mark.parametrize("causal", [False, True])
def test_config5_full_size_sampled(tracea_gpu, causal):
    # B=4, H=32, S=4096, D=128 bf16, N(0,1).  The oracle evaluates 3 (batch, head) slices at 40
    # sampled query rows each (first/last rows of tiles, random interior); every output element
    # is also checked to be finite and within the range of V.
    b, h, s, d = 4, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(0x7ACEA006)
    q = torch.randn(b, h, s, d, device="cuda", generator=g).bfloat16()
    k = torch.randn(b, h, s, d, device="cuda", generator=g).bfloat16()
    v = torch.randn(b, h, s, d, device="cuda", generator=g).bfloat16()
    o = tracea_gpu.attention(q, k, v, causal=causal)
    assert torch.isfinite(o.float()).all().item()
    assert o.float().abs().max().item() <= v.float().abs().max().item() + 1e-3
    rng = np.random.default_rng(3)
    rows = np.unique(np.concatenate([[0, 1, 63, 64, 127, 128, 4032, 4095], rng.choice(s, 32, replace=False)])).astype(np.int32)
    for (bi, hi) in [(0, 0), (1, 17), (3, 31)]:
        want = oracle.attention(q[bi, hi].float().cpu().numpy(), k[bi, hi].float().cpu().numpy(),
                                v[bi, hi].float().cpu().numpy(), 1.0 / np.sqrt(d), causal, rows=rows)
        got = o[bi, hi].float().cpu().numpy()[rows]
        assert_close_scaled(got, want, _tol(d, "bf16"), "configuration 5 slice (%d,%d) causal=%s" % (bi, hi, causal))


def test_strided_views_and_error_paths(tracea_gpu):
    from tracea_amd import capi
    b, h, s, d = 2, 3, 96, 64
    qkv = torch.randn(b, s, 3, h, d, device="cuda").half()   # packed projection layout
    q, k, v = [qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)]  # [B,H,S,D] views, D contiguous
    o = tracea_gpu.attention(q, k, v, causal=True)
    want = oracle.attention_bhsd(*[t.float().cpu().numpy() for t in (q, k, v)], 1.0 / 8.0, True)
    assert_close_scaled(o.float().cpu().numpy(), want, _tol(d, "f16"), "strided q/k/v")
    bad = torch.zeros(1, 1, 8, 160, device="cuda", dtype=torch.float16)   # above the kernels' 128
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.attention(bad, bad, bad)
    assert e.value.status == capi.UNSUPPORTED_CONFIG
    f = torch.zeros(1, 1, 8, 64, device="cuda")
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.attention(f, f, f)
    assert e.value.status == capi.UNSUPPORTED_CONFIG
    a = torch.zeros(1, 1, 8, 64, device="cuda", dtype=torch.float16)
    with pytest.raises(capi.TraceaError) as e:
        tracea_gpu.attention(a, a[:, :, :4], a)
    assert e.value.status == capi.INVALID_PARAMS


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_other_head_dimensions_and_unaligned_tensors_run_from_padded_copies(tracea_gpu, dtype):
    """Head dimensions off 64 and 128 (the reference compiles its kernel per head dimension:
    src/kernels/attention/cuda_emitter.rs:39-58), a strided head dimension, odd strides and bases off
    16 bytes: padded copies, the caller's scale (1/sqrt of the true D by default), result copied out."""
    tdt, rnd = (torch.bfloat16, round_bf16) if dtype == "bf16" else (torch.float16, round_f16)
    for (b, h, s, d) in [(2, 3, 77, 32), (1, 2, 200, 80), (2, 2, 130, 96), (1, 1, 64, 8), (1, 2, 33, 1), (1, 2, 150, 127)]:
        q, k, v = _inputs(b, h, s, d, 7 * s + d, rnd)
        for causal in (False, True):
            want = oracle.attention_bhsd(q, k, v, 1.0 / np.sqrt(d), causal)
            got = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=causal)
            assert got.shape == (b, h, s, d)
            assert_close_scaled(got.float().cpu().numpy(), want, _tol(d, dtype), "D=%d S=%d causal=%s %s" % (d, s, causal, dtype))
    # an explicit scale goes through as given
    b, h, s, d = 1, 2, 90, 40
    q, k, v = _inputs(b, h, s, d, 5, rnd)
    got = tracea_gpu.attention(_dev(q, tdt), _dev(k, tdt), _dev(v, tdt), causal=True, scale=0.25)
    assert_close_scaled(got.float().cpu().numpy(), oracle.attention_bhsd(q, k, v, 0.25, True), _tol(d, dtype), "explicit scale")
    # D = 64 the kernels could read, but: head dimension strided (a [B,H,D,S] tensor seen transposed), a
    # sequence stride of 65 elements, a base 2 bytes off
    b, h, s, d = 2, 2, 100, 64
    q, k, v = _inputs(b, h, s, d, 11, rnd)
    want = oracle.attention_bhsd(q, k, v, 1.0 / 8.0, False)
    qt = _dev(q.transpose(0, 1, 3, 2), tdt).permute(0, 1, 3, 2)
    assert qt.stride(3) != 1
    kw = torch.zeros(b, h, s, 65, device="cuda", dtype=tdt)
    kw[..., :64] = _dev(k, tdt)
    flat = torch.zeros(b * h * s * d + 8, device="cuda", dtype=tdt)
    vo = flat[1:1 + b * h * s * d].view(b, h, s, d)
    vo.copy_(_dev(v, tdt))
    assert vo.data_ptr() % 16 != 0
    out_wide = torch.full((b, h, s, 72), 7.0, device="cuda", dtype=tdt)
    got = tracea_gpu.attention(qt, kw[..., :64], vo, causal=False, out=out_wide[..., 3:67])
    assert_close_scaled(got.float().cpu().numpy(), want, _tol(d, dtype), "unaligned tensors")
    assert (out_wide[..., :3] == 7.0).all() and (out_wide[..., 67:] == 7.0).all()   # nothing written beside the result
