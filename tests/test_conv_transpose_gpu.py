"""Transposed convolution parity on the GPU, through the C ABI, against the CPU
oracle.  fp32 operands (the reference's only case): max |err| < 1e-4, the bar of
examples/verify_conv_transpose.rs:204; f16/bf16 operands: the half-precision
bound of the convolution tests, 2e-2*sqrt(K)/sqrt(1024) with K = C*taps."""
import ctypes as C
import math

import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_f16, round_bf16, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


SHAPES = [  # n, h, w, c, k, r, s, stride, pad, output_padding
    (1, 2, 2, 1, 1, 2, 2, 1, 0, 0),          # examples/verify_conv_transpose.rs:66-69
    (2, 8, 8, 16, 24, 4, 4, 2, 1, 0),        # the VAE decoder layer, small (benchmark.rs:567-570)
    (1, 5, 7, 8, 8, 3, 3, 2, 1, 1),
    (3, 6, 5, 12, 20, 3, 3, 1, 1, 0),
    (1, 3, 3, 4, 4, 2, 2, 3, 0, 1),          # stride larger than the filter
    (2, 4, 6, 8, 16, 5, 3, (3, 2), (2, 1), (2, 1)),
    (1, 7, 7, 3, 5, 3, 3, 2, 0, 0),          # channel counts no vector width divides
]


def _operands(shape, seed, rounder=None):
    n, h, w, c, k, r, s = shape[:7]
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (n, h, w, c)).astype(np.float32)        # verify_conv_transpose.rs:89
    wt = rng.uniform(-0.5, 0.5, (c, r, s, k)).astype(np.float32)   # verify_conv_transpose.rs:94
    if rounder is not None:
        x, wt = rounder(x), rounder(wt)
    return x, wt


@pytest.mark.parametrize("shape", SHAPES)
def test_fp32_matches_the_oracle_to_the_reference_bar(tracea_gpu, shape):
    stride, pad, opad = shape[7:]
    x, wt = _operands(shape, 1)
    want = oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad)
    y = tracea_gpu.conv_transpose2d(_dev(x), _dev(wt), stride=stride, padding=pad, output_padding=opad)
    assert tuple(y.shape) == want.shape and y.dtype == torch.float32
    diff = np.abs(y.cpu().numpy() - want)
    assert diff.max() < 1e-4                                   # verify_conv_transpose.rs:204
    assert math.sqrt(float((diff.astype(np.float64) ** 2).mean())) < 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", SHAPES[1:])
def test_half_precision_operands(tracea_gpu, shape, dtype):
    n, h, w, c, k, r, s, stride, pad, opad = shape
    tdt, rounder = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    x, wt = _operands(shape, 2, rounder)
    want = oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad)
    sh, sw = oracle._pair(stride)
    taps = -(-r // sh) * -(-s // sw)
    tol = tol_half(c * taps, dtype)
    y = tracea_gpu.conv_transpose2d(_dev(x, tdt), _dev(wt, tdt), stride=stride, padding=pad, output_padding=opad)
    assert y.dtype == tdt
    assert_close_scaled(y.float().cpu().numpy(), want, tol, "%s half out" % (shape,))
    y32 = tracea_gpu.conv_transpose2d(_dev(x, tdt), _dev(wt, tdt), stride=stride, padding=pad, output_padding=opad,
                                      out_dtype=torch.float32)
    # fp32 output of half operands: only the accumulation order separates it from the oracle
    assert_close_scaled(y32.cpu().numpy(), want, 1e-5 * math.sqrt(c * taps) + 1e-6, "%s f32 out" % (shape,))


@pytest.mark.parametrize("layout", ["crsk", "ckrs", "krsc", "rskc"])
@pytest.mark.parametrize("tdt", [torch.float32, torch.float16])
def test_filter_storage_orders_agree(tracea_gpu, layout, tdt):
    shape = (2, 6, 6, 16, 8, 4, 4, 2, 1, 0)
    x, wt = _operands(shape, 3, round_f16)
    want = oracle.conv_transpose2d_nhwc(x, wt, 2, 1, 0)
    perm = {"crsk": (0, 1, 2, 3), "ckrs": (0, 3, 1, 2), "krsc": (3, 1, 2, 0), "rskc": (1, 2, 3, 0)}[layout]
    dw = _dev(wt, tdt).permute(*perm).contiguous()
    y = tracea_gpu.conv_transpose2d(_dev(x, tdt), dw, stride=2, padding=1, weight_layout=layout,
                                    out_dtype=torch.float32)
    assert_close_scaled(y.cpu().numpy(), want, 1e-4, layout)


def test_torch_module_weights_and_result(tracea_gpu):
    # the layout torch.nn.ConvTranspose2d holds ([C_in, C_out, R, S]) and torch's own answer
    torch.manual_seed(0)
    m = torch.nn.ConvTranspose2d(16, 8, 4, stride=2, padding=1, bias=True).cuda()
    x = torch.randn(2, 16, 9, 9, device="cuda")
    want = m(x).permute(0, 2, 3, 1)
    y = tracea_gpu.conv_transpose2d(x.permute(0, 2, 3, 1).contiguous(), m.weight.detach(), bias=m.bias.detach(),
                                    stride=2, padding=1, epilogue="bias", weight_layout="ckrs")
    assert torch.allclose(y, want, atol=1e-4, rtol=0)


def test_epilogue_kinds_and_chain(tracea_gpu):
    from tracea_amd import capi
    shape = (2, 5, 5, 8, 16, 3, 3, 2, 1, 1)
    n, h, w, c, k, r, s, stride, pad, opad = shape
    x, wt = _operands(shape, 4, round_f16)
    rng = np.random.default_rng(9)
    bias = (rng.standard_normal(k) * 0.3).astype(np.float32)
    acc = oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad)
    res = round_f16(rng.standard_normal(acc.shape))
    dx, dw = _dev(x, torch.float16), _dev(wt, torch.float16)
    tol = tol_half(c * 4, "f16")
    y = tracea_gpu.conv_transpose2d(dx, dw, bias=_dev(bias), stride=stride, padding=pad, output_padding=opad,
                                    epilogue="bias+relu")
    want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
    assert_close_scaled(y.float().cpu().numpy(), want, tol, "bias+relu")
    y = tracea_gpu.conv_transpose2d(dx, dw, residual=_dev(res, torch.float16), stride=stride, padding=pad,
                                    output_padding=opad, epilogue="residual+relu")
    want = oracle.epilogue_apply(acc, [(oracle.EPI_RESIDUAL_ADD, res), (oracle.EPI_RELU,)])
    assert_close_scaled(y.float().cpu().numpy(), want, tol, "residual+relu")
    gamma = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(k)).astype(np.float32)
    mean = (0.1 * rng.standard_normal(k)).astype(np.float32)
    var = (0.5 + rng.random(k)).astype(np.float32)
    ops = [(capi.OP_BATCHNORM, _dev(gamma), _dev(beta), _dev(mean), _dev(var), 1e-5), (capi.OP_SILU,)]
    y = tracea_gpu.conv_transpose2d_ex(dx, dw, ops, stride=stride, padding=pad, output_padding=opad)
    want = oracle.epilogue_apply(acc, [(oracle.EPI_BATCHNORM, gamma, beta, mean, var, 1e-5), (oracle.EPI_SILU,)])
    assert_close_scaled(y.float().cpu().numpy(), want, tol, "bn+silu")


def test_adjoint_identity_at_the_vae_decoder_shape(tracea_gpu):
    # benchmark.rs:567-570: 32x32x512 -> 64x64x256, 4x4, stride 2, pad 1.  Too large for the CPU
    # checker in seconds; the defining property <convT_w(x), y> == <x, conv_w'(y)> is checked
    # with the convolution kernel, and a sample of output pixels against the oracle on a crop.
    n, h, w, c, k, r, s, stride, pad = 1, 32, 32, 512, 256, 4, 4, 2, 1
    g = torch.Generator(device="cuda").manual_seed(1)
    x = (torch.rand(n, h, w, c, device="cuda", generator=g) * 2 - 1).half()
    wt = ((torch.rand(c, r, s, k, device="cuda", generator=g) - 0.5) / math.sqrt(c)).half()
    z = tracea_gpu.conv_transpose2d(x, wt, stride=stride, padding=pad, out_dtype=torch.float32)
    assert tuple(z.shape) == (1, 64, 64, 256)
    y = (torch.rand(z.shape, device="cuda", generator=g) * 2 - 1).half()
    # w[c, r, s, k] as stored is the filter bank [K'=C, R, S, C'=K] of the convolution that maps back
    back = tracea_gpu.conv2d(y, wt, stride=stride, padding=pad, out_dtype=torch.float32)
    assert tuple(back.shape) == tuple(x.shape)
    lhs = float((z.double() * y.double()).sum())
    rhs = float((x.double() * back.double()).sum())
    assert abs(lhs - rhs) <= 2e-3 * max(1.0, abs(lhs), abs(rhs))
    # a 6x6 input crop around the centre determines the 8x8 output block in its middle
    crop = x[:, 13:19, 13:19, :].float().cpu().numpy()
    want = oracle.conv_transpose2d_nhwc(crop, wt.float().cpu().numpy(), stride, pad)   # 12x12 outputs
    got = z[:, 26:38, 26:38, :].cpu().numpy()
    assert_close_scaled(got[:, 2:10, 2:10, :], want[:, 2:10, 2:10, :], 1e-4, "centre block")


def test_large_batch_runs_in_several_passes(tracea_gpu):
    # 40 images x 64x64 pixels x 4x4x64 columns of fp32 partial products = 640 MiB: two passes
    n, h, w, c, k, r, s = 40, 64, 64, 8, 64, 4, 4
    g = torch.Generator(device="cuda").manual_seed(2)
    x = (torch.rand(n, h, w, c, device="cuda", generator=g) * 2 - 1).half()
    wt = (torch.rand(c, r, s, k, device="cuda", generator=g) - 0.5).half()
    z = tracea_gpu.conv_transpose2d(x, wt, stride=2, padding=1)
    for b in (0, 31, 32, 39):   # either side of the pass boundary
        one = tracea_gpu.conv_transpose2d(x[b:b + 1].contiguous(), wt, stride=2, padding=1)
        assert torch.allclose(z[b].float(), one[0].float(), atol=2e-3, rtol=0)
    want = oracle.conv_transpose2d_nhwc(x[39:40, :8, :8].float().cpu().numpy(), wt.float().cpu().numpy(), 2, 1)
    assert_close_scaled(z[39, :14, :14].float().cpu().numpy(), want[0, :14, :14], tol_half(c * 4, "f16"), "corner")


def test_argument_errors(tracea_gpu):
    from tracea_amd import capi
    x = torch.zeros(1, 4, 4, 8, device="cuda", dtype=torch.float16)
    w = torch.zeros(8, 3, 3, 16, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError, match="output shape must be"):
        tracea_gpu.conv_transpose2d(x, w, stride=2, out=torch.zeros(1, 8, 8, 16, device="cuda", dtype=torch.float16))
    with pytest.raises(RuntimeError, match="both alike"):
        tracea_gpu.conv_transpose2d(x, w.float(), stride=2)
    with pytest.raises(RuntimeError, match="channels"):
        tracea_gpu.conv_transpose2d(x, torch.zeros(4, 3, 3, 16, device="cuda", dtype=torch.float16))
    vx, vw = tracea_gpu._view(x), tracea_gpu._transposed_weight_view(w, "crsk")
    out = torch.zeros(1, 9, 9, 16, device="cuda", dtype=torch.float16)
    vo = tracea_gpu._view(out)
    p = capi.ConvTranspose2dParams(2, 2, 0, 0, 0, 0, 1, 1, 2, capi.EPI_IDENTITY, None)
    assert capi.lib().tracea_conv_transpose2d(vx.c, vw.c, None, None, C.byref(vo.c), p) == capi.UNSUPPORTED_CONFIG
    assert "groups" in capi.last_error()
    p = capi.ConvTranspose2dParams(2, 2, 0, 0, 0, 0, 2, 2, 1, capi.EPI_IDENTITY, None)
    assert capi.lib().tracea_conv_transpose2d(vx.c, vw.c, None, None, C.byref(vo.c), p) == capi.UNSUPPORTED_CONFIG
    assert "dilation" in capi.last_error()
    p = capi.ConvTranspose2dParams(0, 2, 0, 0, 0, 0, 1, 1, 1, capi.EPI_IDENTITY, None)
    assert capi.lib().tracea_conv_transpose2d(vx.c, vw.c, None, None, C.byref(vo.c), p) == capi.INVALID_PARAMS


PHASE_SHAPES = [  # n, h, w, c, k, r, s, stride, pad, output_padding: every phase has taps and no negative padding
    (2, 8, 8, 16, 24, 4, 4, 2, 1, 0),            # uniform phases: one launch, phase in blockIdx.z
    (2, 9, 7, 32, 40, 3, 3, 2, 1, 1),            # phases of 2x2, 2x1, 1x2 and 1x1 taps: four launches
    (1, 6, 10, 8, 16, 5, 3, (3, 2), (2, 1), (2, 1)),
    (3, 5, 5, 24, 8, 2, 2, 2, 0, 0),
    (1, 12, 12, 64, 72, 6, 6, 3, 2, 0),
    (2, 7, 6, 16, 16, 3, 4, (1, 2), (1, 1), (0, 0)),
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", PHASE_SHAPES)
def test_formulation_by_output_phase_against_the_oracle_and_the_other_formulation(tracea_gpu, shape, dtype):
    """The phase path forced on and off on the same operands, with a chain that reads a residual
    through the row map: both match the oracle within the operator's tolerance."""
    from tracea_amd import capi
    n, h, w, c, k, r, s, stride, pad, opad = shape
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    rng = np.random.default_rng(h * 31 + c)
    x = rnd(rng.uniform(-1, 1, (n, h, w, c)))
    wt = rnd(rng.uniform(-0.5, 0.5, (c, r, s, k)))
    bias = rng.standard_normal(k).astype(np.float32)
    ho, wo = oracle.conv_transpose_out_shape(h, w, r, s, stride, pad, opad)
    res = rnd(rng.standard_normal((n, ho, wo, k)))
    ref = np.maximum(oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad) + bias + res, 0.0)
    got = {}
    try:
        for mode in (1, 0):
            capi.lib().tracea_set_conv_transpose_by_phase(mode)
            y = tracea_gpu.conv_transpose2d_ex(
                _dev(x, tdt), _dev(wt, tdt),
                [(capi.OP_BIAS_ADD, _dev(bias)), (capi.OP_RESIDUAL_ADD, _dev(res, tdt)), (capi.OP_RELU,)],
                stride=stride, padding=pad, output_padding=opad)
            got[mode] = y.float().cpu().numpy()
            assert_close_scaled(got[mode], ref, tol_half(c * r * s, dtype), "mode %d %s %s" % (mode, dtype, shape))
    finally:
        capi.lib().tracea_set_conv_transpose_by_phase(1)
    # the two differ by the order of fp32 additions and one output rounding at most
    ulp = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert np.abs(got[1] - got[0]).max() <= ulp * max(1.0, np.abs(ref).max())


def test_filter_cache_reuses_the_regrouped_bank_until_it_is_cleared(tracea_gpu):
    """With the filter cache on, the first call builds the regrouped bank and later calls allocate nothing
    and give the same bits as without the cache; filters changed in place are seen after a clear."""
    from tracea_amd import capi
    n, h, w, c, k, r, s, stride, pad = 2, 16, 16, 32, 24, 4, 4, 2, 1
    rng = np.random.default_rng(77)
    x = _dev(round_f16(rng.uniform(-1, 1, (n, h, w, c))), torch.float16)
    wt = _dev(round_f16(rng.uniform(-0.5, 0.5, (c, r, s, k))), torch.float16)
    run = lambda: tracea_gpu.conv_transpose2d(x, wt, stride=stride, padding=pad)
    plain = run().clone()
    assert capi.last_variant("conv2d") is not None  # the by-phase formulation
    try:
        capi.lib().tracea_set_conv_transpose_filter_cache(1)
        first = run().clone()
        torch.cuda.synchronize()
        out = torch.empty_like(first)
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            tracea_gpu.conv_transpose2d(x, wt, stride=stride, padding=pad, out=out)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        assert torch.equal(first, plain) and torch.equal(out, plain)
        # another stride / padding of the same filters is another bank
        other = tracea_gpu.conv_transpose2d(x, wt, stride=stride, padding=0)
        capi.lib().tracea_set_conv_transpose_filter_cache(0)
        assert torch.equal(other, tracea_gpu.conv_transpose2d(x, wt, stride=stride, padding=0))
        capi.lib().tracea_set_conv_transpose_filter_cache(1)
        # filters changed in place: the cached bank is the old one until the cache is cleared
        wt.mul_(2.0)
        stale = run().clone()
        assert torch.equal(stale, plain)
        capi.lib().tracea_conv_transpose_filter_cache_clear()
        fresh = run()
        assert torch.allclose(fresh.float(), 2.0 * plain.float(), atol=2e-2, rtol=2e-3) and not torch.equal(fresh, plain)
    finally:
        capi.lib().tracea_set_conv_transpose_filter_cache(0)
        capi.lib().tracea_conv_transpose_filter_cache_clear()
