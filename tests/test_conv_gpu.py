"""Implicit-GEMM convolution parity on the GPU, through the C ABI, against the
CPU oracle: coordinate tables bit for bit, values within 2e-2*sqrt(K)/sqrt(1024)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_f16, round_bf16, tol_for_k, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


COORD_SHAPES = [
    (32, 56, 56, 64, 64, 3, 3, 1, 1, 1),
    (32, 28, 28, 128, 128, 3, 3, 1, 1, 1),
    (32, 56, 56, 64, 128, 3, 3, 2, 1, 1),
    (32, 56, 56, 64, 128, 1, 1, 2, 0, 1),
    (3, 9, 7, 24, 8, 5, 3, 2, 2, 1),
]


@pytest.mark.parametrize("shape", COORD_SHAPES)
def test_coordinate_tables_bit_exact(tracea_gpu, shape):
    from tracea_amd import capi
    blk = capi.ConvParamsBlock()
    assert capi.lib().tracea_conv_params_pack(*shape, C.byref(blk)) == capi.SUCCESS
    ref = oracle.conv_params(*shape)
    assert bytes(blk) == bytes(ref)
    rows_ref, base_ref, cols_ref = oracle.conv_coords(ref)
    m, k = rows_ref.shape[0], cols_ref.shape[0]
    rows = torch.empty(m, 3, dtype=torch.int32, device="cuda")
    base = torch.empty(m, dtype=torch.int64, device="cuda")
    cols = torch.empty(k, 3, dtype=torch.int32, device="cuda")
    st = capi.lib().tracea_conv_coords_device(C.byref(blk), rows.data_ptr(), base.data_ptr(), cols.data_ptr(), None)
    assert st == capi.SUCCESS, capi.last_error()
    torch.cuda.synchronize()
    assert np.array_equal(rows.cpu().numpy(), rows_ref)
    assert np.array_equal(base.cpu().numpy(), base_ref)
    assert np.array_equal(cols.cpu().numpy(), cols_ref)


SMALL = [  # n, h, w, c, k, r, s, stride, pad, dilation
    (1, 8, 8, 32, 32, 3, 3, 1, 1, 1),   # examples/verify_conv2d.rs:52-60
    (3, 14, 14, 64, 128, 3, 3, 2, 1, 1),
    (2, 9, 7, 16, 24, 1, 1, 2, 0, 1),
    (1, 12, 12, 8, 40, 5, 3, 1, 2, 1),
    (2, 10, 10, 16, 16, 3, 3, 1, 2, 2),
    (5, 7, 7, 72, 8, 3, 3, 1, 1, 1),
]


@pytest.mark.parametrize("variant", range(40))
def test_small_shapes_every_variant_both_filter_layouts(tracea_gpu, variant):
    from tracea_amd import capi
    names = capi.variants("conv2d")
    if variant >= len(names):
        pytest.skip("no such variant")
    capi.force_variant("conv2d", variant)
    try:
        for shape in SMALL:
            n, h, w, c, k, r, s, stride, pad, dil = shape
            rng = np.random.default_rng(variant * 100 + h + c)
            x = round_f16(rng.standard_normal((n, h, w, c)))
            w_rsck = round_f16(rng.standard_normal((r, s, c, k)) * np.sqrt(2.0 / (r * s * c)))
            bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
            acc = oracle.conv2d_nhwc(x, w_rsck, stride, pad, dil)
            want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
            dx = _dev(x, torch.float16)
            dw_rsck = _dev(w_rsck, torch.float16)
            dw_krsc = dw_rsck.permute(3, 0, 1, 2).contiguous()
            tol = tol_half(r * s * c, "f16")
            y = tracea_gpu.conv2d(dx, dw_krsc, bias=_dev(bias), stride=stride, padding=pad, dilation=dil,
                                  epilogue="bias+relu")
            assert_close_scaled(y.float().cpu().numpy(), want, tol, "%s krsc %s" % (names[variant], shape))
            y = tracea_gpu.conv2d(dx, dw_rsck, bias=_dev(bias), stride=stride, padding=pad, dilation=dil,
                                  epilogue="bias+relu", weight_layout="rsck")
            assert_close_scaled(y.float().cpu().numpy(), want, tol, "%s rsck %s" % (names[variant], shape))
    finally:
        capi.force_variant("conv2d", -1)


PATCH_SHAPES = [  # n, h, w, c, k, r, s, stride, pad, dilation: all with C % 16 == 0
    (2, 20, 20, 64, 64, 3, 3, 1, 1, 1),    # 400 pixels: several tiles per image, last one partial
    (1, 33, 17, 32, 72, 3, 3, 1, 1, 1),    # K = 288: partial last filter tile, N not a tile multiple
    (3, 14, 14, 64, 128, 3, 3, 2, 1, 1),   # stride 2
    (2, 12, 12, 16, 40, 5, 3, 1, 2, 1),    # 5x3 taps, K = 240
    (2, 13, 11, 48, 24, 3, 3, 1, 2, 2),    # dilation 2, C/8 even -> padded pixel pitch
    (4, 9, 9, 128, 96, 1, 1, 1, 0, 1),     # 1x1
    (1, 40, 40, 16, 16, 3, 3, (2, 1), (0, 2), 1),  # asymmetric stride and padding
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_patch_resident_variants(tracea_gpu, dtype):
    """The LDS-patch convolution kernels against the oracle, forced one by one (a variant
    whose patch does not fit a shape falls back to the streamed kernel of the same tile)."""
    from tracea_amd import capi
    names = capi.variants("conv2d")
    patch = [i for i, nm in enumerate(names) if nm.endswith("_patch")]
    assert patch, "no patch-resident variant in the build"
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rnd = round_f16 if dtype == "f16" else round_bf16
    ran = set()
    try:
        for vi in patch:
            capi.force_variant("conv2d", vi)
            for shape in PATCH_SHAPES:
                n, h, w, c, k, r, s, stride, pad, dil = shape
                rng = np.random.default_rng(vi * 1000 + h * 7 + c)
                x = rnd(rng.standard_normal((n, h, w, c)))
                wk = rnd(rng.standard_normal((k, r, s, c)) * np.sqrt(2.0 / (r * s * c)))
                bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
                ref = torch.nn.functional.conv2d(
                    torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(wk).permute(0, 3, 1, 2).double(),
                    bias=torch.from_numpy(bias).double(), stride=stride, padding=pad, dilation=dil)
                ref = torch.relu(ref).permute(0, 2, 3, 1).numpy()
                if isinstance(stride, int):  # the oracle takes symmetric geometry: cross-check torch with it once
                    acc = oracle.conv2d_nhwc(x, np.ascontiguousarray(wk.transpose(1, 2, 3, 0)), stride, pad, dil)
                    want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
                    assert np.abs(want - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
                y = tracea_gpu.conv2d(_dev(x, tdt), _dev(wk, tdt), bias=_dev(bias), stride=stride, padding=pad,
                                      dilation=dil, epilogue="bias+relu")
                assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(r * s * c, dtype),
                                    "%s %s %s" % (names[vi], dtype, shape))
                ran.add(capi.last_variant("conv2d"))
    finally:
        capi.force_variant("conv2d", -1)
    assert {names[i] for i in patch} <= ran, "a patch-resident variant never ran: %s" % sorted(ran)


RESIDENT_SHAPES = [  # n, h, w, k, stride, pad, dilation: 64 input channels, 3x3 (K = 576, the kernel's filter size)
    (2, 20, 20, 64, 1, 1, 1),     # 400 pixels per image
    (3, 56, 56, 64, 1, 1, 1),     # tiles of whole rows, as configuration 3 cuts them
    (1, 33, 17, 128, 1, 1, 1),    # two filter slabs, tiles that start and end inside rows
    (2, 15, 22, 40, 1, 1, 1),     # 40 filters: partial channel groups (general epilogue)
    (2, 19, 19, 64, 2, 1, 1),     # stride 2
    (1, 24, 18, 64, 1, 2, 2),     # dilation 2
    (2, 12, 30, 64, 1, 0, 1),     # no padding
    (1, 9, 70, 64, 1, (1, 3), 1), # wide rows, asymmetric padding
]


# the members that keep the input patch in LDS with the filter slab resident beside it or in a ring of taps,
# and the input channels each is compiled for
LDS_MEMBERS = [("c448x64_k576_resident", 64), ("c400x64_c64_w16_resident", 64), ("c400x64_c64_w8_w16_resident", 64),
               ("c208x64_c128_s4_w16_patch", 128)]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("member,cin", LDS_MEMBERS)
def test_filter_resident_variant(tracea_gpu, dtype, member, cin):
    """The kernels that keep the input patch in LDS together with the filter slab (or a ring of its taps),
    forced, against the oracle: tile cuts, strides, dilation, padding, partial filter slabs."""
    from tracea_amd import capi
    names = capi.variants("conv2d")
    assert member in names, "no member %s in the build" % member
    vi = [names.index(member)]
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rnd = round_f16 if dtype == "f16" else round_bf16
    kg = 9 * cin
    capi.force_variant("conv2d", vi[0])
    try:
        for shape in RESIDENT_SHAPES:
            n, h, w, k, stride, pad, dil = shape
            rng = np.random.default_rng(h * 31 + w + k)
            x = rnd(rng.standard_normal((n, h, w, cin)))
            wk = rnd(rng.standard_normal((k, 3, 3, cin)) * np.sqrt(2.0 / kg))
            bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
            ref = torch.nn.functional.conv2d(
                torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(wk).permute(0, 3, 1, 2).double(),
                bias=torch.from_numpy(bias).double(), stride=stride, padding=pad, dilation=dil)
            ref = torch.relu(ref).permute(0, 2, 3, 1).numpy()
            if isinstance(pad, int):  # the oracle takes symmetric geometry: torch is cross-checked with it
                acc = oracle.conv2d_nhwc(x, np.ascontiguousarray(wk.transpose(1, 2, 3, 0)), stride, pad, dil)
                want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
                assert np.abs(want - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
            y = tracea_gpu.conv2d(_dev(x, tdt), _dev(wk, tdt), bias=_dev(bias), stride=stride, padding=pad,
                                  dilation=dil, epilogue="bias+relu")
            assert capi.last_variant("conv2d") == names[vi[0]], "%s refused %s" % (member, shape)
            assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(kg, dtype), "%s %s %s" % (member, dtype, shape))
    finally:
        capi.force_variant("conv2d", -1)


# the members for few pixels and many channels (K split over the waves of a workgroup)
KSPLIT_MEMBERS = [("c112x64_c256_s4_w16_ksplit", 256), ("c64x64_c512_s4_w16_ksplit", 512),
                  ("c32x64_c256_s4_w16_ksplit", 256), ("c16x64_c256_s4_w16_ksplit", 256)]
KSPLIT_SHAPES = [  # n, h, w, k, filter size, stride, pad, dilation
    (32, 14, 14, 256, 3, 1, 1, 1),    # a ResNet's 14x14 stage at batch 32: tiles of 98 pixels (7 rows) at 256 channels
    (32, 7, 7, 512, 3, 1, 1, 1),      # its 7x7 stage: one tile of 49 pixels per image
    (2, 14, 14, 64, 3, 1, 1, 1),      # small launch: tiles of one pixel block
    (16, 14, 14, 128, 3, 1, 1, 1),    # tiles of 25 pixels that start and end inside rows
    (1, 13, 9, 40, 3, 1, 1, 1),       # 40 filters: partial channel groups (general epilogue)
    (2, 15, 7, 64, 3, 2, 1, 1),       # stride 2
    (1, 12, 10, 64, 3, 1, 2, 2),      # dilation 2
    (2, 9, 12, 64, 3, 1, 0, 1),       # no padding
    (1, 5, 20, 64, 3, 1, (1, 3), 1),  # wide rows, asymmetric padding
    (8, 14, 14, 128, 1, 1, 0, 1),     # 1x1 filter: two stages in all
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("member,cin", KSPLIT_MEMBERS)
def test_ksplit_variant(tracea_gpu, dtype, member, cin):
    """The kernels that split K over the waves of a workgroup (patch in LDS, filters through a ring of
    128-channel stages, partial sums added in wave order), forced, against torch in double and the oracle."""
    from tracea_amd import capi
    names = capi.variants("conv2d")
    assert member in names, "no member %s in the build" % member
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rnd = round_f16 if dtype == "f16" else round_bf16
    capi.force_variant("conv2d", names.index(member))
    try:
        for shape in KSPLIT_SHAPES:
            n, h, w, k, fs, stride, pad, dil = shape
            kg = fs * fs * cin
            rng = np.random.default_rng(h * 31 + w + k)
            x = rnd(rng.standard_normal((n, h, w, cin)))
            wk = rnd(rng.standard_normal((k, fs, fs, cin)) * np.sqrt(2.0 / kg))
            bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
            ref = torch.nn.functional.conv2d(
                torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(wk).permute(0, 3, 1, 2).double(),
                bias=torch.from_numpy(bias).double(), stride=stride, padding=pad, dilation=dil)
            ref = torch.relu(ref).permute(0, 2, 3, 1).numpy()
            if isinstance(pad, int) and n <= 16:  # the oracle takes symmetric geometry: torch is cross-checked with it
                acc = oracle.conv2d_nhwc(x, np.ascontiguousarray(wk.transpose(1, 2, 3, 0)), stride, pad, dil)
                want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
                assert np.abs(want - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
            y = tracea_gpu.conv2d(_dev(x, tdt), _dev(wk, tdt), bias=_dev(bias), stride=stride, padding=pad,
                                  dilation=dil, epilogue="bias+relu")
            assert capi.last_variant("conv2d") == member, "%s refused %s" % (member, shape)
            assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(kg, dtype), "%s %s %s" % (member, dtype, shape))
    finally:
        capi.force_variant("conv2d", -1)


THIN_SHAPES = [  # n, h, w, k, filter (r, s), stride, pad, dilation: 8 input channels
    (32, 224, 224, 64, (7, 7), 4, 3, 1),          # the ResNet benchmark's first layer at batch 32
    (2, 60, 44, 64, (7, 7), 4, 3, 1),             # small launch
    (1, 37, 53, 40, (7, 7), 2, 3, 1),             # stride 2, 40 filters (general epilogue)
    (3, 30, 30, 128, (7, 7), 1, 3, 1),            # stride 1, two filter slabs
    (1, 40, 33, 64, (7, 7), 4, 0, 1),             # no padding
    (2, 31, 29, 64, (7, 5), (3, 2), (2, 4), 1),   # 7x5 filter, mixed strides, asymmetric padding
    (2, 45, 38, 64, (7, 8), (2, 4), (6, 1), (2, 1)),  # 8 taps per row, filter rows 2 apart
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_thin8_variant(tracea_gpu, dtype):
    """The first-layer kernel (8 input channels, filter bank in registers, patch in LDS), forced, against
    torch in double and, on symmetric geometry, the oracle."""
    from tracea_amd import capi
    member = "c128x64_c8_r7_w16_thin"
    names = capi.variants("conv2d")
    assert member in names, "no member %s in the build" % member
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rnd = round_f16 if dtype == "f16" else round_bf16
    capi.force_variant("conv2d", names.index(member))
    try:
        for shape in THIN_SHAPES:
            n, h, w, k, (fr, fs), stride, pad, dil = shape
            kg = fr * fs * 8
            rng = np.random.default_rng(h * 31 + w + k)
            x = rnd(rng.standard_normal((n, h, w, 8)))
            x[..., 3:] = 0.0 if n == 32 else x[..., 3:]     # the benchmark's image: 3 real channels
            wk = rnd(rng.standard_normal((k, fr, fs, 8)) * np.sqrt(2.0 / kg))
            bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
            ref = torch.nn.functional.conv2d(
                torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(wk).permute(0, 3, 1, 2).double(),
                bias=torch.from_numpy(bias).double(), stride=stride, padding=pad, dilation=dil)
            ref = torch.relu(ref).permute(0, 2, 3, 1).numpy()
            if isinstance(pad, int) and isinstance(stride, int) and fr == fs and n <= 3:
                acc = oracle.conv2d_nhwc(x, np.ascontiguousarray(wk.transpose(1, 2, 3, 0)), stride, pad, dil)
                want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
                assert np.abs(want - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
            y = tracea_gpu.conv2d(_dev(x, tdt), _dev(wk, tdt), bias=_dev(bias), stride=stride, padding=pad,
                                  dilation=dil, epilogue="bias+relu")
            assert capi.last_variant("conv2d") == member, "%s refused %s" % (member, shape)
            assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(kg, dtype), "%s %s %s" % (member, dtype, shape))
    finally:
        capi.force_variant("conv2d", -1)


def test_thin8_variant_operator_chains(tracea_gpu):
    """The first-layer kernel's register epilogue in all its forms and two chains outside it."""
    from tracea_amd import capi
    member = "c128x64_c8_r7_w16_thin"
    n, h, w, k = 6, 50, 62, 64
    rng = np.random.default_rng(78)
    x = round_f16(rng.standard_normal((n, h, w, 8)))
    w_rsck = round_f16(rng.standard_normal((7, 7, 8, k)) * np.sqrt(2.0 / 392))
    acc = oracle.conv2d_nhwc(x, w_rsck, 2, 3, 1)
    bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
    (gamma, beta, mean, var), (scale, shift) = _bn_params(rng, k)
    res = round_f16(rng.standard_normal(acc.shape))
    dx, dw = _dev(x, torch.float16), _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous()
    O, E = capi, oracle
    aff = {"bias": ((O.OP_BIAS_ADD, _dev(bias)), (E.EPI_BIAS_ADD, bias)),
           "ss": ((O.OP_SCALE_SHIFT, _dev(scale), _dev(shift)), (E.EPI_SCALE_SHIFT, scale, shift)),
           "bn": ((O.OP_BATCHNORM, _dev(gamma), _dev(beta), _dev(mean), _dev(var), 1e-5), (E.EPI_BATCHNORM, gamma, beta, mean, var, 1e-5))}
    relu = ((O.OP_RELU,), (E.EPI_RELU,))
    resid = ((O.OP_RESIDUAL_ADD, _dev(res, torch.float16)), (E.EPI_RESIDUAL_ADD, res))
    chains = [[], [aff["bn"], relu], [aff["bias"]], [aff["ss"], relu, resid, relu], [resid], [relu, resid],
              [aff["bias"], resid, relu], [aff["bias"], ((O.OP_SILU,), (E.EPI_SILU,))], [resid, aff["ss"]]]
    capi.force_variant("conv2d", member)
    try:
        for chain in chains:
            want = oracle.epilogue_apply(acc, [c[1] for c in chain])
            y = tracea_gpu.conv2d_ex(dx, dw, [c[0] for c in chain], stride=2, padding=3)
            assert capi.last_variant("conv2d") == member
            assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(392), "%s chain %s" % (member, [c[1][0] for c in chain]))
    finally:
        capi.force_variant("conv2d", -1)


@pytest.mark.parametrize("member,cin", LDS_MEMBERS + KSPLIT_MEMBERS)
def test_filter_resident_variant_operator_chains(tracea_gpu, member, cin):
    """Every form of their straight-line epilogue ([affine] [ReLU] [residual] [ReLU]) and chains outside it
    (SiLU and GELU among them), against the oracle's chain on the oracle's accumulator."""
    from tracea_amd import capi
    names = capi.variants("conv2d")
    vi = names.index(member)
    # (the K-split members on a launch that gives them tiles of four pixel blocks)
    n, h, w, k = (2, 18, 25, 64) if cin < 256 else (128, 10, 10, 64)
    kg = 9 * cin
    rng = np.random.default_rng(77)
    x = round_f16(rng.standard_normal((n, h, w, cin)))
    w_rsck = round_f16(rng.standard_normal((3, 3, cin, k)) * np.sqrt(2.0 / kg))
    acc = oracle.conv2d_nhwc(x, w_rsck, 1, 1, 1)
    bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
    (gamma, beta, mean, var), (scale, shift) = _bn_params(rng, k)
    res = round_f16(rng.standard_normal(acc.shape))
    dx, dw = _dev(x, torch.float16), _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous()
    dres, dbias = _dev(res, torch.float16), _dev(bias)
    O, E = capi, oracle
    aff = {"bias": ((O.OP_BIAS_ADD, dbias), (E.EPI_BIAS_ADD, bias)),
           "bias16": ((O.OP_BIAS_ADD, _dev(round_f16(bias), torch.float16)), (E.EPI_BIAS_ADD, round_f16(bias))),
           "ss": ((O.OP_SCALE_SHIFT, _dev(scale), _dev(shift)), (E.EPI_SCALE_SHIFT, scale, shift)),
           "bn": ((O.OP_BATCHNORM, _dev(gamma), _dev(beta), _dev(mean), _dev(var), 1e-5), (E.EPI_BATCHNORM, gamma, beta, mean, var, 1e-5))}
    relu = ((O.OP_RELU,), (E.EPI_RELU,))
    resid = ((O.OP_RESIDUAL_ADD, dres), (E.EPI_RESIDUAL_ADD, res))
    gelu = ((O.OP_GELU,), (E.EPI_GELU,))
    silu = ((O.OP_SILU,), (E.EPI_SILU,))
    chains = [[]]
    for a in (None, "bias", "ss", "bn"):                      # the 16 forms (each affine kind once over them)
        for r1 in (False, True):
            for rs in (False, True):
                for r2 in (False, True):
                    c = ([aff[a]] if a else []) + ([relu] if r1 else []) + ([resid] if rs else []) + ([relu] if r2 else [])
                    if c and (a != "bn" or rs):                # keep the list short: BatchNorm with a residual only
                        chains.append(c)
    chains += [[aff["bias16"], relu], [relu, aff["bias"]], [resid, aff["ss"]], [aff["bias"], gelu], [resid, resid, relu],
               [aff["ss"], aff["bias"], relu], [silu], [aff["bias"], silu], [aff["bn"], silu, resid]]  # outside the fast form: general path
    capi.force_variant("conv2d", vi)
    try:
        for chain in chains:
            want = oracle.epilogue_apply(acc, [c[1] for c in chain])
            y = tracea_gpu.conv2d_ex(dx, dw, [c[0] for c in chain], stride=1, padding=1)
            assert capi.last_variant("conv2d") == names[vi]
            assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(kg), "%s chain %s" % (member, [c[1][0] for c in chain]))
        # fp32 output and a bf16 residual on f16 operands leave the fast form too
        y = tracea_gpu.conv2d_ex(dx, dw, [aff["bias"][0], relu[0]], stride=1, padding=1, out_dtype=torch.float32)
        want = oracle.epilogue_apply(acc, [aff["bias"][1], relu[1]])
        assert y.dtype == torch.float32
        assert_close_scaled(y.cpu().numpy(), want, tol_for_k(kg), "fp32 output")
        resb = round_bf16(res)
        y = tracea_gpu.conv2d_ex(dx, dw, [(O.OP_RESIDUAL_ADD, _dev(resb, torch.bfloat16)), relu[0]], stride=1, padding=1)
        want = oracle.epilogue_apply(acc, [(E.EPI_RESIDUAL_ADD, resb), relu[1]])
        assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(kg), "bf16 residual on f16 operands")
    finally:
        capi.force_variant("conv2d", -1)


@pytest.mark.parametrize("kernel", ["t128x64x64_w4x1_p2", "t64x64x64_w2x2_p2", "c256x64_w8x1_s3_patch",
                                    "c448x64_k576_resident", "c400x64_c64_w16_resident", None])
def test_conv_silu_kinds_through_tracea_conv2d(tracea_gpu, kernel):
    """TRACEA_EPILOGUE_SILU and TRACEA_EPILOGUE_BIAS_SILU through tracea_conv2d on the streamed, the
    patch-resident and the filter-resident kernels (and whatever the selector picks), against
    oracle.epilogue_apply on the oracle's accumulator (x / (1 + exp(-x)), src/kernels/gpu/epilogue.cuh)."""
    from tracea_amd import capi
    rng = np.random.default_rng(0x51)
    x = round_f16(rng.standard_normal((2, 20, 20, 64)))
    w_rsck = round_f16(rng.standard_normal((3, 3, 64, 64)) * np.sqrt(2.0 / 576))
    bias = (rng.standard_normal(64) * 0.5).astype(np.float32)
    acc = oracle.conv2d_nhwc(x, w_rsck, 1, 1, 1)
    dx, dw = _dev(x, torch.float16), _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous()
    if kernel is not None:
        capi.force_variant("conv2d", kernel)
    try:
        y = tracea_gpu.conv2d(dx, dw, stride=1, padding=1, epilogue="silu")
        if kernel is not None:
            assert capi.last_variant("conv2d") == kernel
        want = oracle.epilogue_apply(acc, [(oracle.EPI_SILU,)])
        assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(576), "silu on %s" % kernel)
        y = tracea_gpu.conv2d(dx, dw, bias=_dev(bias), stride=1, padding=1, epilogue="bias+silu")
        want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_SILU,)])
        assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(576), "bias+silu on %s" % kernel)
    finally:
        capi.force_variant("conv2d", -1)


def test_k576_with_other_channel_counts_runs_on_another_kernel(tracea_gpu):
    """K = 576 with 16 or 32 input channels (6x6 and 3x6 filters): the kernels compiled for 3x3x64 must
    refuse and the selector's choice must compute it."""
    from tracea_amd import capi
    for cin, (r, sz) in ((16, (6, 6)), (32, (3, 6))):
        rng = np.random.default_rng(cin)
        x = round_f16(rng.standard_normal((32, 56, 56, cin)))
        w_rsck = round_f16(rng.standard_normal((r, sz, cin, 64)) * np.sqrt(2.0 / 576))
        dx, dw = _dev(x, torch.float16), _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous()
        y = tracea_gpu.conv2d(dx, dw, stride=1, padding=(1, 2), epilogue="relu")
        used = capi.last_variant("conv2d")
        assert used is not None and not used.endswith("_resident"), used
        ref = torch.relu(torch.nn.functional.conv2d(
            torch.from_numpy(x[:2]).permute(0, 3, 1, 2).double(), torch.from_numpy(w_rsck).permute(3, 2, 0, 1).double(),
            padding=(1, 2))).permute(0, 2, 3, 1).numpy()
        assert_close_scaled(y[:2].float().cpu().numpy(), ref, tol_for_k(576), "C=%d" % cin)


def test_asymmetric_stride_and_padding_bf16(tracea_gpu):
    torch_f = torch.nn.functional
    rng = np.random.default_rng(9)
    x = round_bf16(rng.standard_normal((2, 11, 13, 16)))
    wk = round_bf16(rng.standard_normal((24, 3, 5, 16)) * 0.1)
    y = tracea_gpu.conv2d(_dev(x, torch.bfloat16), _dev(wk, torch.bfloat16), stride=(2, 1), padding=(1, 2))
    ref = torch_f.conv2d(torch.from_numpy(x).permute(0, 3, 1, 2).double(), torch.from_numpy(wk).permute(0, 3, 1, 2).double(),
                         stride=(2, 1), padding=(1, 2)).permute(0, 2, 3, 1).numpy()
    assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(3 * 5 * 16, "bf16"), "asymmetric conv")


def test_config3_full_size_bias_relu(tracea_gpu):
    # N=32, 56x56x64 -> 64, 3x3 s1 p1, bias+ReLU; activations N(0,1), Kaiming weights, bias N(0,0.1)
    rng = np.random.default_rng(0x7ACEA003)
    x = round_f16(rng.standard_normal((32, 56, 56, 64)))
    w_rsck = round_f16(rng.standard_normal((3, 3, 64, 64)) * np.sqrt(2.0 / 576))
    bias = (rng.standard_normal(64) * 0.1).astype(np.float32)
    acc = oracle.conv2d_nhwc(x, w_rsck, 1, 1)
    want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
    dw = _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous()
    y = tracea_gpu.conv2d(_dev(x, torch.float16), dw, bias=_dev(bias), stride=1, padding=1, epilogue="bias+relu")
    assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(576), "configuration 3")


def _bn_params(rng, ch):
    gamma = rng.uniform(0.5, 1.5, ch).astype(np.float32)
    beta = (rng.standard_normal(ch) * 0.1).astype(np.float32)
    mean = (rng.standard_normal(ch) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, ch).astype(np.float32)
    scale = (gamma / np.sqrt(var + 1e-5)).astype(np.float32)
    shift = (beta - mean * scale).astype(np.float32)
    return (gamma, beta, mean, var), (scale, shift)


def test_config4_fused_basic_block(tracea_gpu):
    # conv3x3+BN+ReLU -> conv3x3+BN+residual+ReLU, N=32, 128 channels, 28x28; fusion order of
    # src/core/optimizer.rs:122-150 (BN producers gamma,beta,mean,var; then Add; then Relu).
    from tracea_amd import capi
    rng = np.random.default_rng(0x7ACEA004)
    ch = 128
    x = round_f16(rng.standard_normal((32, 28, 28, ch)))
    w1 = round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch)))
    w2 = round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch)))
    bn1, fold1 = _bn_params(rng, ch)
    bn2, fold2 = _bn_params(rng, ch)
    # oracle: y1 stored in f16, as on the device
    y1 = oracle.epilogue_apply(oracle.conv2d_nhwc(x, w1, 1, 1), [(oracle.EPI_SCALE_SHIFT,) + fold1, (oracle.EPI_RELU,)])
    y1 = round_f16(y1)
    y2 = oracle.epilogue_apply(oracle.conv2d_nhwc(y1, w2, 1, 1),
                               [(oracle.EPI_SCALE_SHIFT,) + fold2, (oracle.EPI_RESIDUAL_ADD, x.reshape(-1, ch)), (oracle.EPI_RELU,)])
    dx = _dev(x, torch.float16)
    dw1 = _dev(w1, torch.float16).permute(3, 0, 1, 2).contiguous()
    dw2 = _dev(w2, torch.float16).permute(3, 0, 1, 2).contiguous()
    d1 = tracea_gpu.conv2d_ex(dx, dw1, [(capi.OP_SCALE_SHIFT, _dev(fold1[0]), _dev(fold1[1])), (capi.OP_RELU,)],
                              stride=1, padding=1)
    assert_close_scaled(d1.float().cpu().numpy(), y1, tol_for_k(9 * ch), "block conv1")
    d2 = tracea_gpu.conv2d_ex(d1, dw2, [(capi.OP_SCALE_SHIFT, _dev(fold2[0]), _dev(fold2[1])),
                                        (capi.OP_RESIDUAL_ADD, dx), (capi.OP_RELU,)], stride=1, padding=1)
    assert_close_scaled(d2.float().cpu().numpy(), y2, tol_for_k(9 * ch), "block output")
    # unfolded BatchNorm gives the same block output up to fp32 rounding of the fold
    u1 = tracea_gpu.conv2d_ex(dx, dw1, [(capi.OP_BATCHNORM,) + tuple(_dev(t) for t in bn1) + (1e-5,), (capi.OP_RELU,)],
                              stride=1, padding=1)
    assert (u1.float() - d1.float()).abs().max().item() <= 2e-2


def test_config4_downsample_block(tracea_gpu):
    # 64ch 56x56 -> 128ch 28x28: conv3x3 s2 + BN + ReLU -> conv3x3 s1 + BN, shortcut conv1x1 s2 + BN, add, ReLU
    from tracea_amd import capi
    rng = np.random.default_rng(0x7ACEA005)
    x = round_f16(rng.standard_normal((32, 56, 56, 64)))
    w1 = round_f16(rng.standard_normal((3, 3, 64, 128)) * np.sqrt(2.0 / 576))
    w2 = round_f16(rng.standard_normal((3, 3, 128, 128)) * np.sqrt(2.0 / 1152))
    ws = round_f16(rng.standard_normal((1, 1, 64, 128)) * np.sqrt(2.0 / 64))
    _, f1 = _bn_params(rng, 128)
    _, f2 = _bn_params(rng, 128)
    _, fs = _bn_params(rng, 128)
    y1 = round_f16(oracle.epilogue_apply(oracle.conv2d_nhwc(x, w1, 2, 1), [(oracle.EPI_SCALE_SHIFT,) + f1, (oracle.EPI_RELU,)]))
    sc = round_f16(oracle.epilogue_apply(oracle.conv2d_nhwc(x, ws, 2, 0), [(oracle.EPI_SCALE_SHIFT,) + fs]))
    y2 = oracle.epilogue_apply(oracle.conv2d_nhwc(y1, w2, 1, 1),
                               [(oracle.EPI_SCALE_SHIFT,) + f2, (oracle.EPI_RESIDUAL_ADD, sc.reshape(-1, 128)), (oracle.EPI_RELU,)])
    dx = _dev(x, torch.float16)
    k = lambda w: _dev(w, torch.float16).permute(3, 0, 1, 2).contiguous()
    d1 = tracea_gpu.conv2d_ex(dx, k(w1), [(capi.OP_SCALE_SHIFT, _dev(f1[0]), _dev(f1[1])), (capi.OP_RELU,)], stride=2, padding=1)
    ds = tracea_gpu.conv2d_ex(dx, k(ws), [(capi.OP_SCALE_SHIFT, _dev(fs[0]), _dev(fs[1]))], stride=2, padding=0)
    d2 = tracea_gpu.conv2d_ex(d1, k(w2), [(capi.OP_SCALE_SHIFT, _dev(f2[0]), _dev(f2[1])), (capi.OP_RESIDUAL_ADD, ds), (capi.OP_RELU,)],
                              stride=1, padding=1)
    assert_close_scaled(d1.float().cpu().numpy(), y1, tol_for_k(576), "downsample conv1")
    assert_close_scaled(ds.float().cpu().numpy(), sc, tol_for_k(64), "shortcut 1x1")
    assert_close_scaled(d2.float().cpu().numpy(), y2, tol_for_k(1152), "downsample block output")


def test_error_paths(tracea_gpu):
    from tracea_amd import capi
    x = torch.zeros(1, 8, 8, 16, device="cuda", dtype=torch.float16)
    w = torch.zeros(8, 3, 3, 16, device="cuda", dtype=torch.float16)
    out = torch.zeros(1, 8, 8, 8, device="cuda", dtype=torch.float16)

    def call(xv, wv, ov, **kw):
        p = dict(stride_h=1, stride_w=1, padding_h=1, padding_w=1, dilation_h=1, dilation_w=1, groups=1)
        p.update(kw)
        params = capi.Conv2dParams(p["stride_h"], p["stride_w"], p["padding_h"], p["padding_w"], p["dilation_h"],
                                   p["dilation_w"], p["groups"], 0, None)
        from tracea_amd.ops import _view
        vx, vw, vo = _view(xv), _view(wv), _view(ov)
        return capi.lib().tracea_conv2d(vx.c, vw.c, None, None, C.byref(vo.c), params)

    assert call(x, w, out) == capi.SUCCESS
    assert call(x, w, out, groups=2) == capi.UNSUPPORTED_CONFIG       # tracea-ffi/src/lib.rs:158-163
    assert call(x, w, out, stride_h=0) == capi.INVALID_PARAMS
    assert call(x[0], w, out) == capi.INVALID_PARAMS                  # rank 3
    assert call(x.float(), w.float(), out) == capi.UNSUPPORTED_CONFIG  # fp32 conv
    assert call(x, w, torch.zeros(1, 7, 8, 8, device="cuda", dtype=torch.float16)) == capi.INVALID_PARAMS
    assert call(x.permute(0, 3, 1, 2).contiguous().permute(0, 2, 3, 1), w, out) == capi.UNSUPPORTED_CONFIG  # NCHW storage
    x12 = torch.zeros(1, 8, 8, 12, device="cuda", dtype=torch.float16)
    w12 = torch.zeros(8, 3, 3, 12, device="cuda", dtype=torch.float16)
    assert call(x12, w12, out) == capi.SUCCESS                        # C % 8 != 0: from padded copies (next test)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_channels_that_are_no_multiple_of_8_run_from_padded_copies(tracea_gpu, dtype):
    """An RGB first layer (3 channels, 7x7 stride 2), 12 channels, [R,S,C,K] filters with a ragged K, operands that do
    not start on 16 bytes: copied with the channels padded to 8 and run by the tile kernels; the reference's kernel
    reads such channels element by element (src/emitter/cuda/conv.rs:228-240)."""
    from tracea_amd import capi
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    rnd = round_f16 if dtype == "f16" else round_bf16
    cases = [(2, 40, 36, 3, 64, 7, 7, 2, 3, "krsc"), (3, 9, 11, 12, 20, 3, 3, 1, 1, "krsc"), (1, 10, 10, 5, 13, 3, 1, 1, 0, "rsck"),
             (2, 8, 8, 16, 12, 3, 3, 1, 1, "rsck"), (1, 6, 7, 1, 8, 1, 1, 1, 0, "krsc")]
    for (n, h, w, c, k, r, s, stride, pad, layout) in cases:
        rng = np.random.default_rng(n + 10 * c + k)
        x = rnd(rng.standard_normal((n, h, w, c)))
        w_rsck = rnd(rng.standard_normal((r, s, c, k)) * np.sqrt(2.0 / (r * s * c)))
        bias = (rng.standard_normal(k) * 0.1).astype(np.float32)
        want = oracle.epilogue_apply(oracle.conv2d_nhwc(x, w_rsck, stride, pad, 1), [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,)])
        dx = _dev(x, tdt)
        dw = _dev(w_rsck, tdt)
        if layout == "krsc":
            dw = dw.permute(3, 0, 1, 2).contiguous()
        y = tracea_gpu.conv2d(dx, dw, bias=_dev(bias), stride=stride, padding=pad, epilogue="bias+relu",
                              weight_layout=layout)
        assert_close_scaled(y.float().cpu().numpy(), want, tol_for_k(r * s * c) if dtype == "f16" else tol_half(r * s * c, "bf16"),
                            "%s %s" % (dtype, (n, h, w, c, k, r, s, stride, pad, layout)))
    # an activation tensor that does not start on 16 bytes
    n, h, w, c, k = 1, 9, 9, 16, 8
    rng = np.random.default_rng(5)
    x = rnd(rng.standard_normal((n, h, w, c)))
    w_rsck = rnd(rng.standard_normal((3, 3, c, k)) * np.sqrt(2.0 / (9 * c)))
    buf = torch.zeros(n * h * w * c + 1, device="cuda", dtype=tdt)
    xv = buf[1:].view(n, h, w, c)
    xv.copy_(_dev(x, tdt))
    y = tracea_gpu.conv2d(xv, _dev(w_rsck, tdt).permute(3, 0, 1, 2).contiguous(), stride=1, padding=1)
    assert_close_scaled(y.float().cpu().numpy(), oracle.conv2d_nhwc(x, w_rsck, 1, 1, 1),
                        tol_for_k(9 * c) if dtype == "f16" else tol_half(9 * c, "bf16"), "unaligned x")


@pytest.mark.parametrize("seed", [11, 12])
def test_random_geometry_on_the_patch_in_lds_members(tracea_gpu, seed):
    """Seeded random geometry (sizes, filter extents, strides, padding, dilation, batch, filter count, operand
    type, chain) on every 16x16x32 member that keeps the input patch in LDS, forced where its plan takes the
    shape, against torch's fp32 convolution of the same half-precision operands."""
    from tracea_amd import capi
    rng = np.random.default_rng(seed)
    names = capi.variants("conv2d")
    ran = {}
    for _ in range(60):
        c = int(rng.choice([8, 64, 128, 256, 512]))
        fr = int(rng.choice([1, 3, 3, 3, 5]))
        fs = fr if rng.random() < 0.8 else int(rng.choice([1, 3, 5]))
        stride = (int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))) if rng.random() < 0.3 else int(rng.choice([1, 1, 1, 2]))
        dil = int(rng.choice([1, 1, 1, 2]))
        if c == 8:
            fr, fs, dil = 7, int(rng.choice([7, 5, 8])), 1
            stride = int(rng.choice([2, 4])) if isinstance(stride, int) else (stride[0] + 1, 2 * stride[1])
        pad = (int(rng.integers(0, 4)), int(rng.integers(0, 4))) if rng.random() < 0.3 else int(rng.integers(0, 3))
        n = int(rng.choice([1, 2, 4, 8, 16]))
        h, w = (int(rng.integers(20, 90)), int(rng.integers(20, 90))) if c == 8 else (int(rng.integers(5, 30)), int(rng.integers(5, 30)))
        k = int(rng.choice([64, 128, 40, 72]))
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        if h + 2 * ph < dil * (fr - 1) + 1 or w + 2 * pw < dil * (fs - 1) + 1:
            continue
        tdt = torch.float16 if rng.random() < 0.7 else torch.bfloat16
        epi = str(rng.choice(["bias+relu", "none", "bias"]))
        x = torch.randn(n, h, w, c, device="cuda").to(tdt)
        wt = (torch.randn(k, fr, fs, c, device="cuda") * (2.0 / (fr * fs * c)) ** 0.5).to(tdt)
        bias = torch.randn(k, device="cuda") * 0.1
        ref = torch.nn.functional.conv2d(x.float().permute(0, 3, 1, 2), wt.float().permute(0, 3, 1, 2),
                                         bias=bias if "bias" in epi else None, stride=stride, padding=pad, dilation=dil)
        ref = (torch.relu(ref) if "relu" in epi else ref).permute(0, 2, 3, 1).cpu().numpy()
        for member in [nm for nm in names if ("_c%d_" % c) in nm and "_w16_" in nm]:
            capi.force_variant("conv2d", member)
            try:
                y = tracea_gpu.conv2d(x, wt, bias=bias if "bias" in epi else None, stride=stride, padding=pad, dilation=dil,
                                      epilogue=epi)
            finally:
                capi.force_variant("conv2d", -1)
            if capi.last_variant("conv2d") != member:
                continue  # (its plan does not take the shape: another kernel ran, tested elsewhere)
            ran[member] = ran.get(member, 0) + 1
            assert_close_scaled(y.float().cpu().numpy(), ref, tol_half(fr * fs * c, "f16" if tdt == torch.float16 else "bf16"),
                                "%s %s" % (member, (n, h, w, c, k, fr, fs, stride, pad, dil, epi)))
    assert len(ran) >= 5 and sum(ran.values()) >= 40, ran
