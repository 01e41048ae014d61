"""Split-K launches (few output tiles, long K): same results as the unsplit kernels to the
parity bar, with operator chains applied once after the sum, for both B layouts, K tails
and convolutions; the switch and the report of the split through the C ABI."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_f16, round_bf16, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


@pytest.fixture
def split_switch(tracea_gpu):
    from tracea_amd import capi
    capi.lib().tracea_set_split_k(1)
    yield capi
    capi.lib().tracea_set_split_k(1)


GEMMS = [(49, 512, 4608), (64, 64, 8192), (100, 72, 2056), (8, 1000, 4096), (196, 256, 2304)]


@pytest.mark.parametrize("shape", GEMMS)
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_split_matches_oracle_and_unsplit(tracea_gpu, split_switch, shape, dtype):
    capi = split_switch
    m, n, k = shape
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    rng = np.random.default_rng(m * 7 + k)
    a = rnd(rng.standard_normal((m, k)) / np.sqrt(k))
    bt = rnd(rng.standard_normal((n, k)))
    bias = (rng.standard_normal(n) * 0.2).astype(np.float32)
    res = rnd(rng.standard_normal((m, n)))
    want = oracle.epilogue_apply(oracle.gemm_f64(a, bt.T), [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RESIDUAL_ADD, res),
                                                             (oracle.EPI_RELU,)])
    da, dbt, dbias, dres = _dev(a, tdt), _dev(bt, tdt), _dev(bias), _dev(res, tdt)
    ops = [(capi.OP_BIAS_ADD, dbias), (capi.OP_RESIDUAL_ADD, dres), (capi.OP_RELU,)]
    for b in (dbt.t(), dbt.t().contiguous()):                 # K-contiguous and N-contiguous B
        got = tracea_gpu.gemm_ex(da, b, ops)
        splits = capi.lib().tracea_last_split_k()
        assert splits >= 2, "%s was expected to split" % (shape,)
        assert_close_scaled(got.float().cpu().numpy(), want, tol_half(k, dtype), "split %s x%d" % (shape, splits))
        capi.lib().tracea_set_split_k(0)
        ref = tracea_gpu.gemm_ex(da, b, ops)
        assert capi.lib().tracea_last_split_k() == 1
        capi.lib().tracea_set_split_k(1)
        # the chain runs once, after the sum: split and unsplit differ by accumulation order only
        assert_close_scaled(got.float().cpu().numpy(), ref.float().cpu().numpy(), 2.0 ** (-7 if dtype == "bf16" else -10),
                            "split vs unsplit %s" % (shape,))


def test_every_variant_splits_correctly(tracea_gpu, split_switch):
    capi = split_switch
    m, n, k = 96, 136, 2120                                  # K tail (2120 = 33*64 + 8), N not a tile multiple
    rng = np.random.default_rng(3)
    a = round_f16(rng.standard_normal((m, k)) / np.sqrt(k))
    bt = round_f16(rng.standard_normal((n, k)))
    want = oracle.gemm_f64(a, bt.T)
    da, dbt = _dev(a, torch.float16), _dev(bt, torch.float16)
    names = capi.variants("gemm")
    ran_split = 0
    try:
        for i, nm in enumerate(names):
            capi.force_variant("gemm", i)
            for b in (dbt.t(), dbt.t().contiguous()):
                got = tracea_gpu.gemm(da, b, out_dtype=torch.float32)
                ran_split += capi.lib().tracea_last_split_k() > 1
                assert_close_scaled(got.cpu().numpy(), want, tol_half(k, "f16"), nm)
    finally:
        capi.force_variant("gemm", -1)
    assert ran_split >= len(names)


CONVS = [  # n, h, w, c, k, r, s, stride, pad
    (1, 7, 7, 512, 512, 3, 3, 1, 1),      # the last stage of ResNet-18 at batch 1
    (1, 14, 14, 256, 256, 3, 3, 1, 1),
    (2, 9, 9, 64, 24, 5, 5, 2, 2),
]


@pytest.mark.parametrize("shape", CONVS)
def test_conv_split_matches_oracle(tracea_gpu, split_switch, shape):
    capi = split_switch
    n, h, w, c, k, r, s, stride, pad = shape
    rng = np.random.default_rng(h + c)
    x = round_f16(rng.standard_normal((n, h, w, c)))
    w_rsck = round_f16(rng.standard_normal((r, s, c, k)) * np.sqrt(2.0 / (r * s * c)))
    scale = rng.uniform(0.5, 1.5, k).astype(np.float32)
    shift = (rng.standard_normal(k) * 0.1).astype(np.float32)
    acc = oracle.conv2d_nhwc(x, w_rsck, stride, pad, 1)
    res = round_f16(rng.standard_normal(acc.shape))
    want = oracle.epilogue_apply(acc, [(oracle.EPI_SCALE_SHIFT, scale, shift), (oracle.EPI_RESIDUAL_ADD, res), (oracle.EPI_RELU,)])
    dx = _dev(x, torch.float16)
    ops = [(capi.OP_SCALE_SHIFT, _dev(scale), _dev(shift)), (capi.OP_RESIDUAL_ADD, _dev(res, torch.float16)), (capi.OP_RELU,)]
    for layout, dw in (("rsck", _dev(w_rsck, torch.float16)),
                       ("krsc", _dev(w_rsck, torch.float16).permute(3, 0, 1, 2).contiguous())):
        got = tracea_gpu.conv2d_ex(dx, dw, ops, stride=stride, padding=pad, weight_layout=layout)
        assert capi.lib().tracea_last_split_k() >= 2
        assert_close_scaled(got.float().cpu().numpy(), want, tol_half(r * s * c, "f16"), "%s %s" % (shape, layout))


@pytest.fixture
def launch_switch(split_switch):
    capi = split_switch
    capi.lib().tracea_set_split_k_one_launch(1)
    yield capi
    capi.lib().tracea_set_split_k_one_launch(1)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_one_launch_split_equals_the_two_launch_form_bit_for_bit(tracea_gpu, launch_switch, dtype):
    """The tile's last workgroup sums the partial products in K order, whoever it is: the result is that of
    the reduction kernel bit for bit, on repeated calls (the counters are back at zero after each) and for
    every variant that can take the one-launch form."""
    capi = launch_switch
    tdt, rnd = (torch.float16, round_f16) if dtype == "f16" else (torch.bfloat16, round_bf16)
    one_launch = 0
    # (two, four and four K ranges on the default variants, a K tail, ragged M and N; the last two are split
    # more finely and stay with two launches)
    for (m, n, k) in [(3136, 64, 576), (784, 128, 1152), (512, 512, 1024), (300, 200, 1096), (96, 136, 1096), (49, 512, 4608),
                      (100, 72, 2056)]:
        rng = np.random.default_rng(m + n + k)
        a = _dev(rnd(rng.standard_normal((m, k)) / np.sqrt(k)), tdt)
        bt = _dev(rnd(rng.standard_normal((n, k))), tdt)
        bias = _dev((rng.standard_normal(n) * 0.2).astype(np.float32))
        res = _dev(rnd(rng.standard_normal((m, n))), tdt)
        ops = [(capi.OP_BIAS_ADD, bias), (capi.OP_RESIDUAL_ADD, res), (capi.OP_RELU,)]
        for b in (bt.t(), bt.t().contiguous()):
            capi.lib().tracea_set_split_k_one_launch(0)
            two = tracea_gpu.gemm_ex(a, b, ops)
            assert capi.lib().tracea_last_split_k() >= 2 and capi.lib().tracea_last_split_k_launches() == 2
            capi.lib().tracea_set_split_k_one_launch(1)
            for rep in range(3):
                one = tracea_gpu.gemm_ex(a, b, ops)
                assert capi.lib().tracea_last_split_k() >= 2
                one_launch += capi.lib().tracea_last_split_k_launches() == 1
                assert torch.equal(one, two), "(%d, %d, %d) call %d" % (m, n, k, rep)
    assert one_launch >= 3 * 2 * 3


def test_one_launch_split_on_every_variant_that_takes_it(tracea_gpu, launch_switch):
    capi = launch_switch
    m, n, k = 96, 136, 1096                                  # 18 K tiles of 64 (the last one 8 wide): at most 4 ranges
    rng = np.random.default_rng(5)
    a = _dev(round_f16(rng.standard_normal((m, k)) / np.sqrt(k)), torch.float16)
    bt = _dev(round_f16(rng.standard_normal((n, k))), torch.float16)
    names = capi.variants("gemm")
    took = 0
    try:
        for i, nm in enumerate(names):
            capi.force_variant("gemm", i)
            for b in (bt.t(), bt.t().contiguous()):
                capi.lib().tracea_set_split_k_one_launch(0)
                two = tracea_gpu.gemm(a, b, out_dtype=torch.float32)
                capi.lib().tracea_set_split_k_one_launch(1)
                one = tracea_gpu.gemm(a, b, out_dtype=torch.float32)
                took += capi.lib().tracea_last_split_k_launches() == 1
                assert torch.equal(one, two), nm
    finally:
        capi.force_variant("gemm", -1)
    assert took >= 6


def test_one_launch_conv_split_and_graph_replay(tracea_gpu, launch_switch):
    """ResNet-18's 28x28x128 stage at batch 1 on a streamed variant (784 pixels, K = 1152, four K ranges): one
    kernel, the same bits as two, also when the launch is replayed from a HIP graph with other split launches
    between the replays."""
    capi = launch_switch
    rng = np.random.default_rng(11)
    x = _dev(round_f16(rng.standard_normal((1, 28, 28, 128))), torch.float16)
    w = _dev(round_f16(rng.standard_normal((128, 3, 3, 128)) * np.sqrt(2.0 / 1152)), torch.float16)
    bias = _dev((rng.standard_normal(128) * 0.1).astype(np.float32))
    ops = [(capi.OP_BIAS_ADD, bias), (capi.OP_RELU,)]
    capi.force_variant("conv2d", "t128x64x64_w4x1_p2")
    try:
        _conv_one_and_two_launches(tracea_gpu, capi, x, w, ops)
    finally:
        capi.force_variant("conv2d", -1)


def _conv_one_and_two_launches(tracea_gpu, capi, x, w, ops):
    capi.lib().tracea_set_split_k_one_launch(0)
    two = tracea_gpu.conv2d_ex(x, w, ops, stride=1, padding=1, weight_layout="krsc")
    assert capi.lib().tracea_last_split_k_launches() == 2
    capi.lib().tracea_set_split_k_one_launch(1)
    one = tracea_gpu.conv2d_ex(x, w, ops, stride=1, padding=1, weight_layout="krsc")
    assert capi.lib().tracea_last_split_k() >= 2 and capi.lib().tracea_last_split_k_launches() == 1
    assert torch.equal(one, two)
    out = torch.empty_like(one)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        tracea_gpu.conv2d_ex(x, w, ops, stride=1, padding=1, weight_layout="krsc", out=out)   # buffers of this stream
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        tracea_gpu.conv2d_ex(x, w, ops, stride=1, padding=1, weight_layout="krsc", out=out)
    a = torch.randn(512, 1024, device="cuda").half()
    b = torch.randn(1024, 512, device="cuda").half()
    for rep in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, two), "replay %d" % rep
        tracea_gpu.gemm(a, b)                                 # eager work between the replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(768, 1024, 1024), (512, 512, 1024), (100, 36, 2052), (1536, 1536, 1536)])
def test_fp32_one_launch_split_equals_the_two_launch_form(tracea_gpu, launch_switch, shape):
    """The fp32 GEMM on 64x64 tiles: K ranges summed by the tile's last workgroup or by the reduction kernel,
    the same ranges in the same order, hence the same bits; and the float64 product within 1e-4 sqrt(K)."""
    capi = launch_switch
    m, n, k = shape
    rng = np.random.default_rng(m + n + k)
    a = _dev(rng.uniform(-1, 1, (m, k)).astype(np.float32))
    b = _dev(rng.uniform(-1, 1, (k, n)).astype(np.float32))
    bias = _dev(rng.standard_normal(n).astype(np.float32))
    capi.lib().tracea_set_split_k_one_launch(0)
    two = tracea_gpu.gemm(a, b, bias=bias, epilogue="bias")
    splits = capi.lib().tracea_last_split_k()
    assert splits >= 2 and capi.lib().tracea_last_split_k_launches() == 2
    capi.lib().tracea_set_split_k_one_launch(1)
    for rep in range(3):
        one = tracea_gpu.gemm(a, b, bias=bias, epilogue="bias")
        assert capi.lib().tracea_last_split_k() == splits and capi.lib().tracea_last_split_k_launches() == 1
        assert torch.equal(one, two), "call %d" % rep
    want = a.double().cpu().numpy() @ b.double().cpu().numpy() + bias.double().cpu().numpy()
    np.testing.assert_allclose(one.cpu().numpy(), want, rtol=0, atol=1e-4 * np.sqrt(k))


def test_large_problems_are_not_split(tracea_gpu, split_switch):
    capi = split_switch
    a = torch.randn(2048, 1024, device="cuda").half()
    b = torch.randn(1024, 2048, device="cuda").half()
    tracea_gpu.gemm(a, b)
    assert capi.lib().tracea_last_split_k() == 1            # 64+ tiles already fill the device
    a = torch.randn(64, 256, device="cuda").half()          # few tiles but a short K
    tracea_gpu.gemm(a, torch.randn(256, 64, device="cuda").half())
    assert capi.lib().tracea_last_split_k() == 1


# shapes of few 64x64 tiles and a long K (1024^3 fills the device with 256 such tiles and is not split)
@pytest.mark.parametrize("shape", [(512, 512, 1024), (256, 256, 4096), (100, 36, 2052)])
def test_fp32_gemm_split_matches_float64(tracea_gpu, split_switch, shape):
    capi = split_switch
    m, n, k = shape
    rng = np.random.default_rng(m + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64) + bias
    got = tracea_gpu.gemm(_dev(a), _dev(b), bias=_dev(bias), epilogue="bias")
    assert capi.lib().tracea_last_split_k() >= 2
    assert got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=0, atol=1e-4 * np.sqrt(k))
