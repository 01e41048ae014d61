"""The reference's Python surface on the device, checked the way its own scripts check it:
against torch on the same tensors (examples/jit_conv_verify.py:23-26, tests/python/
fa2_verification.py) and against the CPU oracle."""
import math

import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture
def tracea(tracea_gpu):
    from tracea_amd import tracea_compat
    return tracea_compat


def test_ops_gemm_row_major_with_epilogue_string(tracea):
    g = torch.Generator(device="cuda").manual_seed(0)
    x = (torch.randn(256, 128, device="cuda", generator=g) / math.sqrt(128)).half()
    w = torch.randn(128, 192, device="cuda", generator=g).half()       # [K,N] row-major, as ops.py:12-37
    bias = torch.randn(192, device="cuda", generator=g)
    y = tracea.ops.gemm(x, w, bias=bias, epilogue="bias+relu")
    want = oracle.epilogue_apply(oracle.gemm_f64(x.float().cpu().numpy(), w.float().cpu().numpy()),
                                 [(oracle.EPI_BIAS_ADD, bias.cpu().numpy()), (oracle.EPI_RELU,)])
    assert y.dtype == torch.float16 and tuple(y.shape) == (256, 192)
    assert_close_scaled(y.float().cpu().numpy(), want, tol_half(128, "f16"), "ops.gemm")


def test_ops_conv2d_chain_in_the_callers_order(tracea):
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(2, 10, 10, 16, device="cuda", generator=g).half()
    w = (torch.randn(24, 3, 3, 16, device="cuda", generator=g) / 12).half()
    bias = torch.randn(24, device="cuda", generator=g)
    res = torch.randn(2, 10, 10, 24, device="cuda", generator=g).half()
    y = tracea.ops.conv2d(x, w, bias=bias, residual=res, epilogue="bias+residual+relu", stride=1, padding=1)
    acc = oracle.conv2d_nhwc(x.float().cpu().numpy(), w.permute(1, 2, 3, 0).float().cpu().numpy(), 1, 1, 1)
    want = oracle.epilogue_apply(acc, [(oracle.EPI_BIAS_ADD, bias.cpu().numpy()),
                                       (oracle.EPI_RESIDUAL_ADD, res.float().cpu().numpy()), (oracle.EPI_RELU,)])
    assert_close_scaled(y.float().cpu().numpy(), want, tol_half(144, "f16"), "ops.conv2d")


def test_ops_conv_transpose2d_reference_storage(tracea):
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.rand(1, 8, 8, 16, device="cuda", generator=g) * 2 - 1
    w_crsk = torch.rand(16, 4, 4, 8, device="cuda", generator=g) - 0.5     # the kernel's [C*R*S, K] rows
    w = w_crsk.permute(3, 1, 2, 0)                                         # dims [K,R,S,C] as python.rs:465 reads
    y = tracea.ops.conv_transpose2d(x, w, stride=2, padding=1)
    want = oracle.conv_transpose2d_nhwc(x.cpu().numpy(), w_crsk.cpu().numpy(), 2, 1)
    assert tuple(y.shape) == want.shape
    assert np.abs(y.cpu().numpy() - want).max() < 1e-4


def test_ops_attention_is_causal_by_default(tracea):
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = [torch.randn(1, 2, 256, 64, device="cuda", generator=g).half() for _ in range(3)]
    o = tracea.ops.attention(q, k, v)
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert torch.allclose(o.float(), want, atol=2e-2, rtol=0)
    o2 = tracea.ops.attention(q, k, v, causal=False)
    want2 = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert torch.allclose(o2.float(), want2, atol=2e-2, rtol=0)


def test_context_methods_write_the_callers_output_and_check_shapes(tracea):
    ctx = tracea.Context()
    a = torch.randn(64, 32, device="cuda").half()
    b = torch.randn(32, 48, device="cuda").half()
    c = torch.zeros(64, 48, device="cuda", dtype=torch.float16)
    kid = ctx.gemm(a, b, c, 64, 48, 32)
    ctx.synchronize()
    assert isinstance(kid, int)
    assert torch.allclose(c.float(), a.float() @ b.float(), atol=5e-2, rtol=0)
    with pytest.raises(ValueError, match="arguments say"):
        ctx.gemm(a, b, c, 64, 48, 16)
    q = torch.randn(1, 1, 128, 64, device="cuda").half()
    o = torch.empty_like(q)
    # conv_transpose2d returns the kernel that ran: a convolution variant when the call went out by phase
    xt = torch.randn(1, 8, 8, 16, device="cuda").half()
    wt = torch.randn(16, 4, 4, 16, device="cuda").half() * 0.1
    ot = torch.zeros(1, 16, 16, 16, device="cuda", dtype=torch.float16)
    from tracea_amd import capi
    kid_t = ctx.conv_transpose2d(xt, wt, ot, 1, 16, 8, 8, 16, 4, 4, stride=2, pad=1)
    assert kid_t >= 0 and capi.variants("conv2d")[kid_t] == capi.last_variant("conv2d") and capi.last_variant("gemm") is None
    ctx.attention(q, q, q, o, 1, 1, 128, 64, 64, causal=False, scale_sqrt=False)
    want = torch.softmax(q[0, 0].float() @ q[0, 0].float().t(), dim=-1) @ q[0, 0].float()
    assert torch.allclose(o[0, 0].float(), want, atol=2e-2, rtol=0)


def test_module_matches_torch_and_falls_back(tracea):
    torch.manual_seed(4)
    ref = torch.nn.Conv2d(16, 32, 3, stride=2, padding=1).cuda().half()
    m = tracea.TraceaConv2d(16, 32, 3, stride=2, padding=1).cuda().half()
    m.load_state_dict(ref.state_dict())
    x = torch.randn(2, 16, 14, 14, device="cuda").half()
    from tracea_amd import capi
    capi.lib().tracea_force_variant(b"conv2d", -1)
    with torch.no_grad():
        y = m(x)
        assert capi.last_variant("conv2d") is not None          # the library ran, not torch
        assert y.grad_fn is None and tuple(y.shape) == tuple(ref(x).shape)
        assert torch.allclose(y.float(), ref(x).float(), atol=3e-2, rtol=0)
        # a changed weight is picked up (the repacked copy is per weight version)
        m.weight.mul_(2.0)
        ref.weight.mul_(2.0)
        assert torch.allclose(m(x).float(), ref(x).float(), atol=6e-2, rtol=0)
    # a step that needs gradients goes through PyTorch: the kernels here are forward only
    yg = m(x)
    assert yg.grad_fn is not None
    yg.float().sum().backward()
    assert m.weight.grad is not None and torch.isfinite(m.weight.grad.float()).all()
    # fp32 modules and grouped convolutions take torch's path and agree exactly
    ref32 = torch.nn.Conv2d(16, 32, 3, padding=1, groups=2).cuda()
    m32 = tracea.TraceaConv2d(16, 32, 3, padding=1, groups=2).cuda()
    m32.load_state_dict(ref32.state_dict())
    x32 = torch.randn(1, 16, 8, 8, device="cuda")
    assert torch.equal(m32(x32), ref32(x32))


def test_patch_conv2d_builds_tracea_modules(tracea):
    try:
        tracea.patch_conv2d()
        layer = torch.nn.Conv2d(8, 8, 3, padding=1).cuda().half()
        assert isinstance(layer, tracea.TraceaConv2d)
        x = torch.randn(1, 8, 12, 12, device="cuda").half()
        with torch.no_grad():
            y = layer(x)
    finally:
        tracea.unpatch_conv2d()
    ref = torch.nn.functional.conv2d(x.float(), layer.weight.float(), layer.bias.float(), padding=1)
    assert torch.allclose(y.float(), ref, atol=3e-2, rtol=0)
