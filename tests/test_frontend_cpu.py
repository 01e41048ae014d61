"""The reference's Python surface without a device: the epilogue string grammar
(src/interface/python.rs:41-87) and the argument checks that precede any launch."""
import pytest

torch = pytest.importorskip("torch")

from tracea_amd import capi
from tracea_amd import tracea_compat as tracea


def test_package_surface():
    # tracea-python/python/tracea/__init__.py:15
    for name in ("ops", "__version__", "patch_conv2d", "TraceaConv2d", "Context"):
        assert hasattr(tracea, name)
    for name in ("gemm", "conv2d", "conv_transpose2d", "attention"):
        assert callable(getattr(tracea.ops, name))


def test_epilogue_grammar():
    b, r = torch.zeros(4), torch.zeros(2, 4)
    assert tracea.parse_epilogue(None) == []
    assert tracea.parse_epilogue("identity") == []
    assert tracea.parse_epilogue("relu") == [(capi.OP_RELU,)]
    assert tracea.parse_epilogue(" Bias + ReLU ", bias=b) == [(capi.OP_BIAS_ADD, b), (capi.OP_RELU,)]
    chain = tracea.parse_epilogue("bias+residual+silu", bias=b, residual=r)
    assert [c[0] for c in chain] == [capi.OP_BIAS_ADD, capi.OP_RESIDUAL_ADD, capi.OP_SILU]
    assert chain[1][1] is r
    assert tracea.parse_epilogue("gelu+identity")[0] == (capi.OP_GELU,)
    # order is the caller's: residual before bias stays that way
    assert [c[0] for c in tracea.parse_epilogue("residual+bias", bias=b, residual=r)] == \
        [capi.OP_RESIDUAL_ADD, capi.OP_BIAS_ADD]


def test_epilogue_grammar_errors():
    with pytest.raises(ValueError, match="no bias argument"):
        tracea.parse_epilogue("bias+relu")
    with pytest.raises(ValueError, match="no reference provided"):
        tracea.parse_epilogue("residual")
    with pytest.raises(ValueError, match="Unknown epilogue op: tanh"):
        tracea.parse_epilogue("relu+tanh")
    with pytest.raises(ValueError, match="at most 4"):
        tracea.parse_epilogue("relu+relu+relu+relu+relu")


def test_functional_ops_check_shapes_before_anything_else():
    with pytest.raises(ValueError, match="Shape mismatch"):
        tracea.ops.gemm(torch.zeros(4, 8), torch.zeros(7, 4))
    with pytest.raises(ValueError, match="Expected NHWC input and KRSC weight"):
        tracea.ops.conv2d(torch.zeros(4, 8, 8), torch.zeros(8, 3, 3, 8))
    with pytest.raises(ValueError, match="Channel mismatch"):
        tracea.ops.conv2d(torch.zeros(1, 8, 8, 8), torch.zeros(8, 3, 3, 16))


def test_module_falls_back_off_the_gpu_and_for_unsupported_configurations():
    # on the CPU every configuration falls back, so the module must equal torch's
    torch.manual_seed(0)
    ref = torch.nn.Conv2d(8, 4, 3, padding=1)
    m = tracea.TraceaConv2d(8, 4, 3, padding=1)
    m.load_state_dict(ref.state_dict())
    x = torch.randn(2, 8, 6, 6)
    assert torch.equal(m(x), ref(x))
    g = tracea.TraceaConv2d(8, 8, 3, groups=2)
    assert not g._tracea_supported(x)
    d = tracea.TraceaConv2d(8, 8, 3, dilation=2)
    assert not d._tracea_supported(x)
    p = tracea.TraceaConv2d(8, 8, 3, padding=1, padding_mode="reflect")
    assert not p._tracea_supported(x)


def test_patch_and_unpatch():
    original = torch.nn.Conv2d
    try:
        tracea.patch_conv2d()
        assert torch.nn.Conv2d is tracea.TraceaConv2d
        assert isinstance(torch.nn.Conv2d(8, 8, 1), original)   # still a Conv2d for isinstance checks
    finally:
        tracea.unpatch_conv2d()
    assert torch.nn.Conv2d is original


def test_operator_arrays_refuse_half_precision_channel_vectors():
    # BatchNorm / scale-shift vectors are read as fp32 by the kernels; model.half() leaves them f16
    from tracea_amd import ops
    v16, v32 = torch.ones(8, dtype=torch.float16), torch.ones(8)
    with pytest.raises(ValueError):
        ops._ops_array([(capi.OP_BATCHNORM, v32, v32, v16, v32, 1e-5)])
    with pytest.raises(ValueError):
        ops._ops_array([(capi.OP_SCALE_SHIFT, v16, v16)])
    arr, keep = ops._ops_array([(capi.OP_SCALE_SHIFT, v32, v32), (capi.OP_BIAS_ADD, v16)])
    assert arr[0].dtype == capi.F32 and arr[1].dtype == capi.F16 and len(keep) == 3
