"""The operators that are not contractions (softmax, standalone BatchNorm / ReLU / Add, global
average pooling, batched linear) on the GPU through the C ABI, against float64 numpy and against
torch's CPU routines for the same operators as an independent library.  Arithmetic is fp32 on the
device: fp32 storage is held to 2e-6 (softmax, pooling) / 1e-5 (BatchNorm) scaled by max(1,|ref|),
half storage to its output rounding (2^-11 f16, 2^-8 bf16) on top."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_bf16, round_f16, tol_half

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tracea_amd import capi  # noqa: E402

TYPES = {"f32": (torch.float32, lambda v: np.asarray(v, dtype=np.float32), 0.0),
         "f16": (torch.float16, round_f16, 2.0 ** -11), "bf16": (torch.bfloat16, round_bf16, 2.0 ** -8)}


def _dev(a, tdt):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda().to(tdt)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(7, 1000), (4, 3, 5), (1, 1), (130, 64), (3, 5000)])
def test_softmax_last_axis(tracea_gpu, dtype, shape):
    tdt, rnd, ulp = TYPES[dtype]
    rng = np.random.default_rng(sum(shape))
    x = rnd(rng.standard_normal(shape) * 4)
    got = tracea_gpu.softmax(_dev(x, tdt)).float().cpu().numpy()
    e = np.exp(x.astype(np.float64) - x.max(axis=-1, keepdims=True))
    ref = e / e.sum(axis=-1, keepdims=True)
    assert_close_scaled(got, ref, 2e-6 + ulp, "softmax")
    lib = torch.softmax(torch.from_numpy(x).double(), dim=-1).numpy()
    assert_close_scaled(got, lib, 2e-6 + ulp, "softmax against torch")
    if dtype == "f32":
        np.testing.assert_allclose(got.sum(axis=-1), 1.0, atol=1e-5)


def test_softmax_is_shift_invariant_and_survives_large_inputs(tracea_gpu):
    x = torch.tensor([[1000.0, 1001.0, 999.0, -1e30]], device="cuda")
    got = tracea_gpu.softmax(x).cpu().numpy()
    ref = np.exp(np.array([0.0, 1.0, -1.0])) / np.exp(np.array([0.0, 1.0, -1.0])).sum()
    np.testing.assert_allclose(got[0, :3], ref, rtol=1e-6)
    assert got[0, 3] == 0.0


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 5, 6, 64), (3, 7, 7, 20), (1, 1, 1, 8), (50, 33)])
def test_standalone_batchnorm(tracea_gpu, dtype, shape):
    # (x - mean) * rsqrt(var + eps) * gamma + beta per channel (src/emitter/cuda/nn.rs:56-66)
    tdt, rnd, ulp = TYPES[dtype]
    c = shape[-1]
    rng = np.random.default_rng(c)
    x = rnd(rng.standard_normal(shape))
    gamma, beta = rng.uniform(0.5, 1.5, c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
    mean, var = rng.standard_normal(c).astype(np.float32), rng.uniform(0.5, 2.0, c).astype(np.float32)
    g = lambda v: torch.from_numpy(v).cuda()
    got = tracea_gpu.batchnorm(_dev(x, tdt), g(gamma), g(beta), g(mean), g(var), 1e-5).float().cpu().numpy()
    ref = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-5) * gamma + beta
    assert_close_scaled(got, ref, 1e-5 + ulp, "batchnorm")
    if len(shape) == 4:
        t = torch.from_numpy(x).double().permute(0, 3, 1, 2)
        lib = torch.nn.functional.batch_norm(t, torch.from_numpy(mean).double(), torch.from_numpy(var).double(),
                                             torch.from_numpy(gamma).double(), torch.from_numpy(beta).double(),
                                             False, 0.0, 1e-5).permute(0, 2, 3, 1).numpy()
        assert_close_scaled(got, lib, 1e-5 + ulp, "batchnorm against torch")


def test_relu_and_add_as_one_pass(tracea_gpu):
    rng = np.random.default_rng(1)
    x = round_f16(rng.standard_normal((4, 9, 9, 24)))
    y = round_f16(rng.standard_normal((4, 9, 9, 24)))
    dx, dy = _dev(x, torch.float16), _dev(y, torch.float16)
    got = tracea_gpu.apply_epilogue(dx, [(capi.OP_RESIDUAL_ADD, dy), (capi.OP_RELU,)])
    ref = round_f16(np.maximum(x + y, 0.0))
    np.testing.assert_array_equal(got.float().cpu().numpy(), ref)  # one rounding of an exact fp32 sum
    # in place
    tracea_gpu.apply_epilogue(dx, [(capi.OP_RELU,)], out=dx)
    np.testing.assert_array_equal(dx.float().cpu().numpy(), np.maximum(x, 0.0))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 7, 7, 512), (3, 5, 4, 70), (1, 1, 1, 1), (4, 56, 56, 64)])
def test_global_avg_pool(tracea_gpu, dtype, shape):
    tdt, rnd, ulp = TYPES[dtype]
    rng = np.random.default_rng(shape[1] * shape[3])
    x = rnd(rng.standard_normal(shape) + 0.5)
    got = tracea_gpu.global_avg_pool(_dev(x, tdt)).float().cpu().numpy()
    ref = x.astype(np.float64).mean(axis=(1, 2))
    assert got.shape == (shape[0], shape[3])
    assert_close_scaled(got, ref, 3e-6 + ulp, "global average pool")
    lib = torch.nn.functional.adaptive_avg_pool2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), 1)[:, :, 0, 0].numpy()
    assert_close_scaled(got, lib, 3e-6 + ulp, "global average pool against torch")


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("batched_w", [True, False])
def test_linear_batched(tracea_gpu, dtype, batched_w):
    # src/emitter/cuda/nn.rs:113-131: C[b] = A[b] B[b]; a shared weight folds the batch into the rows
    tdt, rnd, _ = TYPES[dtype]
    b, m, k, n = 3, 50, 136, 72
    rng = np.random.default_rng(7)
    a = rnd(rng.standard_normal((b, m, k)) / np.sqrt(k))
    w = rnd(rng.standard_normal((b, k, n) if batched_w else (k, n)))
    bias = rng.standard_normal(n).astype(np.float32)
    got = tracea_gpu.linear(_dev(a, tdt), _dev(w, tdt), bias=torch.from_numpy(bias).cuda(), epilogue="bias+relu",
                            out_dtype=torch.float32).cpu().numpy()
    for i in range(b):
        ref = np.maximum(oracle.gemm_f64(a[i], w[i] if batched_w else w) + bias[None, :], 0.0)
        tol = 1e-4 if dtype == "f32" else tol_half(k, dtype)
        assert_close_scaled(got[i], ref, tol, "linear batch %d" % i)
    if not batched_w:
        assert capi.last_variant("gemm") is not None or dtype == "f32"
    # a strided batch (every other matrix of a larger buffer) goes batch by batch
    big = _dev(np.repeat(a, 2, axis=0), tdt)
    got2 = tracea_gpu.linear(big[::2], _dev(w, tdt), out_dtype=torch.float32).cpu().numpy()
    for i in range(b):
        ref = oracle.gemm_f64(a[i], w[i] if batched_w else w)
        assert_close_scaled(got2[i], ref, 1e-4 if dtype == "f32" else tol_half(k, dtype), "strided batch %d" % i)


def test_bad_arguments(tracea_gpu):
    x = torch.zeros(2, 8, 4, 4, device="cuda").permute(0, 2, 3, 1)  # NHWC view of NCHW storage
    with pytest.raises(capi.TraceaError, match="channel axis last"):
        tracea_gpu.softmax(x)
    with pytest.raises(capi.TraceaError, match="channel axis last"):
        tracea_gpu.global_avg_pool(x)
    y = torch.zeros(2, 4, 4, 8, device="cuda")
    with pytest.raises(capi.TraceaError, match="differ in shape"):
        tracea_gpu.softmax(y, out=torch.zeros(2, 4, 4, 4, device="cuda"))
    with pytest.raises(capi.TraceaError, match=r"expected \[2,8\]"):
        tracea_gpu.global_avg_pool(y, out=torch.zeros(2, 4, device="cuda"))
    with pytest.raises(capi.TraceaError, match="BatchNorm needs"):
        tracea_gpu.apply_epilogue(y, [(capi.OP_BATCHNORM, torch.zeros(8, device="cuda"))])
    with pytest.raises(capi.TraceaError, match="do not agree"):
        tracea_gpu.linear(torch.zeros(2, 4, 8, device="cuda"), torch.zeros(3, 8, 8, device="cuda"))
    with pytest.raises(capi.TraceaError, match="residual"):
        tracea_gpu.linear(torch.zeros(2, 4, 8, device="cuda"), torch.zeros(8, 8, device="cuda"), epilogue="residual")
