"""Pins the epilogue functors and the magic-number division of the oracle."""
import math

import numpy as np
import pytest

import oracle


def _apply1(kind, x, *extra):
    return oracle.epilogue_apply(np.array([x], np.float32).reshape(1, -1), [(kind,) + extra])[0]


def test_scalar_functors_closed_form():
    # src/kernels/gpu/epilogue.cuh:12-63
    xs = np.array([-20.0, -3.0, -1.0, -0.0, 0.0, 0.5, 1.0, 3.0, 20.0], np.float32)
    relu = oracle.epilogue_apply(xs.reshape(1, -1), [(oracle.EPI_RELU,)])[0]
    assert (relu == np.maximum(xs, 0)).all()
    silu = oracle.epilogue_apply(xs.reshape(1, -1), [(oracle.EPI_SILU,)])[0]
    want = np.array([x / (1.0 + math.exp(-x)) for x in xs.astype(np.float64)])
    assert np.abs(silu - want).max() < 1e-6
    gelu = oracle.epilogue_apply(xs.reshape(1, -1), [(oracle.EPI_GELU,)])[0]
    want = np.array([0.5 * x * (1.0 + math.tanh(0.79788456 * (x + 0.044715 * x ** 3))) for x in xs.astype(np.float64)])
    assert np.abs(gelu - want).max() < 2e-6
    # limits: SiLU(-20) ~ -4e-8, SiLU(20) ~ 20, GELU(-20) = 0, GELU(20) = 20
    assert abs(silu[0]) < 1e-6 and abs(silu[-1] - 20) < 1e-5
    assert gelu[0] == 0 and gelu[-1] == 20


def test_bias_residual_indexing_and_order():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 7)).astype(np.float32)
    bias = rng.standard_normal(7).astype(np.float32)
    res = rng.standard_normal((5, 7)).astype(np.float32)
    got = oracle.epilogue_apply(x, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RELU,), (oracle.EPI_RESIDUAL_ADD, res)])
    assert np.array_equal(got, np.maximum(x + bias[None, :], 0) + res)
    # order matters: relu after the residual differs
    got2 = oracle.epilogue_apply(x, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_RESIDUAL_ADD, res), (oracle.EPI_RELU,)])
    assert np.array_equal(got2, np.maximum(x + bias[None, :] + res, 0))
    assert not np.array_equal(got, got2)
    fused = oracle.epilogue_apply(x, [(oracle.EPI_BIAS_ADD_SILU, bias)])
    two = oracle.epilogue_apply(x, [(oracle.EPI_BIAS_ADD, bias), (oracle.EPI_SILU,)])
    assert np.array_equal(fused, two)


def test_batchnorm_formula_and_folded_identity():
    # src/emitter/metal/utils.rs:56-73: (v-mean)*rsqrt(var+eps)*gamma+beta
    rng = np.random.default_rng(1)
    x = rng.standard_normal((9, 16)).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, 16).astype(np.float32)
    beta = (rng.standard_normal(16) * 0.1).astype(np.float32)
    mean = (rng.standard_normal(16) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, 16).astype(np.float32)
    eps = 1e-5
    got = oracle.epilogue_apply(x, [(oracle.EPI_BATCHNORM, gamma, beta, mean, var, eps)])
    want = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + eps) * gamma + beta
    assert np.abs(got - want).max() < 2e-6
    scale = (gamma.astype(np.float64) / np.sqrt(var.astype(np.float64) + eps)).astype(np.float32)
    shift = (beta.astype(np.float64) - mean.astype(np.float64) * scale).astype(np.float32)
    folded = oracle.epilogue_apply(x, [(oracle.EPI_SCALE_SHIFT, scale, shift)])
    assert np.abs(folded - want).max() < 2e-6
    # gamma=1, beta=0, mean=0, var=1-eps is the identity
    ident = oracle.epilogue_apply(x, [(oracle.EPI_BATCHNORM, np.ones(16, np.float32), np.zeros(16, np.float32),
                                      np.zeros(16, np.float32), np.full(16, 1 - eps, np.float32), eps)])
    assert np.abs(ident - x).max() < 1e-6


def test_magic_u32_values():
    # src/emitter/cuda/conv.rs:6-16: n<=1 -> (0,0); power of two -> (0, log2); else (ceil(2^p/n), p)
    assert oracle.magic_u32(0) == (0, 0)
    assert oracle.magic_u32(1) == (0, 0)
    assert oracle.magic_u32(2) == (0, 1)
    assert oracle.magic_u32(64) == (0, 6)
    assert oracle.magic_u32(1 << 20) == (0, 20)
    for d in (3, 7, 28, 56, 192, 384, 576, 784, 3136):
        m, p = oracle.magic_u32(d)
        assert p == 32 and m == -(-(1 << 32) // d), (d, m, p)


@pytest.mark.parametrize("d", [1, 2, 3, 7, 28, 56, 64, 128, 192, 384, 576, 784, 3136])
def test_fast_divmod_exhaustive(d):
    # every divisor the configurations use, every dividend below 2^20
    # (largest real dividend: 100352 rows of the N=32 56x56 convolution)
    assert oracle.divmod_check(d, 1 << 20) == -1


def test_fast_divmod_spot_values():
    m, p = oracle.magic_u32(3136)
    for n in (0, 1, 3135, 3136, 3137, 100351):
        assert oracle.fast_divmod(n, m, p - 32, 3136) == divmod(n, 3136)
    assert oracle.fast_divmod(77, 0, 6, 64) == (1, 13)
    assert oracle.fast_divmod(77, 0, 0, 1) == (77, 0)
