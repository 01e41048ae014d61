"""Shared helpers of the parity tests."""
import math

import numpy as np


def tol_for_k(k):
    """Tolerance of the half-precision kernels against an fp32/fp64 reference:
    max|err| <= 2e-2 * sqrt(K) / sqrt(1024), applied as err <= tol * max(1, |ref|)."""
    return 2e-2 * math.sqrt(k) / math.sqrt(1024.0)


def tol_half(k, dtype):
    """tol_for_k plus the rounding of the stored result itself (half a unit in the last place,
    relative 2^-8 for bf16 and 2^-11 for f16), which no kernel can go below and which exceeds
    the K-dependent term for very short reductions."""
    return tol_for_k(k) + (2.0 ** -8 if dtype == "bf16" else 2.0 ** -11)


def assert_close_scaled(got, ref, tol, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    err = np.abs(got - ref) / np.maximum(1.0, np.abs(ref))
    worst = float(err.max()) if err.size else 0.0
    assert np.isfinite(got).all(), what + ": non-finite output"
    assert worst <= tol, "%s: max scaled err %.4g > tol %.4g" % (what, worst, tol)
    return worst


def round_f16(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_bf16(x):
    """Round-to-nearest-even float32 -> bfloat16 -> float32, in numpy."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(x.shape)
