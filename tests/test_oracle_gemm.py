"""Pins the CPU GEMM restatements (oracle/tracea_oracle.c) without the reference:
closed forms, the reference's own 16^3 known answer, float64 numpy, the += contract."""
import numpy as np
import pytest

import oracle


def test_all_ones_closed_form_and_accumulate_contract():
    # examples/cpu_bench.rs:88-90 feeds A = B = 1: every C element is K; the
    # kernel accumulates (src/kernels/cpu/gemm.rs:163-171), so a second call gives 2K.
    m = n = k = 256
    a = np.ones((m, k), np.float32)
    b = np.ones((k, n), np.float32)
    c = np.zeros((m, n), np.float32)
    oracle.gemm_cpu_packed(a, b, c)
    assert (c == k).all()
    oracle.gemm_cpu_packed(a, b, c)
    assert (c == 2 * k).all()


def test_reference_known_answer_16cubed():
    # tests/numerical_parity.rs:72-73: A[i] = 0.05 i - 0.4, B[i] = 0.02 i - 0.1.
    # Closed form: C[r,c] = sum_l (0.05(16r+l)-0.4)(0.02(16l+c)-0.1), in exact rationals.
    from fractions import Fraction as F
    m = n = k = 16
    a = (np.arange(m * k, dtype=np.float32) * np.float32(0.05) - np.float32(0.4)).reshape(m, k)
    b = (np.arange(k * n, dtype=np.float32) * np.float32(0.02) - np.float32(0.1)).reshape(k, n)
    exact = np.empty((m, n))
    for r in range(m):
        for c in range(n):
            exact[r, c] = float(sum((F(5, 100) * (16 * r + l) - F(4, 10)) * (F(2, 100) * (16 * l + c) - F(1, 10))
                                    for l in range(k)))
    got = np.zeros((m, n), np.float32)
    oracle.gemm_cpu_packed(a, b, got, mc=16, nc=16, kc=16, mr=4, nthreads=1)
    # the reference accepts 5e-2 against fp32 sgemm; fp32 inputs carry ~1e-6 relative error
    assert np.abs(got - exact).max() < 5e-4
    assert np.abs(oracle.gemm_f64(a, b) - exact).max() < 5e-4


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (100, 48, 70), (6, 16, 1), (131, 160, 517)])
@pytest.mark.parametrize("mr", [4, 6])
def test_packed_matches_float64(shape, mr):
    m, n, k = shape
    rng = np.random.default_rng(1234 + m + mr)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    c = np.zeros((m, n), np.float32)
    oracle.gemm_cpu_packed(a, b, c, mr=mr)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    # fp32 summation of K products of magnitude <= 1: error <= K * eps32 * sum|a||b| bound, loosely
    bound = k * np.finfo(np.float32).eps * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)).max()
    assert np.abs(c - ref).max() <= bound


def test_packed_tilings_agree_up_to_rounding():
    rng = np.random.default_rng(7)
    a = rng.uniform(-1, 1, (192, 300)).astype(np.float32)
    b = rng.uniform(-1, 1, (300, 96)).astype(np.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    for (mc, nc, kc) in [(128, 128, 256), (64, 32, 64), (192, 96, 300), (6, 16, 8)]:
        c = np.zeros((192, 96), np.float32)
        oracle.gemm_cpu_packed(a, b, c, mc=mc, nc=nc, kc=kc, nthreads=3)
        assert np.abs(c - ref).max() < 1e-3


def test_packed_rejects_bad_register_tile():
    a = np.zeros((8, 8), np.float32)
    with pytest.raises(ValueError):
        oracle.gemm_cpu_packed(a, a, a.copy(), mr=5)


def test_gemm_f64_row_and_column_major_b():
    rng = np.random.default_rng(3)
    a = rng.standard_normal((37, 129)).astype(np.float32)
    b = rng.standard_normal((129, 53)).astype(np.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(oracle.gemm_f64(a, b) - ref).max() < 1e-10
    b_colmajor = np.ascontiguousarray(b.T).T  # same values, [N,K] storage
    assert not b_colmajor.flags.c_contiguous
    assert np.abs(oracle.gemm_f64(a, b_colmajor) - ref).max() < 1e-10
    # a transposed B (swapped stride pair) must NOT reproduce the product
    bt = np.ascontiguousarray(rng.standard_normal((129, 129)).astype(np.float32))
    a2 = rng.standard_normal((37, 129)).astype(np.float32)
    assert np.abs(oracle.gemm_f64(a2, bt) - a2.astype(np.float64) @ bt.T.astype(np.float64)).max() > 1.0
