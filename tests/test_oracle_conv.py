"""Pins the convolution oracle: coordinate tables by brute force, values by
special cases with textbook answers and by torch's conv2d as an independent
library routine (recipe of examples/jit_conv_verify.py:23-26)."""
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

SHAPES = [  # n, h, w, c, k, r, s, stride, pad, dilation
    (2, 8, 8, 32, 32, 3, 3, 1, 1, 1),   # examples/verify_conv2d.rs:52-60 (batch 2)
    (1, 7, 9, 8, 16, 3, 3, 2, 1, 1),
    (2, 6, 6, 16, 8, 1, 1, 2, 0, 1),
    (1, 9, 9, 8, 8, 3, 3, 1, 2, 2),
    (1, 5, 6, 24, 40, 5, 3, 1, 2, 1),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_coordinate_tables_match_brute_force(shape):
    n, h, w, c, k, r, s, stride, pad, dil = shape
    p = oracle.conv_params(n, h, w, c, k, r, s, stride, pad, dil)
    ho = (h + 2 * pad - dil * (r - 1) - 1) // stride + 1
    wo = (w + 2 * pad - dil * (s - 1) - 1) // stride + 1
    assert (p.h_out, p.w_out) == (ho, wo)
    rows, base, cols = oracle.conv_coords(p)
    m = 0
    for bn in range(n):
        for y in range(ho):
            for x in range(wo):
                assert tuple(rows[m]) == (bn, y, x)
                assert base[m] == bn * h * w * c
                m += 1
    assert m == rows.shape[0]
    kk = 0
    for rf in range(r):
        for sf in range(s):
            for ci in range(c):
                assert tuple(cols[kk]) == (rf, sf, ci)
                kk += 1
    assert kk == cols.shape[0]


def test_params_block_layout_is_80_bytes():
    import ctypes
    assert ctypes.sizeof(oracle.ConvParams) == 80
    p = oracle.conv_params(32, 56, 56, 64, 64, 3, 3, 1, 1, 1)
    assert (p.batch, p.h_in, p.w_in, p.c_in, p.k_out, p.h_out, p.w_out, p.r_sz, p.s_sz,
            p.stride, p.pad, p.dilation) == (32, 56, 56, 64, 64, 56, 56, 3, 3, 1, 1, 1)
    assert (p.hw_m, p.hw_s) == (-(-(1 << 32) // 3136), 0)
    assert (p.w_m, p.w_s) == (-(-(1 << 32) // 56), 0)
    assert (p.sic_m, p.sic_s) == (-(-(1 << 32) // 192), 0)
    assert (p.c_m, p.c_s) == (0, 6)


def test_all_ones_counts_window_overlap():
    # interior outputs see R*S*C ones, borders fewer: the count of in-bounds taps
    n, h, w, c, k = 1, 6, 7, 8, 4
    x = np.ones((n, h, w, c), np.float32)
    wt = np.ones((3, 3, c, k), np.float32)
    y = oracle.conv2d_nhwc(x, wt, stride=1, pad=1)
    for i in range(h):
        for j in range(w):
            taps = sum(1 for a in (-1, 0, 1) for b in (-1, 0, 1) if 0 <= i + a < h and 0 <= j + b < w)
            assert (y[0, i, j] == taps * c).all()


def test_1x1_is_a_gemm_and_delta_filter_is_a_shift():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 5, 6, 8)).astype(np.float32)
    w1 = rng.standard_normal((1, 1, 8, 12)).astype(np.float32)
    y = oracle.conv2d_nhwc(x, w1)
    ref = x.reshape(-1, 8).astype(np.float64) @ w1.reshape(8, 12).astype(np.float64)
    assert np.abs(y.reshape(-1, 12) - ref).max() < 1e-5
    # filter with a single 1 at tap (r=0,s=2), channel i -> output channel i: y[h,w] = x[h-1,w+1]
    wd = np.zeros((3, 3, 8, 8), np.float32)
    for ch in range(8):
        wd[0, 2, ch, ch] = 1.0
    y = oracle.conv2d_nhwc(x, wd, stride=1, pad=1)
    want = np.zeros_like(x)
    want[:, 1:, :-1, :] = x[:, :-1, 1:, :]
    assert np.array_equal(y, want)
    # stride 2 picks every other output of the stride-1 result
    y1 = oracle.conv2d_nhwc(x, wd, stride=1, pad=1)
    y2 = oracle.conv2d_nhwc(x, wd, stride=2, pad=1)
    assert np.array_equal(y2, y1[:, ::2, ::2, :])


@pytest.mark.parametrize("shape", SHAPES)
def test_matches_torch_conv2d(shape):
    torch = pytest.importorskip("torch")
    n, h, w, c, k, r, s, stride, pad, dil = shape
    rng = np.random.default_rng(hash(shape) % (1 << 31))
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    wt = rng.standard_normal((r, s, c, k)).astype(np.float32)
    y = oracle.conv2d_nhwc(x, wt, stride, pad, dil)
    yt = torch.nn.functional.conv2d(torch.from_numpy(x).permute(0, 3, 1, 2).double(),
                                    torch.from_numpy(wt).permute(3, 2, 0, 1).double(),
                                    stride=stride, padding=pad, dilation=dil).permute(0, 2, 3, 1).numpy()
    assert y.shape == yt.shape
    assert np.abs(y - yt).max() < 1e-4


def test_committed_fixture():
    # vectors written by tests/golden/make_fixtures.py from torch.nn.functional.conv2d (float64)
    d = np.load(os.path.join(GOLDEN, "conv2d_small.npz"))
    y = oracle.conv2d_nhwc(d["x"], d["w_rsck"], int(d["stride"]), int(d["pad"]), int(d["dilation"]))
    assert np.abs(y - d["y"]).max() < 1e-4
