"""Pins the transposed-convolution oracle: the reference's own scatter-form CPU
statement (examples/verify_conv_transpose.rs:12-54) restated as brute force,
special cases with closed answers, the adjoint identity that ties it to the
already pinned convolution oracle, and torch's conv_transpose2d as an
independent library routine."""
import numpy as np
import pytest

import oracle

SHAPES = [  # n, h, w, c, k, r, s, stride, pad, output_padding
    (1, 2, 2, 1, 1, 2, 2, 1, 0, 0),     # examples/verify_conv_transpose.rs:66-69, the minimal case
    (2, 4, 5, 3, 4, 3, 3, 2, 1, 1),
    (1, 5, 4, 2, 3, 4, 4, 2, 1, 0),     # 4x4 stride 2 pad 1: the VAE decoder layer, small
    (1, 3, 3, 2, 2, 2, 2, 3, 0, 1),     # stride larger than the filter: some outputs get no tap
    (2, 4, 4, 4, 2, 3, 2, (2, 1), (0, 1), (1, 0)),
    (1, 6, 5, 2, 2, 5, 3, (3, 2), (2, 1), (2, 1)),
]


def scatter_reference(x, w, stride, pad, output_padding):
    """The reference's loop nest: every input pixel scatters through every tap."""
    n, h, wd, c = x.shape
    _, r, s, k = w.shape
    sh, sw = oracle._pair(stride)
    ph, pw = oracle._pair(pad)
    ho, wo = oracle.conv_transpose_out_shape(h, wd, r, s, stride, pad, output_padding)
    y = np.zeros((n, ho, wo, k), dtype=np.float64)
    for b in range(n):
        for hi in range(h):
            for wi in range(wd):
                for rr in range(r):
                    for ss in range(s):
                        oh, ow = hi * sh - ph + rr, wi * sw - pw + ss
                        if 0 <= oh < ho and 0 <= ow < wo:
                            y[b, oh, ow, :] += x[b, hi, wi, :].astype(np.float64) @ w[:, rr, ss, :].astype(np.float64)
    return y


@pytest.mark.parametrize("shape", SHAPES)
def test_gather_form_equals_the_reference_scatter_form(shape):
    n, h, w, c, k, r, s, stride, pad, opad = shape
    rng = np.random.default_rng(hash(shape[:7]) & 0xffff)
    x = rng.uniform(-1, 1, (n, h, w, c)).astype(np.float32)       # verify_conv_transpose.rs:89
    wt = rng.uniform(-0.5, 0.5, (c, r, s, k)).astype(np.float32)  # verify_conv_transpose.rs:94
    got = oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad)
    want = scatter_reference(x, wt, stride, pad, opad)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-6)


def test_minimal_case_by_hand():
    # 2x2 input, one channel, 2x2 filter, stride 1: the full 2-D polynomial product
    x = np.array([[1.0, 2.0], [3.0, 4.0]], dtype=np.float32).reshape(1, 2, 2, 1)
    w = np.array([[10.0, 20.0], [30.0, 40.0]], dtype=np.float32).reshape(1, 2, 2, 1)
    y = oracle.conv_transpose2d_nhwc(x, w)[0, :, :, 0]
    want = np.array([[10, 40, 40], [60, 200, 160], [90, 240, 160]], dtype=np.float32)
    np.testing.assert_array_equal(y, want)


def test_all_ones_counts_contributing_taps():
    # x = 1, w = 0.1 (the debugging values of verify_conv_transpose.rs:91,96):
    # each output holds 0.1 * C * (number of (r, s) taps that reach an input pixel)
    n, h, w, c, k, r, s, stride, pad = 1, 4, 4, 3, 2, 4, 4, 2, 1
    x = np.ones((n, h, w, c), dtype=np.float32)
    wt = np.full((c, r, s, k), 0.1, dtype=np.float32)
    y = oracle.conv_transpose2d_nhwc(x, wt, stride, pad)
    ho, wo = oracle.conv_transpose_out_shape(h, w, r, s, stride, pad, 0)
    assert y.shape == (n, ho, wo, k) == (1, 8, 8, 2)

    def taps(o, size_in, kernel):
        return sum(1 for t in range(kernel) if (o + pad - t) >= 0 and (o + pad - t) % stride == 0
                   and (o + pad - t) // stride < size_in)
    for oh in range(ho):
        for ow in range(wo):
            want = 0.1 * c * taps(oh, h, r) * taps(ow, w, s)
            assert abs(y[0, oh, ow, 0] - want) < 1e-6
    # 4x4 stride 2 pad 1: interior pixels see 2x2 taps, the outermost ring one fewer per side
    assert taps(0, h, r) == 1 and taps(1, h, r) == 2 and taps(ho - 1, h, r) == 1


def test_stride_larger_than_filter_leaves_untouched_outputs_zero():
    x = np.ones((1, 3, 3, 2), dtype=np.float32)
    wt = np.ones((2, 2, 2, 2), dtype=np.float32)
    y = oracle.conv_transpose2d_nhwc(x, wt, stride=3, pad=0, output_padding=1)
    assert y.shape == (1, 9, 9, 2)
    mask = np.zeros((9, 9), dtype=bool)
    for hi in range(3):
        for wi in range(3):
            mask[hi * 3:hi * 3 + 2, wi * 3:wi * 3 + 2] = True
    np.testing.assert_array_equal(y[0, :, :, 0] != 0, mask)
    np.testing.assert_array_equal(y[0][mask], np.full((int(mask.sum()), 2), 2.0, dtype=np.float32))


def test_stride_one_is_a_convolution_with_the_flipped_filter():
    # convT(x, w; stride 1, pad p) == conv(x, flip(w) with C and K exchanged; pad R-1-p)
    rng = np.random.default_rng(3)
    n, h, w, c, k, r, s, pad = 2, 6, 7, 4, 5, 3, 3, 1
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    wt = rng.standard_normal((c, r, s, k)).astype(np.float32)
    got = oracle.conv_transpose2d_nhwc(x, wt, 1, pad)
    w_conv = np.ascontiguousarray(wt[:, ::-1, ::-1, :].transpose(1, 2, 0, 3))  # [R,S,C,K]
    want = oracle.conv2d_nhwc(x, w_conv, stride=1, pad=r - 1 - pad)
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-6)


@pytest.mark.parametrize("stride,pad", [(2, 1), (3, 0), (2, 0)])
def test_adjoint_of_the_convolution(stride, pad):
    # <convT_w(x), y> == <x, conv_w'(y)> with w'[r,s,k,c] = w[c,r,s,k]: the defining property
    rng = np.random.default_rng(11)
    n, h, w, c, k, r, s = 1, 4, 5, 3, 2, 3, 3
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    wt = rng.standard_normal((c, r, s, k)).astype(np.float32)
    z = oracle.conv_transpose2d_nhwc(x, wt, stride, pad)
    y = rng.standard_normal(z.shape).astype(np.float32)
    back = oracle.conv2d_nhwc(y, np.ascontiguousarray(wt.transpose(1, 2, 3, 0)), stride=stride, pad=pad)
    assert back.shape == x.shape
    lhs = float(np.sum(z.astype(np.float64) * y))
    rhs = float(np.sum(x.astype(np.float64) * back))
    assert abs(lhs - rhs) <= 1e-4 * max(1.0, abs(lhs))


@pytest.mark.parametrize("shape", SHAPES[1:])
def test_against_torch_conv_transpose2d(shape):
    torch = pytest.importorskip("torch")
    n, h, w, c, k, r, s, stride, pad, opad = shape
    rng = np.random.default_rng(5)
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    wt = rng.standard_normal((c, r, s, k)).astype(np.float32)
    got = oracle.conv_transpose2d_nhwc(x, wt, stride, pad, opad)
    tx = torch.from_numpy(x).permute(0, 3, 1, 2).double()
    tw = torch.from_numpy(wt).permute(0, 3, 1, 2).double()  # torch: [C_in, C_out, R, S]
    want = torch.nn.functional.conv_transpose2d(tx, tw, stride=stride, padding=pad, output_padding=opad)
    np.testing.assert_allclose(got, want.permute(0, 2, 3, 1).numpy(), rtol=0, atol=5e-6)


def test_bad_arguments_are_rejected():
    x = np.zeros((1, 2, 2, 1), dtype=np.float32)
    w = np.zeros((1, 2, 2, 1), dtype=np.float32)
    with pytest.raises(ValueError):
        oracle.conv_transpose2d_nhwc(x, w, stride=0)
    with pytest.raises(ValueError):
        oracle.conv_transpose2d_nhwc(x, w, stride=1, pad=2)  # (2-1) - 4 + 2 = -1 rows
