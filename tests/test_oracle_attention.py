"""Pins the attention oracle through invariants of softmax attention and
through torch's scaled_dot_product_attention as an independent routine."""
import os

import numpy as np
import pytest

import oracle

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _qkv(s, d, seed):
    rng = np.random.default_rng(seed)
    return [rng.standard_normal((s, d)).astype(np.float32) for _ in range(3)]


def test_constant_values_give_constant_output():
    q, k, _ = _qkv(50, 16, 0)
    v = np.tile(np.arange(16, dtype=np.float32), (50, 1))
    for causal in (False, True):
        o = oracle.attention(q, k, v, 0.25, causal)
        assert np.abs(o - v).max() < 1e-5  # rows of P sum to one


def test_causal_first_row_and_zero_query_prefix_means():
    q, k, v = _qkv(33, 8, 1)
    o = oracle.attention(q, k, v, 0.3, True)
    assert np.abs(o[0] - v[0]).max() < 1e-6  # row 0 sees key 0 only
    zero = np.zeros_like(q)
    o = oracle.attention(zero, k, v, 0.3, True)
    prefix = np.cumsum(v.astype(np.float64), axis=0) / np.arange(1, 34)[:, None]
    assert np.abs(o - prefix).max() < 1e-5  # uniform weights over the visible prefix
    o = oracle.attention(zero, k, v, 0.3, False)
    assert np.abs(o - v.mean(axis=0, dtype=np.float64)).max() < 1e-5


def test_key_permutation_equivariance_noncausal():
    q, k, v = _qkv(40, 8, 2)
    perm = np.random.default_rng(3).permutation(40)
    a = oracle.attention(q, k, v, 0.2, False)
    b = oracle.attention(q, k[perm], v[perm], 0.2, False)
    assert np.abs(a - b).max() < 1e-5


def test_row_subset_equals_full():
    q, k, v = _qkv(64, 16, 4)
    full = oracle.attention(q, k, v, 0.25, True)
    rows = np.array([0, 5, 31, 63], np.int32)
    sub = oracle.attention(q, k, v, 0.25, True, rows=rows)
    assert np.array_equal(sub, full[rows])
    with pytest.raises(ValueError):
        oracle.attention(q, k, v, 0.25, True, rows=np.array([64], np.int32))


@pytest.mark.parametrize("s", [16, 77, 123, 257])  # edge sizes of tests/python/edge_case_fa2.py:56-71
@pytest.mark.parametrize("causal", [False, True])
def test_matches_torch_sdpa(s, causal):
    torch = pytest.importorskip("torch")
    d = 32
    q, k, v = _qkv(s, d, 10 + s)
    scale = 1.0 / np.sqrt(d)
    o = oracle.attention(q, k, v, scale, causal)
    t = [torch.from_numpy(x)[None, None].double() for x in (q, k, v)]
    ot = torch.nn.functional.scaled_dot_product_attention(*t, is_causal=causal, scale=scale)[0, 0].numpy()
    assert np.abs(o - ot).max() < 1e-5


def test_committed_fixture():
    d = np.load(os.path.join(GOLDEN, "attention_small.npz"))
    for causal, key in ((False, "o_dense"), (True, "o_causal")):
        o = oracle.attention_bhsd(d["q"], d["k"], d["v"], float(d["scale"]), causal)
        assert np.abs(o - d[key]).max() < 1e-5
