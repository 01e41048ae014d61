"""Writes the small golden vectors under tests/golden/.

The expected outputs come from torch's float64 CPU routines
(torch.nn.functional.conv2d / scaled_dot_product_attention), an independent
library statement of the same mathematics as the naive loops of the reference
(examples/verify_conv2d.rs:8-44, examples/verify_fa2_numeric.rs:22-93).
Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def conv_fixture():
    rng = np.random.default_rng(20240601)
    n, h, w, c, k, r, s, stride, pad, dil = 2, 9, 8, 16, 24, 3, 3, 2, 1, 1
    x = rng.standard_normal((n, h, w, c)).astype(np.float32)
    wt = (rng.standard_normal((r, s, c, k)) * np.sqrt(2.0 / (r * s * c))).astype(np.float32)
    y = torch.nn.functional.conv2d(torch.from_numpy(x).permute(0, 3, 1, 2).double(),
                                   torch.from_numpy(wt).permute(3, 2, 0, 1).double(),
                                   stride=stride, padding=pad, dilation=dil).permute(0, 2, 3, 1)
    np.savez_compressed(os.path.join(HERE, "conv2d_small.npz"), x=x, w_rsck=wt,
                        y=y.numpy().astype(np.float32), stride=stride, pad=pad, dilation=dil)


def attention_fixture():
    rng = np.random.default_rng(20240602)
    b, h, s, d = 1, 1, 77, 32
    q, k, v = [rng.standard_normal((b, h, s, d)).astype(np.float32) for _ in range(3)]
    scale = 1.0 / np.sqrt(d)
    tq, tk, tv = [torch.from_numpy(t).double() for t in (q, k, v)]
    dense = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, scale=scale)
    causal = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=scale)
    np.savez_compressed(os.path.join(HERE, "attention_small.npz"), q=q, k=k, v=v, scale=scale,
                        o_dense=dense.numpy().astype(np.float32),
                        o_causal=causal.numpy().astype(np.float32))


if __name__ == "__main__":
    conv_fixture()
    attention_fixture()
    print("fixtures written to", HERE)
