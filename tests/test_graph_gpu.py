"""A ResNet basic block given as an unfused operator graph: fused by
tracea_graph_fuse, executed as two tracea_conv2d_ex launches, compared with the
CPU oracle running the same operators one by one (unfused BatchNorm,
src/emitter/metal/utils.rs:56-73; epilogue order src/core/optimizer.rs:122-150)."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_f16, tol_for_k
from test_graph_cpu import basic_block

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def test_fused_basic_block_graph_matches_the_oracle(tracea_gpu):
    from tracea_amd import graph as G
    n, ch, hw = 8, 128, 28
    rng = np.random.default_rng(0x7ACEA014)
    x = round_f16(rng.standard_normal((n, hw, hw, ch)))
    w = {1: round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch))),
         4: round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch)))}
    bn = {}
    for base in (20, 30):
        bn[base] = rng.uniform(0.5, 1.5, ch).astype(np.float32)            # gamma
        bn[base + 1] = (rng.standard_normal(ch) * 0.1).astype(np.float32)  # beta
        bn[base + 2] = (rng.standard_normal(ch) * 0.1).astype(np.float32)  # mean
        bn[base + 3] = rng.uniform(0.5, 1.5, ch).astype(np.float32)        # var

    def bn_op(base):
        return (oracle.EPI_BATCHNORM, bn[base], bn[base + 1], bn[base + 2], bn[base + 3], 1e-5)

    y1 = round_f16(oracle.epilogue_apply(oracle.conv2d_nhwc(x, w[1], 1, 1), [bn_op(20), (oracle.EPI_RELU,)]))
    y2 = oracle.epilogue_apply(oracle.conv2d_nhwc(y1, w[4], 1, 1),
                               [bn_op(30), (oracle.EPI_RESIDUAL_ADD, x.reshape(-1, ch)), (oracle.EPI_RELU,)])

    fused = G.fuse(basic_block(n, ch, hw))
    tensors = {0: torch.from_numpy(x).cuda().half()}
    for pid, v in bn.items():
        tensors[pid] = torch.from_numpy(v).cuda()
    weights = {i: torch.from_numpy(w[i]).cuda().half().permute(3, 0, 1, 2).contiguous() for i in (1, 4)}
    out = G.execute(fused, tensors, weights)
    assert sorted(k for k in out if k < 20) == [0, 1, 4]  # two launches, no standalone BN / add / relu
    assert_close_scaled(out[1].float().cpu().numpy(), y1, tol_for_k(9 * ch), "conv1+BN+ReLU")
    assert_close_scaled(out[4].float().cpu().numpy(), y2, 2 * tol_for_k(9 * ch), "block output")
    # an unfused leftover has no kernel: executing the raw graph must refuse, not fall back
    with pytest.raises(ValueError):
        G.execute(basic_block(n, ch, hw), dict(tensors), weights)
