"""Execution plans on the device: a fused ResNet block against the CPU oracle, the
standalone node kernels against numpy, the reference's ResNet-18 benchmark graph
(src/bin/network_bench.rs:41-215) end to end against torch in fp32, and HIP-graph
replays of a plan against its eager run."""
import numpy as np
import pytest

import oracle
from helpers import assert_close_scaled, round_f16, tol_for_k
from test_graph_cpu import basic_block

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _bn_params(rng, ch):
    return [rng.uniform(0.5, 1.5, ch).astype(np.float32), (rng.standard_normal(ch) * 0.1).astype(np.float32),
            (rng.standard_normal(ch) * 0.1).astype(np.float32), rng.uniform(0.5, 1.5, ch).astype(np.float32)]


@pytest.mark.parametrize("fused", [True, False])
def test_basic_block_plan_matches_the_oracle(tracea_gpu, fused):
    from tracea_amd import graph as G, plan as P
    n, ch, hw = 4, 64, 14
    rng = np.random.default_rng(0x7ACEA020)
    x = round_f16(rng.standard_normal((n, hw, hw, ch)))
    w = {1: round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch))),
         4: round_f16(rng.standard_normal((3, 3, ch, ch)) * np.sqrt(2.0 / (9 * ch)))}
    bn = {20: _bn_params(rng, ch), 30: _bn_params(rng, ch)}

    def bn_op(base):
        return (oracle.EPI_BATCHNORM,) + tuple(bn[base]) + (1e-5,)

    y1 = round_f16(oracle.epilogue_apply(oracle.conv2d_nhwc(x, w[1], 1, 1), [bn_op(20), (oracle.EPI_RELU,)]))
    y2 = oracle.epilogue_apply(oracle.conv2d_nhwc(y1, w[4], 1, 1),
                               [bn_op(30), (oracle.EPI_RESIDUAL_ADD, x.reshape(-1, ch)), (oracle.EPI_RELU,)])
    graph = basic_block(n, ch, hw)
    plan = P.Plan(G.fuse(graph) if fused else graph)
    assert len(plan.describe()["steps"]) == (2 if fused else 7)
    plan.bind(0, torch.from_numpy(x).cuda().half())
    for base, params in bn.items():
        for i, v in enumerate(params):
            plan.bind(base + i, torch.from_numpy(v).cuda())
    plan.bind(1, torch.from_numpy(w[1]).cuda().half(), "weight_rsck")
    plan.bind(4, torch.from_numpy(w[4]).cuda().half().permute(3, 0, 1, 2).contiguous(), "weight")
    plan.run()
    last = plan.describe()["steps"][-1]["op_id"]
    got = plan.output(last, (n, hw, hw, ch)).float().cpu().numpy()
    # unfused, every node rounds its result to f16: one more rounding per node
    assert_close_scaled(got, y2, (2 if fused else 3) * tol_for_k(9 * ch), "block output, fused=%s" % fused)


def test_standalone_nodes_against_numpy(tracea_gpu):
    from tracea_amd import graph as G, plan as P
    n, c, h = 3, 40, 5
    rng = np.random.default_rng(7)
    x = round_f16(rng.standard_normal((n, h, h, c)))
    g = {"operators": [G.input_node(1, "x"), G.relu_node(2, "relu", x.size), G.add_node(3, "add", x.size),
                       G.global_avg_pool_node(4, "gap", n, c, h, h), G.softmax_node(5, "softmax"),
                       G.linear_node(6, "fc", n, 1, 24, c), G.softmax_node(7, "probs")],
         "dependencies": [[1, 2], [2, 3], [1, 3], [3, 4], [4, 5], [4, 6], [6, 7]]}
    wt = round_f16(rng.standard_normal((c, 24)) * 0.2)
    plan = P.Plan(g).bind(1, torch.from_numpy(x).cuda().half())
    plan.bind(6, torch.from_numpy(wt).cuda().half(), "weight")
    plan.run()
    relu = np.maximum(x, 0)
    add = round_f16(round_f16(relu) + x)
    gap = round_f16(add.reshape(n, h * h, c).mean(axis=1))

    def softmax(v):
        e = np.exp(v - v.max(axis=-1, keepdims=True))
        return e / e.sum(axis=-1, keepdims=True)

    # intermediates give their bytes back after their last consumer; only results nobody reads
    # (here the two softmax nodes) are still in the arena after the run
    np.testing.assert_allclose(plan.output(5, (n, c)).float().cpu().numpy(), softmax(gap), atol=1e-3)
    fc = round_f16(gap.astype(np.float64) @ wt.astype(np.float64))
    probs = plan.output(7, (n, 24)).float().cpu().numpy()
    np.testing.assert_allclose(probs, softmax(fc), atol=2e-3)
    np.testing.assert_allclose(probs.sum(axis=1), 1.0, atol=2e-3)
    # each kernel on its own, as the single result of a one-node plan
    dx = torch.from_numpy(x).cuda().half()
    one = P.Plan({"operators": [G.input_node(1, "x"), G.relu_node(2, "relu", x.size)], "dependencies": [[1, 2]]})
    one.bind(1, dx).run()
    np.testing.assert_array_equal(one.output(2, x.shape).float().cpu().numpy(), relu)
    one = P.Plan({"operators": [G.input_node(1, "x"), G.input_node(2, "y"), G.add_node(3, "add", x.size)],
                  "dependencies": [[1, 3], [2, 3]]})
    one.bind(1, dx).bind(2, torch.from_numpy(relu).cuda().half()).run()
    np.testing.assert_array_equal(one.output(3, x.shape).float().cpu().numpy(), round_f16(x + round_f16(relu)))
    one = P.Plan({"operators": [G.input_node(1, "x"), G.global_avg_pool_node(4, "gap", n, c, h, h)],
                  "dependencies": [[1, 4]]})
    one.bind(1, dx).run()
    np.testing.assert_allclose(one.output(4, (n, c)).float().cpu().numpy(), x.reshape(n, h * h, c).mean(axis=1),
                               atol=1e-3)
    params = _bn_params(rng, c)
    bn_graph = {"operators": [G.input_node(1, "x")] + [G.input_node(10 + i, "p%d" % i) for i in range(4)] +
                             [G.batchnorm_node(2, "bn", n, c, h, h)],
                "dependencies": [[1, 2], [10, 2], [11, 2], [12, 2], [13, 2]]}
    one = P.Plan(bn_graph).bind(1, dx)
    for i, v in enumerate(params):
        one.bind(10 + i, torch.from_numpy(v).cuda())
    one.run()
    want = oracle.epilogue_apply(x.reshape(-1, c), [(oracle.EPI_BATCHNORM,) + tuple(params) + (1e-5,)])
    np.testing.assert_allclose(one.output(2, (n * h * h, c)).float().cpu().numpy(), want, atol=4e-3)


def _resnet18(batch, seed):
    """Plan, bound tensors and a torch fp32 model of the same network."""
    from tracea_amd import graph as G, plan as P
    graph, info = G.resnet18_graph(batch)
    fused = G.fuse(graph)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    plan = P.Plan(fused)
    image = torch.zeros(batch, 224, 224, 8, device="cuda", dtype=torch.float16)
    image[..., :3] = torch.randn(batch, 224, 224, 3, device="cuda", generator=gen).half()
    plan.bind(info["input"], image)
    weights, bns = {}, {}
    for oid, (k, r, s, c) in info["convs"].items():
        w = (torch.randn(k, r, s, c, device="cuda", generator=gen) * (2.0 / (r * s * c)) ** 0.5).half()
        if c == 8:
            w[..., 3:] = 0
        weights[oid] = w
        plan.bind(oid, w, "weight")
    for oid, (params, c) in info["bn"].items():
        vals = [torch.rand(c, device="cuda", generator=gen) * 0.5 + 0.75, torch.randn(c, device="cuda", generator=gen) * 0.1,
                torch.randn(c, device="cuda", generator=gen) * 0.1, torch.rand(c, device="cuda", generator=gen) * 0.5 + 0.75]
        bns[oid] = vals
        for pid, v in zip(params, vals):
            plan.bind(pid, v)
    fc = (torch.randn(512, 1000, device="cuda", generator=gen) * 512 ** -0.5).half()
    plan.bind(info["fc"], fc, "weight")

    def reference():
        # the unfused graph, node by node, in fp32 (NCHW for torch's convolution)
        F = torch.nn.functional
        vals = {info["input"]: image.float().permute(0, 3, 1, 2)}
        prod = {}
        for src, dst in graph["dependencies"]:
            prod.setdefault(dst, []).append(src)
        for node in graph["operators"]:
            (kind, body), = node.items()
            oid = body["op_id"]
            if kind == "Input":
                continue
            ins = prod[oid]
            if kind == "Conv2d":
                vals[oid] = F.conv2d(vals[ins[0]], weights[oid].float().permute(0, 3, 1, 2), stride=body["stride"],
                                     padding=body["padding"])
            elif kind == "BatchNorm":
                g_, b_, m_, v_ = bns[oid]
                vals[oid] = F.batch_norm(vals[ins[0]], m_, v_, g_, b_, False, 0.0, body["epsilon"])
            elif kind == "Relu":
                vals[oid] = torch.relu(vals[ins[0]])
            elif kind == "Elementwise":
                vals[oid] = vals[ins[0]] + vals[ins[1]]
            elif kind == "GlobalAveragePool":
                vals[oid] = vals[ins[0]].mean(dim=(2, 3))
            elif kind == "Linear":
                vals[oid] = vals[ins[0]] @ fc.float()
        return vals[info["output"]]

    return plan, info, reference


def test_resnet18_end_to_end_against_torch_fp32(tracea_gpu):
    plan, info, reference = _resnet18(batch=2, seed=11)
    want = reference()
    plan.run()
    got = plan.output(info["output"], (2, 1000)).float()
    scale = float(want.abs().max())
    assert scale > 0.1
    # 20 half-precision layers deep: errors relative to the size of the logits
    assert float((got - want).abs().max()) <= 3e-2 * scale
    assert torch.equal(got.argmax(dim=1), want.argmax(dim=1))


def test_hip_graph_replays_equal_the_eager_run(tracea_gpu):
    plan, info, _ = _resnet18(batch=1, seed=12)
    plan.run()
    torch.cuda.synchronize()
    eager = plan.output(info["output"], (1, 1000)).clone()
    plan.capture()
    scratch = torch.zeros(1 << 20, device="cuda")
    for i in range(4):
        plan.output(info["output"]).zero_()          # a replay must write the result again
        scratch.add_(1.0)                            # eager work and a synchronisation between replays
        torch.cuda.synchronize()
        plan.replay()
        torch.cuda.synchronize()
        assert torch.equal(plan.output(info["output"], (1, 1000)), eager), "replay %d" % i
    assert float(scratch[0]) == 4.0


@pytest.mark.parametrize("n,c,h,classes", [(3, 44, 5, 24), (32, 512, 7, 1000), (1, 512, 7, 1000)])
@pytest.mark.parametrize("slot", ["weight", "weight_t"])
def test_pool_and_linear_in_one_launch(tracea_gpu, monkeypatch, n, c, h, classes, slot):
    """A pooling node read by one Linear node runs inside the Linear's launch: means as the pooling node
    alone computes them (same bits, still written to its place), logits against float64 and close to the
    two-launch plan's (another order of the fp32 sums)."""
    from tracea_amd import graph as G, plan as P
    rng = np.random.default_rng(c + classes)
    x = round_f16(rng.standard_normal((n, h, h, c)))
    wt = round_f16(rng.standard_normal((c, classes)) * 0.2)
    g = {"operators": [G.input_node(1, "x"), G.global_avg_pool_node(2, "gap", n, c, h, h), G.linear_node(3, "fc", n, 1, classes, c)],
         "dependencies": [[1, 2], [2, 3]]}
    dw = torch.from_numpy(wt if slot == "weight" else np.ascontiguousarray(wt.T)).cuda().half()

    def run():
        plan = P.Plan(g).bind(1, torch.from_numpy(x).cuda().half()).bind(3, dw, slot)
        plan.run()
        torch.cuda.synchronize()
        return plan, plan.output(2, (n, c)).clone(), plan.output(3, (n, classes)).float().cpu().numpy()

    one, gap_one, fc_one = run()
    assert [s["kind"] for s in one.describe()["steps"]] == ["Linear"] and one.describe()["steps"][0]["pooled_from"] == 2
    monkeypatch.setenv("TRACEA_PLAN_SPLIT_HEAD", "1")
    two, gap_two, fc_two = run()
    assert [s["kind"] for s in two.describe()["steps"]] == ["GlobalAveragePool", "Linear"]
    assert torch.equal(gap_one, gap_two)
    gap = gap_two.float().cpu().numpy()
    np.testing.assert_allclose(gap, x.reshape(n, h * h, c).mean(axis=1), atol=1e-3)
    want = gap.astype(np.float64) @ wt.astype(np.float64)
    tol = 2e-3 * max(1.0, np.abs(want).max())
    np.testing.assert_allclose(fc_one, want, atol=tol)
    np.testing.assert_allclose(fc_one, fc_two, atol=tol)


def test_side_by_side_steps_give_the_serial_result(tracea_gpu, monkeypatch):
    """TRACEA_PLAN_SIDE_BY_SIDE=1: the shortcut convolutions run on the plan's side stream beside the
    blocks' first convolutions; eager and as a replayed HIP graph the logits equal the serial plan's."""
    plan, info, _ = _resnet18(batch=2, seed=13)
    plan.run()
    torch.cuda.synchronize()
    serial = plan.output(info["output"], (2, 1000)).clone()
    monkeypatch.setenv("TRACEA_PLAN_SIDE_BY_SIDE", "1")
    forked, info2, _ = _resnet18(batch=2, seed=13)
    assert [s["side_by_side"] for s in forked.describe()["steps"]].count("second") == 3
    forked.run()
    torch.cuda.synchronize()
    assert torch.equal(forked.output(info2["output"], (2, 1000)), serial)
    forked.capture()
    for i in range(3):
        forked.output(info2["output"]).zero_()
        torch.cuda.synchronize()
        forked.replay()
        torch.cuda.synchronize()
        assert torch.equal(forked.output(info2["output"], (2, 1000)), serial), "replay %d" % i


def test_unbound_inputs_are_reported_before_any_launch(tracea_gpu):
    from tracea_amd import graph as G, plan as P
    plan = P.Plan(G.fuse(basic_block(1, 16, 8)))
    with pytest.raises(RuntimeError, match="is not bound"):
        plan.run()
    plan.bind(0, torch.zeros(1, 8, 8, 16, device="cuda", dtype=torch.float16))
    with pytest.raises(RuntimeError, match="not bound|no weight bound"):
        plan.run()


def test_attention_and_gemm_nodes_bf16(tracea_gpu):
    from tracea_amd import graph as G, plan as P
    b, h, s, d = 1, 2, 256, 64
    g = {"operators": [G.input_node(1, "q"), G.input_node(2, "k"), G.input_node(3, "v"),
                       {"Attention": dict(op_id=4, name="attn", b=b, s=s, h=h, d=d)},
                       G.gemm_node(5, "proj", b * h * s, 48, d), G.relu_node(6, "act", b * h * s * 48)],
         "dependencies": [[1, 4], [2, 4], [3, 4], [4, 5], [5, 6]]}
    fused = G.fuse(g)
    assert [list(n)[0] for n in fused["operators"]].count("Relu") == 0        # merged into the projection
    gen = torch.Generator(device="cuda").manual_seed(21)
    q, k, v = [torch.randn(b, h, s, d, device="cuda", generator=gen).bfloat16() for _ in range(3)]
    w = (torch.randn(d, 48, device="cuda", generator=gen) * d ** -0.5).bfloat16()
    plan = P.Plan(fused, dtype=torch.bfloat16)
    plan.bind(1, q).bind(2, k).bind(3, v)
    plan.bind(5, w.t().contiguous(), "weight_t")                              # stored [N,K]
    plan.run()
    attn = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    want = torch.relu(attn.bfloat16().float().reshape(-1, d) @ w.float())
    got = plan.output(5, (b * h * s, 48)).float()
    assert float((got - want).abs().max()) <= 3e-2 * max(1.0, float(want.abs().max()))
    # the same plan again after rebinding one input gives the new answer (nothing is cached)
    q2 = torch.randn(b, h, s, d, device="cuda", generator=gen).bfloat16()
    plan.bind(1, q2).run()
    attn2 = torch.nn.functional.scaled_dot_product_attention(q2.float(), k.float(), v.float())
    want2 = torch.relu(attn2.bfloat16().float().reshape(-1, d) @ w.float())
    assert float((plan.output(5, (b * h * s, 48)).float() - want2).abs().max()) <= 3e-2 * max(1.0, float(want2.abs().max()))
