"""Graph fusion through tracea_graph_fuse: the three cases of the reference's
tests/fusion_verification.rs, then the ResNet basic block and the cases where
the rules must not fire (src/core/optimizer.rs:40-60)."""
import pytest

from tracea_amd import graph as G


def _by_id(graph):
    out = {}
    for node in graph["operators"]:
        (kind, body), = node.items()
        out[body["op_id"]] = (kind, body)
    return out


def test_conv_relu_fusion():
    g = {"operators": [G.conv2d_node(1, "conv", 1, 3, 224, 224, 64, 3, 3, 1, 1), G.relu_node(2, "relu", 64 * 224 * 224)],
         "dependencies": [[1, 2]]}
    f = G.fuse(g)
    assert len(f["operators"]) == 1
    kind, body = _by_id(f)[1]
    assert kind == "Conv2d" and body["epilogue"] == ["ReLU"]
    assert f["dependencies"] == []
    # every other field of the node survives untouched
    assert {k: v for k, v in body.items() if k != "epilogue"} == \
        {k: v for k, v in g["operators"][0]["Conv2d"].items() if k != "epilogue"}


def test_conv_bn_relu_fusion():
    ops = [G.conv2d_node(1, "conv", 1, 3, 224, 224, 64, 3, 3, 1, 1), G.batchnorm_node(2, "bn", 1, 64, 224, 224),
           G.relu_node(3, "relu", 64 * 224 * 224), G.input_node(10, "gamma"), G.input_node(11, "beta"),
           G.input_node(12, "mean"), G.input_node(13, "var")]
    deps = [[1, 2], [10, 2], [11, 2], [12, 2], [13, 2], [2, 3]]
    f = G.fuse({"operators": ops, "dependencies": deps})
    assert len(f["operators"]) == 5
    kind, body = _by_id(f)[1]
    assert kind == "Conv2d" and len(body["epilogue"]) == 2
    bn = body["epilogue"][0]["BatchNorm"]
    assert (bn["op_id"], bn["gamma_id"], bn["beta_id"], bn["mean_id"], bn["var_id"]) == (2, 10, 11, 12, 13)
    assert bn["epsilon"] == pytest.approx(1e-5)
    assert body["epilogue"][1] == "ReLU"
    # the parameters now feed the fused node
    assert sorted(map(tuple, f["dependencies"])) == [(10, 1), (11, 1), (12, 1), (13, 1)]


def test_residual_fusion():
    ops = [G.conv2d_node(1, "main_path", 1, 64, 56, 56, 64, 3, 3, 1, 1), G.add_node(2, "add", 64 * 56 * 56),
           G.relu_node(3, "relu", 64 * 56 * 56), G.input_node(0, "input")]
    deps = [[0, 1], [0, 2], [1, 2], [2, 3]]
    f = G.fuse({"operators": ops, "dependencies": deps})
    assert len(f["operators"]) == 2
    kind, body = _by_id(f)[1]
    assert body["epilogue"] == [{"ResidualAdd": {"residual_ptr": 0}}, "ReLU"]
    assert sorted(map(tuple, f["dependencies"])) == [(0, 1)]


def basic_block(n=32, ch=128, hw=28):
    """conv1 -> BN1 -> ReLU -> conv2 -> BN2 -> (+ x) -> ReLU, ids as in the executor test."""
    e = n * ch * hw * hw
    ops = [G.input_node(0, "x"),
           G.conv2d_node(1, "conv1", n, ch, hw, hw, ch, 3, 3, 1, 1), G.batchnorm_node(2, "bn1", n, ch, hw, hw),
           G.relu_node(3, "relu1", e),
           G.conv2d_node(4, "conv2", n, ch, hw, hw, ch, 3, 3, 1, 1), G.batchnorm_node(5, "bn2", n, ch, hw, hw),
           G.add_node(6, "add", e), G.relu_node(7, "relu2", e)]
    deps = [[0, 1], [1, 2]]
    for i, pid in enumerate((20, 21, 22, 23)):
        ops.append(G.input_node(pid, "bn1_" + "gbmv"[i]))
        deps.append([pid, 2])
    deps += [[2, 3], [3, 4], [4, 5]]
    for i, pid in enumerate((30, 31, 32, 33)):
        ops.append(G.input_node(pid, "bn2_" + "gbmv"[i]))
        deps.append([pid, 5])
    deps += [[5, 6], [0, 6], [6, 7]]
    return {"operators": ops, "dependencies": deps}


def test_resnet_basic_block_becomes_two_launches():
    f = G.fuse(basic_block())
    nodes = _by_id(f)
    assert sorted(k for k, (kind, _) in nodes.items() if kind != "Input") == [1, 4]
    e1, e2 = nodes[1][1]["epilogue"], nodes[4][1]["epilogue"]
    assert [list(x)[0] if isinstance(x, dict) else x for x in e1] == ["BatchNorm", "ReLU"]
    assert [list(x)[0] if isinstance(x, dict) else x for x in e2] == ["BatchNorm", "ResidualAdd", "ReLU"]
    assert e2[1]["ResidualAdd"]["residual_ptr"] == 0
    assert e1[0]["BatchNorm"]["gamma_id"] == 20 and e2[0]["BatchNorm"]["var_id"] == 33
    deps = set(map(tuple, f["dependencies"]))
    assert {(0, 1), (1, 4), (0, 4), (20, 1), (33, 4)} <= deps
    assert all(src in nodes and dst in nodes for src, dst in deps)
    assert G.fuse(f) == f  # a fixpoint


def test_rules_that_must_not_fire():
    # two consumers: the conv output is needed unfused
    g = {"operators": [G.conv2d_node(1, "c", 1, 16, 8, 8, 16, 3, 3, 1, 1), G.relu_node(2, "r", 1024),
                       G.add_node(3, "a", 1024)],
         "dependencies": [[1, 2], [1, 3], [2, 3]]}
    f = G.fuse(g)
    assert len(f["operators"]) == 3 and _by_id(f)[1][1]["epilogue"] == []
    # BatchNorm without its four parameter producers
    g = {"operators": [G.conv2d_node(1, "c", 1, 16, 8, 8, 16, 3, 3, 1, 1), G.batchnorm_node(2, "bn", 1, 16, 8, 8)],
         "dependencies": [[1, 2]]}
    assert len(G.fuse(g)["operators"]) == 2
    # Mul is not a residual add; Softmax is no epilogue
    mul = G.add_node(2, "m", 1024)
    mul["Elementwise"]["kind"] = "Mul"
    g = {"operators": [G.input_node(0, "x"), G.gemm_node(1, "g", 64, 64, 64), mul], "dependencies": [[0, 2], [1, 2]]}
    assert len(G.fuse(g)["operators"]) == 3
    g = {"operators": [G.gemm_node(1, "g", 64, 64, 64), {"Softmax": {"op_id": 2, "name": "s", "axis": -1}}],
         "dependencies": [[1, 2]]}
    assert len(G.fuse(g)["operators"]) == 2


def test_gemm_and_linear_fuse_too_and_skip_inputs_follow_earlier_merges():
    # y = relu(gemm2(x) + relu(gemm1(x))): the skip input of the add is node 2, which was merged into node 1
    ops = [G.input_node(0, "x"), G.gemm_node(1, "g1", 64, 64, 64), G.relu_node(2, "r1", 4096),
           {"Linear": {"op_id": 3, "name": "lin", "batch": 1, "m": 64, "n": 64, "k": 64, "epilogue": []}},
           G.add_node(4, "add", 4096), G.relu_node(5, "r2", 4096)]
    deps = [[0, 1], [1, 2], [0, 3], [2, 4], [3, 4], [4, 5]]
    f = G.fuse({"operators": ops, "dependencies": deps})
    nodes = _by_id(f)
    assert sorted(nodes) == [0, 1, 3]
    assert nodes[1][1]["epilogue"] == ["ReLU"]
    assert nodes[3][1]["epilogue"] == [{"ResidualAdd": {"residual_ptr": 1}}, "ReLU"]


def test_malformed_graphs_are_errors():
    for bad in ({"operators": []}, {"operators": [{"Conv2d": {"name": "no id"}}], "dependencies": []},
                {"operators": [], "dependencies": [[1]]}):
        with pytest.raises(ValueError):
            G.fuse(bad)
