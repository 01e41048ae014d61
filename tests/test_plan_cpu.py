"""Execution plans without a device: step order, data / side inputs, arena offsets and
their reuse, the output map and the errors of a malformed graph
(reference: src/runtime/plan.rs:10-53, src/runtime/compiler.rs:100-156)."""
import ctypes as C
import json

import pytest

from tracea_amd import capi
from tracea_amd import graph as G
from test_graph_cpu import basic_block


def compile_plan(graph, dtype=capi.F16):
    h = capi.lib().tracea_plan_compile(json.dumps(graph).encode(), dtype)
    if not h:
        raise ValueError(capi.last_error())
    try:
        desc = json.loads(capi.take_string(capi.lib().tracea_plan_describe(h)))
        assert desc["arena_size"] == capi.lib().tracea_plan_arena_size(h)
        return desc
    finally:
        capi.lib().tracea_plan_destroy(h)


def test_fused_basic_block_is_two_steps_in_two_slots():
    n, ch, hw = 8, 128, 28
    desc = compile_plan(G.fuse(basic_block(n, ch, hw)))
    steps = desc["steps"]
    assert [s["kind"] for s in steps] == ["Conv2d", "Conv2d"]
    size = n * hw * hw * ch * 2
    assert [s["bytes"] for s in steps] == [size, size] and size % 256 == 0
    assert [s["offset"] for s in steps] == [0, size]          # conv2 reads conv1's output: no overlap
    assert desc["arena_size"] == 2 * size
    first, second = steps
    assert first["inputs"] == [0] and [e["kind"] for e in first["epilogue"]] == [capi.OP_BATCHNORM, capi.OP_RELU]
    assert second["inputs"] == [first["op_id"]]
    assert [e["kind"] for e in second["epilogue"]] == [capi.OP_BATCHNORM, capi.OP_RESIDUAL_ADD, capi.OP_RELU]
    assert second["epilogue"][1]["tensors"] == [0]             # the skip input is the block's Input node
    assert desc["output_map"] == {str(first["op_id"]): [0, size], str(second["op_id"]): [size, size]}


def test_unfused_block_runs_every_node_and_reuses_freed_slots():
    n, ch, hw = 2, 16, 8
    desc = compile_plan(basic_block(n, ch, hw))
    kinds = [s["kind"] for s in desc["steps"]]
    assert kinds == ["Conv2d", "BatchNorm", "Relu", "Conv2d", "BatchNorm", "Elementwise", "Relu"]
    size = n * hw * hw * ch * 2
    assert all(s["bytes"] == size for s in desc["steps"])
    # a chain: each intermediate dies when its consumer has run, so two slots alternate
    assert desc["arena_size"] == 2 * size
    assert [s["offset"] for s in desc["steps"]] == [0, size, 0, size, 0, size, 0]
    bn = desc["steps"][1]
    assert len(bn["inputs"]) == 5 and bn["inputs"][0] == desc["steps"][0]["op_id"]
    add = desc["steps"][5]
    assert len(add["inputs"]) == 2 and 0 in add["inputs"]


def test_resnet18_plan_reuses_the_arena(monkeypatch):
    monkeypatch.setenv("TRACEA_PLAN_SIDE_BY_SIDE", "1")
    graph, info = G.resnet18_graph(batch=1)
    assert len(graph["operators"]) == 148
    fused = G.fuse(graph)
    kinds = [list(n)[0] for n in fused["operators"]]
    assert kinds.count("Conv2d") == 20 and kinds.count("BatchNorm") == 0 and kinds.count("Relu") == 0
    assert kinds.count("Elementwise") == 0 and kinds.count("GlobalAveragePool") == 1 and kinds.count("Linear") == 1
    desc = compile_plan(fused)
    steps = desc["steps"]
    # 20 convolutions and the classifier head: the Linear step took over the pooling node in front of it
    # (one launch) and still writes the pooling node's output
    assert len(steps) == 21 and steps[-1]["kind"] == "Linear" and steps[-1]["op_id"] == info["output"]
    pool_id = [list(n.values())[0]["op_id"] for n in fused["operators"] if list(n)[0] == "GlobalAveragePool"][0]
    assert steps[-1]["pooled_from"] == pool_id and steps[-1]["inputs"] == [steps[-2]["op_id"]]
    assert str(pool_id) in desc["output_map"] and desc["output_map"][str(pool_id)][1] == 512 * 2
    lo, size = desc["output_map"][str(pool_id)]
    assert lo + size <= steps[-1]["offset"] or lo >= steps[-1]["offset"] + steps[-1]["bytes"]
    assert lo + size <= steps[-2]["offset"] or lo >= steps[-2]["offset"] + steps[-2]["bytes"]
    total = sum(s["bytes"] for s in steps)
    assert desc["arena_size"] * 3 <= total                        # 1.2 MB against 3.8 MB
    # every step's inputs precede it, and no live tensor overlaps a step's output
    place = {s["op_id"]: (i, s["offset"], s["offset"] + s["bytes"], s["last_use"]) for i, s in enumerate(steps)}
    for i, s in enumerate(steps):
        reads = list(s["inputs"]) + [t for e in s["epilogue"] for t in e["tensors"]]
        for t in reads:
            if t in place:
                assert place[t][0] < i
        for t, (born, lo, hi, last) in place.items():
            if t != s["op_id"] and born < i <= last:
                assert hi <= s["offset"] or lo >= s["offset"] + s["bytes"], (s["name"], t)
    # residual inputs were resolved to nodes that exist
    ids = {list(n.values())[0]["op_id"] for n in fused["operators"]}
    for s in steps:
        for e in s["epilogue"]:
            assert all(t in ids for t in e["tensors"])
    # a downsampling block: the 1x1 shortcut convolution runs before the convolution that adds it
    names = [s["name"] for s in steps]
    assert names.index("layer_128_block_0_shortcut_conv") < names.index("layer_128_block_0_conv2")
    # ... and beside the block's first convolution, which it does not depend on: the three pairs of the
    # network, each with both outputs and everything either step reads in disjoint memory
    pairs = [(steps[i]["name"], steps[i + 1]["name"]) for i in range(len(steps) - 1) if steps[i]["side_by_side"] == "first"]
    assert pairs == [("layer_%d_block_0_conv1" % c, "layer_%d_block_0_shortcut_conv" % c) for c in (128, 256, 512)]
    assert [s["side_by_side"] for s in steps].count("second") == 3
    for i, s in enumerate(steps):
        if s["side_by_side"] != "first":
            continue
        nxt = steps[i + 1]
        assert nxt["side_by_side"] == "second" and s["op_id"] not in nxt["inputs"]
        spans = [(s["offset"], s["offset"] + s["bytes"]), (nxt["offset"], nxt["offset"] + nxt["bytes"])]
        for t in set(list(s["inputs"]) + list(nxt["inputs"])):
            if t in place:
                spans.append((place[t][1], place[t][2]))
                assert place[t][3] >= i + 1               # kept until the second step is done
        spans = sorted(set(spans))
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), spans


def test_split_head_switch(monkeypatch):
    """TRACEA_PLAN_SPLIT_HEAD=1 (read when a plan is compiled) keeps pooling and the linear layer two steps."""
    graph, _ = G.resnet18_graph(batch=1)
    monkeypatch.setenv("TRACEA_PLAN_SPLIT_HEAD", "1")
    steps = compile_plan(G.fuse(graph))["steps"]
    assert len(steps) == 22 and [s["kind"] for s in steps[-2:]] == ["GlobalAveragePool", "Linear"]
    assert all(s["pooled_from"] == 0 for s in steps)


def test_plan_is_serial_by_default(monkeypatch):
    """Without TRACEA_PLAN_SIDE_BY_SIDE=1 (read when a plan is compiled) every step stays on the caller's stream."""
    graph, _ = G.resnet18_graph(batch=1)
    monkeypatch.delenv("TRACEA_PLAN_SIDE_BY_SIDE", raising=False)
    steps = compile_plan(G.fuse(graph))["steps"]
    assert all(s["side_by_side"] == "no" for s in steps)


def test_graph_outputs_stay_allocated_to_the_end():
    g = {"operators": [G.input_node(1, "x"), G.relu_node(2, "a", 4096), G.relu_node(3, "b", 4096),
                       G.relu_node(4, "c", 4096)],
         "dependencies": [[1, 2], [1, 3], [3, 4]]}
    desc = compile_plan(g)
    by = {s["op_id"]: s for s in desc["steps"]}
    assert by[2]["last_use"] == 3 and by[4]["last_use"] == 3      # results nobody reads: kept
    assert by[3]["last_use"] == 2                                # read by step index 2
    assert len({by[2]["offset"], by[3]["offset"], by[4]["offset"]}) == 3
    assert desc["arena_size"] == 3 * 8192


def test_ids_out_of_edge_order_are_sorted_topologically():
    g = {"operators": [G.relu_node(2, "late", 64), G.relu_node(5, "early", 64), G.input_node(9, "x")],
         "dependencies": [[9, 5], [5, 2]]}
    assert [s["name"] for s in compile_plan(g)["steps"]] == ["early", "late"]


@pytest.mark.parametrize("graph,message", [
    ({"operators": [G.input_node(1, "x"), G.input_node(4, "y"), G.relu_node(2, "a", 8)],
      "dependencies": [[1, 2], [4, 2]]}, "needs 1 inputs, the graph gives 2"),
    ({"operators": [G.relu_node(2, "a", 8), G.relu_node(3, "b", 8)], "dependencies": [[2, 3], [3, 2]]}, "cycle"),
    ({"operators": [G.input_node(1, "x"), G.relu_node(2, "a", 8)], "dependencies": [[1, 2], [7, 2]]},
     "unknown producer 7"),
    ({"operators": [G.input_node(1, "x"), {"MaxPool": {"op_id": 2, "name": "p"}}], "dependencies": [[1, 2]]},
     "no kernel here"),
    ({"operators": [G.input_node(1, "x"), G.conv2d_node(2, "c", 1, 3, 8, 8, 8, 3, 3, 1, 1)], "dependencies": [[1, 2]]},
     "multiple of 8"),
    ({"operators": [G.input_node(1, "x"), G.conv2d_node(2, "c", 1, 8, 8, 8, 16, 3, 3, 1, 1), G.relu_node(3, "r", 100)],
      "dependencies": [[1, 2], [2, 3]]}, "its producer writes 1024"),
    ({"operators": [G.input_node(1, "x"), G.batchnorm_node(2, "bn", 1, 8, 4, 4)], "dependencies": [[1, 2]]},
     "needs 5 inputs"),
    ({"operators": [G.input_node(1, "x"), {"Elementwise": dict(op_id=2, name="m", kind="Mul", n=8)}],
      "dependencies": [[1, 2], [1, 2]]}, "only kind"),
    ({"operators": [G.input_node(1, "x"), G.input_node(1, "y")], "dependencies": []}, "duplicate op_id 1"),
])
def test_malformed_graphs_are_refused(graph, message):
    with pytest.raises(ValueError, match=message):
        compile_plan(graph)


def test_bind_sized_refuses_short_and_wrongly_typed_tensors():
    # what a bound pointer must hold is known from the consumers of the Input node: the data input of the
    # first convolution and the skip tensor in the plan's type, BatchNorm parameters as float32 vectors
    n, ch, hw = 2, 16, 8
    h = capi.lib().tracea_plan_compile(json.dumps(G.fuse(basic_block(n, ch, hw))).encode(), capi.F16)
    assert h
    try:
        desc = json.loads(capi.take_string(capi.lib().tracea_plan_describe(h)))
        first, second = desc["steps"]
        bind = capi.lib().tracea_plan_bind_sized
        ptr = C.c_void_p(4096)
        x_bytes = n * hw * hw * ch * 2
        assert bind(h, 0, b"input", ptr, x_bytes, capi.F16) == capi.SUCCESS
        assert bind(h, 0, b"input", ptr, x_bytes + 512, -1) == capi.SUCCESS        # larger, type not stated
        assert bind(h, 0, b"input", ptr, x_bytes - 2, capi.F16) == capi.INVALID_PARAMS
        assert "holds %d bytes, the plan reads %d" % (x_bytes - 2, x_bytes) in capi.last_error()
        assert bind(h, 0, b"input", ptr, x_bytes, capi.BF16) == capi.INVALID_PARAMS
        gamma = first["epilogue"][0]["tensors"][0]
        assert bind(h, gamma, b"input", ptr, ch * 4, capi.F32) == capi.SUCCESS
        assert bind(h, gamma, b"input", ptr, ch * 2, capi.F16) == capi.INVALID_PARAMS   # a half-precision parameter vector
        assert bind(h, gamma, b"input", ptr, ch * 4, capi.F16) == capi.INVALID_PARAMS
        w_bytes = ch * 3 * 3 * ch * 2
        assert bind(h, first["op_id"], b"weight", ptr, w_bytes, capi.F16) == capi.SUCCESS
        assert bind(h, second["op_id"], b"weight_rsck", ptr, w_bytes, capi.F16) == capi.SUCCESS
        assert bind(h, first["op_id"], b"weight", ptr, w_bytes - 2, capi.F16) == capi.INVALID_PARAMS
        assert bind(h, first["op_id"], b"weight", ptr, w_bytes, capi.F32) == capi.INVALID_PARAMS
        assert bind(h, 12345, b"weight", ptr, w_bytes, capi.F16) == capi.INVALID_PARAMS   # no such step
    finally:
        capi.lib().tracea_plan_destroy(h)


def test_dtype_and_null_arguments():
    g = {"operators": [G.input_node(1, "x"), G.relu_node(2, "a", 8)], "dependencies": [[1, 2]]}
    with pytest.raises(ValueError, match="f16 or bf16"):
        compile_plan(g, capi.F32)
    assert not capi.lib().tracea_plan_compile(None, capi.F16)
    h = capi.lib().tracea_plan_compile(json.dumps(g).encode(), capi.BF16)
    try:
        off, size = C.c_size_t(), C.c_size_t()
        assert capi.lib().tracea_plan_output(h, 2, C.byref(off), C.byref(size)) == capi.SUCCESS
        assert (off.value, size.value) == (0, 16)
        assert capi.lib().tracea_plan_output(h, 1, C.byref(off), C.byref(size)) == capi.INVALID_PARAMS  # an Input
        assert capi.lib().tracea_plan_bind(h, 2, b"input", C.c_void_p(256)) == capi.INVALID_PARAMS
        assert capi.lib().tracea_plan_bind(h, 1, b"bogus", C.c_void_p(256)) == capi.INVALID_PARAMS
        assert capi.lib().tracea_plan_bind(h, 1, b"input", None) == capi.INVALID_PARAMS
        assert capi.lib().tracea_plan_bind(h, 1, b"input", C.c_void_p(256)) == capi.SUCCESS
        # running needs the runtime: without tracea_init the call reports it and launches nothing
        capi.lib().tracea_shutdown()
        assert capi.lib().tracea_plan_run(h, C.c_void_p(256), 0, None) == capi.UNKNOWN_ERROR
    finally:
        capi.lib().tracea_plan_destroy(h)
