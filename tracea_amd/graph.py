"""Operator graphs: fusion through ``tracea_graph_fuse`` and execution of the
fused graph as one ``tracea_conv2d_ex`` / ``tracea_gemm_ex`` launch per node.

Graphs are dicts in the reference's GraphTopology JSON form
(src/policy/types.rs:29-95,189-192): ``{"operators": [{"Conv2d": {...}}, ...],
"dependencies": [[producer, consumer], ...]}``; fusion rules are those of
src/core/optimizer.rs:12-160.  The builders below spell the operator variants.
"""
import json

from . import capi


def conv2d_node(op_id, name, n, c, h, w, k, r, s, stride=1, padding=0):
    return {"Conv2d": dict(op_id=op_id, name=name, n=n, c=c, h=h, w=w, k=k, r=r, s=s, stride=stride,
                           padding=padding, epilogue=[])}


def gemm_node(op_id, name, m, n, k):
    return {"Gemm": dict(op_id=op_id, name=name, m=m, n=n, k=k, batch=1, kind="Dense", epilogue=[])}


def relu_node(op_id, name, n):
    return {"Relu": dict(op_id=op_id, name=name, n=n)}


def add_node(op_id, name, n):
    return {"Elementwise": dict(op_id=op_id, name=name, kind="Add", n=n)}


def batchnorm_node(op_id, name, n, c, h, w, epsilon=1e-5, momentum=0.1):
    return {"BatchNorm": dict(op_id=op_id, name=name, n=n, c=c, h=h, w=w, epsilon=epsilon, momentum=momentum)}


def input_node(op_id, name):
    return {"Input": dict(op_id=op_id, name=name)}


def fuse(graph):
    """GraphOptimizer::optimize: returns the rewritten graph (a new dict)."""
    text = capi.take_string(capi.lib().tracea_graph_fuse(json.dumps(graph).encode()))
    if text is None:
        raise ValueError("graph_fuse: " + capi.last_error())
    return json.loads(text)


def _kind(node):
    (kind, body), = node.items()
    return kind, body


def _chain(epilogue, tensors):
    """Epilogue list of a fused node -> operator tuples for ops.conv2d_ex / gemm_ex."""
    ops = []
    for e in epilogue:
        if e == "ReLU":
            ops.append((capi.OP_RELU,))
        elif e == "Gelu":
            ops.append((capi.OP_GELU,))
        elif e == "SiLU":
            ops.append((capi.OP_SILU,))
        elif isinstance(e, dict) and "BatchNorm" in e:
            b = e["BatchNorm"]
            ops.append((capi.OP_BATCHNORM, tensors[b["gamma_id"]], tensors[b["beta_id"]], tensors[b["mean_id"]],
                        tensors[b["var_id"]], b["epsilon"]))
        elif isinstance(e, dict) and "ResidualAdd" in e:
            ops.append((capi.OP_RESIDUAL_ADD, tensors[e["ResidualAdd"]["residual_ptr"]]))
        else:
            raise ValueError("epilogue entry %r cannot be executed" % (e,))
    return ops


def execute(graph, tensors, weights):
    """Runs a fused graph on the device, one launch per Conv2d / Gemm node.

    ``tensors`` maps the op_id of every Input node to a device tensor (NHWC
    activations, per-channel BatchNorm parameters); ``weights`` maps the op_id of
    every Conv2d node to its [K,R,S,C] filters, of every Gemm node to its [K,N]
    right operand.  Node outputs are added to ``tensors`` under their op_id.
    The data input of a node is its first producer in the dependency list that
    is not one of its epilogue's side inputs.  Returns ``tensors``.
    """
    from . import ops
    producers = {}
    for src, dst in graph["dependencies"]:
        producers.setdefault(dst, []).append(src)
    pending = [n for n in graph["operators"] if _kind(n)[0] != "Input"]
    while pending:
        progressed = False
        for node in list(pending):
            kind, body = _kind(node)
            oid = body["op_id"]
            side = set()
            for e in body.get("epilogue", []):
                if isinstance(e, dict) and "BatchNorm" in e:
                    side.update(e["BatchNorm"][k] for k in ("gamma_id", "beta_id", "mean_id", "var_id"))
                elif isinstance(e, dict) and "ResidualAdd" in e:
                    side.add(e["ResidualAdd"]["residual_ptr"])
            needs = producers.get(oid, [])
            if any(p not in tensors for p in needs):
                continue
            data = [p for p in needs if p not in side] or [p for p in needs]
            if kind == "Conv2d":
                tensors[oid] = ops.conv2d_ex(tensors[data[0]], weights[oid], _chain(body["epilogue"], tensors),
                                             stride=body["stride"], padding=body["padding"])
            elif kind == "Gemm":
                tensors[oid] = ops.gemm_ex(tensors[data[0]], weights[oid], _chain(body["epilogue"], tensors))
            else:
                raise ValueError("operator %s (%s) was not fused into a contraction and has no kernel here"
                                 % (body.get("name"), kind))
            pending.remove(node)
            progressed = True
        if not progressed:
            raise ValueError("graph has a cycle or an input without a tensor")
    return tensors


def global_avg_pool_node(op_id, name, n, c, h, w):
    return {"GlobalAveragePool": dict(op_id=op_id, name=name, n=n, c=c, h=h, w=w)}


def linear_node(op_id, name, batch, m, n, k):
    return {"Linear": dict(op_id=op_id, name=name, batch=batch, m=m, n=n, k=k, epilogue=[])}


def softmax_node(op_id, name, axis=-1):
    return {"Softmax": dict(op_id=op_id, name=name, axis=axis)}


def resnet18_graph(batch=1, in_channels=8, classes=1000):
    """The ResNet-18 graph of the reference's network benchmark (src/bin/network_bench.rs:41-215):
    7x7 stride-4 stem on 224x224 (no max-pool), four stages of two basic blocks (64/128/256/512
    filters, the first block of stages 2-4 at stride 2 with a 1x1 shortcut), global average pool,
    1000-way linear layer.  Two differences, both needed to run it on the matrix-core kernels:
    every BatchNorm carries its four parameter vectors as Input nodes, so that the fusion rules
    merge it (the reference's benchmark graph leaves them out and its BatchNorms stay
    standalone), and the image has 8 channels (3 used, 5 zero) because the convolution reads
    16-byte channel groups.

    Returns (graph, info): info["convs"] maps op_id -> (k, r, s, c), info["bn"] maps the op_id of
    every BatchNorm to its 4 parameter Input ids and channel count, info["input"] / ["fc"] /
    ["output"] name the image Input, the Linear node and the last node."""
    ops, deps = [], []
    info = {"convs": {}, "bn": {}}
    counter = [0]

    def new_id():
        counter[0] += 1
        return counter[0]

    def add(node, *producers):
        oid = _kind(node)[1]["op_id"]
        ops.append(node)
        for p in producers:
            deps.append([p, oid])
        return oid

    def conv(name, src, c, h, k, r, stride, pad):
        oid = new_id()
        info["convs"][oid] = (k, r, r, c)
        return add(conv2d_node(oid, name, batch, c, h, h, k, r, r, stride, pad), src)

    def bn(name, src, c, h):
        oid = new_id()
        params = []
        for p in ("gamma", "beta", "mean", "var"):
            pid = new_id()
            ops.append(input_node(pid, "%s_%s" % (name, p)))
            params.append(pid)
        info["bn"][oid] = (params, c)
        return add(batchnorm_node(oid, name, batch, c, h, h), src, *params)

    def relu(name, src, c, h):
        return add(relu_node(new_id(), name, batch * c * h * h), src)

    image = new_id()
    ops.append(input_node(image, "input"))
    info["input"] = image
    cur = conv("stem_conv", image, in_channels, 224, 64, 7, 4, 3)
    cur = bn("stem_bn", cur, 64, 56)
    cur = relu("stem_relu", cur, 64, 56)
    size = 56
    for in_c, out_c, stride in ((64, 64, 1), (64, 128, 2), (128, 256, 2), (256, 512, 2)):
        block_in = in_c
        for i in range(2):
            s = stride if i == 0 else 1
            out_size = (size + 2 - 3) // s + 1
            shortcut = cur
            tag = "layer_%d_block_%d" % (out_c, i)
            cur = conv(tag + "_conv1", cur, block_in, size, out_c, 3, s, 1)
            cur = bn(tag + "_bn1", cur, out_c, out_size)
            cur = relu(tag + "_relu1", cur, out_c, out_size)
            cur = conv(tag + "_conv2", cur, out_c, out_size, out_c, 3, 1, 1)
            main = bn(tag + "_bn2", cur, out_c, out_size)
            if block_in != out_c or s != 1:
                sc = conv(tag + "_shortcut_conv", shortcut, block_in, size, out_c, 1, s, 0)
                shortcut = bn(tag + "_shortcut_bn", sc, out_c, out_size)
            cur = add(add_node(new_id(), tag + "_add", batch * out_c * out_size * out_size), main, shortcut)
            cur = relu(tag + "_relu2", cur, out_c, out_size)
            block_in, size = out_c, out_size
    cur = add(global_avg_pool_node(new_id(), "avgpool", batch, 512, size, size), cur)
    fc = add(linear_node(new_id(), "fc", batch, 1, classes, 512), cur)
    info["fc"] = fc
    info["output"] = fc
    return {"operators": ops, "dependencies": deps}, info
