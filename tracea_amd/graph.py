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
