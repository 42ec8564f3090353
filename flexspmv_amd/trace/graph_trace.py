"""``trace_graph``: one fused fx sub-module -> the six lists every generator consumes.

Same call and same result schema as the reference (trace/graph_trace.py:32-328): ``inputs``,
``outputs``, ``selector_register``, ``map_operations``, ``reducer_operations``,
``aggregator_operations`` (the keys are listed in :mod:`flexspmv_amd.ir`).  Two things are done
differently on purpose:

* operations are classified by the identity of the call target, not by searching the target's
  ``repr`` for substrings in a fixed priority (trace/graph_trace.py:229-276), which misfiles any target
  whose text happens to contain an earlier keyword;
* node metadata (shape without the leading dimension, dtype) is read from ``node.meta`` as recorded by
  :func:`flexspmv_amd.frontend.fusion.propagate_meta` instead of EASIER's metadata pass
  (trace/graph_trace.py:10-29).

A selector whose index tensor equals the group's reducer index is marked ``row_aligned``: a kernel may
then take the row id from the merge path instead of reading that index array.
"""
from __future__ import annotations

import operator
from typing import Any, Dict, List, Tuple

import torch
import torch.fx as fx

from ..frontend import lite
from ..ir import GraphBuilder, dtype_name

# call_function targets by identity
_FUNCTIONS = {
    operator.add: "add", torch.add: "add",
    operator.sub: "sub", torch.sub: "sub",
    operator.mul: "mul", torch.mul: "mul",
    operator.truediv: "truediv", torch.div: "truediv", torch.true_divide: "truediv",
    operator.neg: "neg", torch.neg: "neg", torch.negative: "neg",
    operator.pow: "pow", torch.pow: "pow",
    operator.lt: "lt", torch.lt: "lt",
    operator.gt: "gt", torch.gt: "gt",
    operator.getitem: "getitem", operator.setitem: "setitem",
    operator.abs: "abs", torch.abs: "abs",
    torch.exp: "exp", torch.sign: "sign", torch.where: "where", torch.clone: "clone",
    lite.norm: "norm", lite.sum: "sum",
}
# call_method targets by name (exact match)
_METHODS = {
    "add": "add", "sub": "sub", "mul": "mul", "div": "truediv", "true_divide": "truediv", "neg": "neg",
    "pow": "pow", "lt": "lt", "gt": "gt", "abs": "abs", "exp": "exp", "sign": "sign", "where": "where",
    "clone": "clone", "copy_": "copy_", "add_": "add_",
}


def _item_shape(node: fx.Node) -> Tuple[int, ...]:
    shape = tuple(node.meta["flex_shape"][1:])
    return shape if shape else (1,)


def get_node_info(node: fx.Node):
    """(shape without the leading dimension, op, name, target, args, dtype) of one node
    (trace/graph_trace.py:10-29)."""
    return _item_shape(node), node.op, node.name, node.target, node.args, node.meta.get("flex_dtype")


def classify(node: fx.Node) -> str:
    """Operation name of a call_function / call_method node; ValueError for anything the generators
    do not implement, with the reference's message (trace/graph_trace.py:277-279)."""
    if node.op == "call_function" and node.target in _FUNCTIONS:
        return _FUNCTIONS[node.target]
    if node.op == "call_method" and node.target in _METHODS:
        return _METHODS[node.target]
    raise ValueError(f"Operation {node.target} not supported")


def _plain_args(node: fx.Node) -> List[Any]:
    if node.kwargs:
        raise ValueError(f"Operation {node.target} not supported with keyword arguments {dict(node.kwargs)}")
    return [a.name if isinstance(a, fx.Node) else a for a in node.args]


def trace_graph(submodule: fx.GraphModule, traced_model=None):
    """Six lists for one fused sub-module.  ``traced_model`` is accepted for call compatibility with the
    reference, which reads placeholder metadata from it; here every node carries its own."""
    nodes = list(submodule.graph.nodes)
    modules: Dict[str, Any] = {n.target: submodule.get_submodule(n.target) for n in nodes if n.op == "call_module"}
    reducers = [m for m in modules.values() if isinstance(m, lite.Reducer)]
    first = next((n for n in nodes if n.op == "placeholder"), None)
    if first is None:
        raise ValueError("a fused sub-module without tensor inputs cannot be generated")
    b = GraphBuilder(getattr(submodule, "_flexspmv_name", type(submodule).__name__), dtype_name(first.meta["flex_dtype"]))

    # Every streamed tensor and every per-edge value of one kernel is indexed by the same edge id; a
    # tensor of another length (say a [1]-long aggregate broadcast over the edges) cannot take part.
    gathered = {n.args[0] for n in nodes if n.op == "call_module" and isinstance(modules[n.target], lite.Selector)}
    lengths = set()
    for node in nodes:
        if node.op == "placeholder" and node not in gathered:
            lengths.add(node.meta["flex_shape"][0])
        elif node.op in ("call_function", "call_method") or \
                (node.op == "call_module" and isinstance(modules[node.target], lite.Selector)):
            if not (node.op == "call_function" and node.target is lite.sum):
                lengths.add(node.meta["flex_shape"][0])
    if len(lengths) > 1:
        raise ValueError(f"Operation over tensors of different lengths {sorted(lengths)} not supported "
                         "(no broadcasting along the edge dimension)")

    for node in nodes:
        if node.op == "placeholder":
            b.placeholder(node.name, _item_shape(node))
        elif node.op == "call_module":
            mod = modules[node.target]
            if isinstance(mod, lite.Selector):
                aligned = any(mod.idx.shape == r.idx.shape and bool(torch.equal(mod.idx.long(), r.idx.long()))
                              for r in reducers)
                b.select(node.name, node.args[0].name, module=node.target, row_aligned=aligned)
            elif isinstance(mod, lite.Reducer):
                b.reduce(node.name, node.args[0].name, module=node.target)
            else:
                raise ValueError(f"Operation {type(mod).__name__} not supported")
        elif node.op in ("call_function", "call_method"):
            op = classify(node)
            if op == "sum":
                b.aggregate(node.name, node.args[0].name)
                continue
            args = _plain_args(node)
            if op == "getitem":
                index = args[1]
                ok = (isinstance(index, tuple) and len(index) == 2 and index[0] == slice(None, None, None)
                      and isinstance(index[1], int))
                if not ok:            # only x[:, i] exists in the generators (codegen/merged_gen_core.py:186-190)
                    raise ValueError(f"Operation getitem{index!r} not supported")
            if op == "setitem":
                index = args[1]
                if index not in (slice(None, None, None), (slice(None, None, None),), Ellipsis):
                    raise ValueError(f"Operation setitem{index!r} not supported")
                args = [args[0], (slice(None, None, None),), args[2]]
            b.map(op, node.name, args, shape=_item_shape(node))
        elif node.op == "output":
            returned = node.args[0] if isinstance(node.args[0], (list, tuple)) else [node.args[0]]
            b.output(*[r.name for r in returned])
        elif node.op == "get_attr":
            raise ValueError("a fused sub-module takes its tensors as arguments")
    ir = b.build()
    return ir.six()
