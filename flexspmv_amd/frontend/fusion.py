"""``compile``: trace a model written against :mod:`flexspmv_amd.frontend.lite` and fuse its dataflow
into select -> map -> reduce / aggregate sub-modules.

The reference gets this from EASIER: ``esr.compile([model], backend)`` returns a module whose
``jit_engine.graph`` holds one ``call_module`` node per fused sub-graph, and whose fused
``torch.fx.GraphModule`` children are what ``trace_graph`` and ``dynamic_replace_submodule`` work on
(easier_spmv.py:143-150, test_full/utils.py, python_wrapper/dynamic_replace_submodule.py:7-18).  This
module provides the same shape of result from plain ``torch.fx``:

1. symbolic trace with ``Selector`` / ``Reducer`` as leaf modules;
2. shape and dtype of every node from a run on ``meta`` tensors (nothing is executed on real data);
3. grouping: every call node gets a *stage* = number of kernel boundaries on the longest path that
   reaches it.  A boundary is an edge that cannot stay inside one fused kernel: out of a ``Reducer`` or
   an aggregating ``sum``, into a ``Selector`` (a gather needs the whole source tensor), between values
   of different leading dimension, and between an in-place write of a model tensor and a gather of the
   same tensor (per-item reads and writes of one tensor may share a kernel).  Nodes of equal stage joined by non-boundary edges form one fused sub-module; pure
   element-wise groups of equal stage and equal length are merged into one;
4. a top-level graph that calls the fused sub-modules in stage order.
"""
from __future__ import annotations

import operator
from types import SimpleNamespace
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
import torch.fx as fx
import torch.nn as nn

from . import lite

INPLACE_METHODS = ("copy_", "add_")


class _Proxy(fx.Proxy):
    """fx proxies reject item assignment; ``tensor[:] = value`` is how the reference's models store
    results (easier_spmv.py:65-68), so it is recorded as an ``operator.setitem`` node."""

    def __setitem__(self, key, value) -> None:
        self.tracer.create_proxy("call_function", operator.setitem, (self, key, value), {})


class _Tracer(fx.Tracer):
    def proxy(self, node: fx.Node) -> fx.Proxy:
        return _Proxy(node, self)

    def is_leaf_module(self, m: nn.Module, qualname: str) -> bool:
        return isinstance(m, (lite.Selector, lite.Reducer)) or super().is_leaf_module(m, qualname)


def _fetch_attr(root: nn.Module, target: str):
    obj = root
    for atom in target.split("."):
        obj = getattr(obj, atom)
    return obj


def _is_write(node: fx.Node) -> Optional[fx.Node]:
    """The get_attr node a call node writes in place, if any."""
    first = node.args[0] if node.args else None
    if not isinstance(first, fx.Node) or first.op != "get_attr":
        return None
    if node.op == "call_function" and node.target in (operator.setitem, operator.iadd):
        return first
    if node.op == "call_method" and node.target in INPLACE_METHODS:
        return first
    return None


def propagate_meta(gm: fx.GraphModule) -> None:
    """Record ``flex_shape`` / ``flex_dtype`` on every node from a run on meta tensors."""
    env: Dict[fx.Node, Any] = {}

    def look(a):
        return fx.node.map_arg(a, lambda n: env[n])

    for node in gm.graph.nodes:
        val = None
        if node.op == "get_attr":
            t = _fetch_attr(gm, node.target)
            val = torch.empty(tuple(t.shape), dtype=t.dtype, device="meta")
        elif node.op == "placeholder":
            raise TypeError("a model's forward() takes no arguments")
        elif node.op == "call_module":
            mod = gm.get_submodule(node.target)
            x = env[node.args[0]]
            if isinstance(mod, lite.Selector):
                val = torch.empty((mod.idx.shape[0],) + tuple(x.shape[1:]), dtype=x.dtype, device="meta")
            elif isinstance(mod, lite.Reducer):
                if x.shape[0] != mod.idx.shape[0]:
                    raise ValueError(f"{node.name}: Reducer over {mod.idx.shape[0]} edges applied to "
                                     f"{x.shape[0]} items")
                val = torch.empty((mod.n,) + tuple(x.shape[1:]), dtype=x.dtype, device="meta")
            else:
                val = mod(*look(node.args), **look(node.kwargs))
        elif node.op == "call_function":
            val = node.target(*look(node.args), **look(node.kwargs))
        elif node.op == "call_method":
            self_obj, *rest = look(node.args)
            val = getattr(self_obj, node.target)(*rest, **look(node.kwargs))
        elif node.op == "output":
            continue
        if val is None and node.args and isinstance(node.args[0], fx.Node):
            val = env[node.args[0]]          # setitem returns None; it has the shape of its target
        env[node] = val
        if isinstance(val, torch.Tensor):
            node.meta["flex_shape"] = tuple(val.shape)
            node.meta["flex_dtype"] = val.dtype


def _kind(gm: fx.GraphModule, node: fx.Node) -> str:
    if node.op == "call_module":
        mod = gm.get_submodule(node.target)
        if isinstance(mod, lite.Selector):
            return "selector"
        if isinstance(mod, lite.Reducer):
            return "reducer"
        return "module"
    if node.op == "call_function" and node.target is lite.sum:
        return "sum"
    return "map"


def _leading(node: fx.Node) -> Optional[int]:
    shape = node.meta.get("flex_shape")
    return shape[0] if shape else None


def group_nodes(gm: fx.GraphModule) -> List[List[fx.Node]]:
    """Fused groups, each in graph order, listed in an order in which they can be executed."""
    nodes = list(gm.graph.nodes)
    order = {n: i for i, n in enumerate(nodes)}
    calls = [n for n in nodes if n.op in ("call_module", "call_function", "call_method")]
    kind = {n: _kind(gm, n) for n in calls}

    # dependencies: (producer, is_boundary)
    deps: Dict[fx.Node, List[Tuple[fx.Node, bool]]] = {n: [] for n in calls}
    last_writer: Dict[str, fx.Node] = {}
    readers: Dict[str, List[fx.Node]] = {}
    # A model tensor that is stored to and read by per-item operations of the same length can stay in one
    # kernel: the item is loaded once, ``x[:] = v`` and ``x.add_(v)`` also update the register copy, and
    # later operations of the kernel see the new value (the reference generates exactly that,
    # codegen/merged_gen_core.py:203-213).  ``copy_`` does not refresh the register, and a gather needs the
    # whole tensor as it is before or after the store, never in between: those cross a kernel boundary.
    def refreshes_register(w: fx.Node) -> bool:
        return w.target is operator.setitem or w.target == "add_"

    for n in calls:
        written = _is_write(n)
        for p in n.all_input_nodes:
            if p.op == "get_attr":
                key = p.target
                if p is written:
                    for r in readers.get(key, []):
                        if r is not n:
                            deps[n].append((r, kind[r] == "selector"))      # write after read
                    if key in last_writer:
                        deps[n].append((last_writer[key], not refreshes_register(last_writer[key])))
                    last_writer[key] = n
                    readers[key] = []
                else:
                    if key in last_writer:                                   # read after write
                        w = last_writer[key]
                        deps[n].append((w, kind[n] == "selector" or not refreshes_register(w)))
                    readers.setdefault(key, []).append(n)
                continue
            if p not in deps:
                continue
            # a reduction consumes edge values: the length that must match is that of its argument
            n_len = _leading(n.args[0]) if kind[n] in ("reducer", "sum") else _leading(n)
            boundary = (kind[p] in ("reducer", "sum", "module") or kind[n] in ("selector", "module")
                        or _leading(p) != n_len)
            deps[n].append((p, boundary))

    stage: Dict[fx.Node, int] = {}
    for n in calls:
        stage[n] = max([stage[p] + (1 if b else 0) for p, b in deps[n]], default=0)

    parent = {n: n for n in calls}

    def find(x):
        while parent[x] is not x:
            parent[x] = parent[parent[x]]
            x = parent[x]
        return x

    def union(a, b):
        ra, rb = find(a), find(b)
        if ra is not rb:
            if order[ra] < order[rb]:
                parent[rb] = ra
            else:
                parent[ra] = rb

    for n in calls:
        for p, b in deps[n]:
            if not b and stage[p] == stage[n]:
                union(p, n)

    groups: Dict[fx.Node, List[fx.Node]] = {}
    for n in calls:
        groups.setdefault(find(n), []).append(n)

    # pure element-wise groups of one stage and one length run as a single flat kernel
    flat: Dict[Tuple[int, Optional[int]], fx.Node] = {}
    for root in sorted(groups, key=lambda r: order[r]):
        members = groups[root]
        if any(kind[m] != "map" for m in members):
            continue
        lead = {_leading(m) for m in members}
        if len(lead) != 1:
            continue
        key = (stage[root], next(iter(lead)))
        if key in flat:
            groups[flat[key]].extend(members)
            groups[root] = []
        else:
            flat[key] = root
    out = [sorted(g, key=lambda m: order[m]) for g in groups.values() if g]
    out.sort(key=lambda g: (stage[g[0]], order[g[0]]))
    return out


def _build_fused(gm: fx.GraphModule, members: Sequence[fx.Node], name: str) -> Tuple[fx.GraphModule, List[fx.Node],
                                                                                     List[fx.Node]]:
    """(fused GraphModule, external input nodes in placeholder order, member nodes it returns)."""
    inside = set(members)
    g = fx.Graph()
    val: Dict[fx.Node, fx.Node] = {}
    externals: List[fx.Node] = []
    for n in members:
        for p in n.all_input_nodes:
            if p not in inside and p not in val:
                ph = g.placeholder(p.name)
                ph.meta.update({k: v for k, v in p.meta.items() if k.startswith("flex_")})
                val[p] = ph
                externals.append(p)
    for n in members:
        new = g.node_copy(n, lambda x: val[x])
        new.meta.update({k: v for k, v in n.meta.items() if k.startswith("flex_")})
        val[n] = new
    returned = [n for n in members if any(u not in inside for u in n.users)]
    g.output([val[n] for n in returned])
    fused = fx.GraphModule(gm, g, class_name=name)
    fused._flexspmv_name = name
    return fused, externals, returned


class CompiledModule(fx.GraphModule):
    """The traced model: calling it runs the fused sub-modules in order.  ``jit_engine.graph`` is the
    top-level graph with one ``call_module`` node per fused sub-module, as in the reference."""

    def __init__(self, root, graph, original: nn.Module, fused_names: List[str]):
        super().__init__(root, graph, class_name=type(original).__name__ + "Compiled")
        self.__dict__["_original"] = original
        self.__dict__["fused_names"] = list(fused_names)
        self.__dict__["jit_engine"] = SimpleNamespace(graph=self.graph)

    def __getattr__(self, name: str):
        try:
            return super().__getattr__(name)
        except AttributeError:
            original = self.__dict__.get("_original")
            if original is None:
                raise
            return getattr(original, name)


def _drop_unused_values(graph: fx.Graph) -> None:
    """Remove call nodes whose value nobody uses, except in-place stores (``x[:] = v``, ``x.copy_(v)``,
    ``x.add_(v)``), which are kept for their effect.  (fx's own dead-code pass does not know that the
    in-place methods have effects.)"""
    changed = True
    while changed:
        changed = False
        for node in reversed(list(graph.nodes)):
            if node.op not in ("call_module", "call_function", "call_method", "get_attr") or node.users:
                continue
            store = (node.op == "call_function" and node.target in (operator.setitem, operator.iadd)) or \
                    (node.op == "call_method" and isinstance(node.target, str) and node.target.endswith("_"))
            if not store:
                graph.erase_node(node)
                changed = True


def compile_module(model: nn.Module) -> CompiledModule:
    traced_graph = _Tracer().trace(model)
    _drop_unused_values(traced_graph)
    gm = fx.GraphModule(model, traced_graph)
    propagate_meta(gm)
    groups = group_nodes(gm)

    top = fx.Graph()
    holder: Dict[str, Any] = {}      # what the top-level module refers to: the model's own tensors (same
    val: Dict[fx.Node, fx.Node] = {}  # storage) and the fused sub-modules
    for n in gm.graph.nodes:
        if n.op == "get_attr":
            val[n] = top.node_copy(n)
            val[n].meta.update(n.meta)
            holder[n.target] = _fetch_attr(model, n.target)
    fused_names: List[str] = []
    for i, members in enumerate(groups):
        kinds = {_kind(gm, m) for m in members}
        tag = "select_reduce" if "reducer" in kinds else ("select_map" if "selector" in kinds else "map")
        name = f"fused{i}_{tag}"
        fused, externals, returned = _build_fused(gm, members, name)
        holder[name] = fused
        call = top.call_module(name, tuple(val[p] for p in externals))
        for k, n in enumerate(returned):
            item = top.call_function(operator.getitem, (call, k))
            item.meta.update({kk: v for kk, v in n.meta.items() if kk.startswith("flex_")})
            val[n] = item
        fused_names.append(name)
    for n in gm.graph.nodes:
        if n.op == "output":
            top.output(fx.node.map_arg(n.args[0], lambda x: val[x]))
    top.lint()
    return CompiledModule(holder, top, model, fused_names)


def init(comm_backend: str = "none") -> None:
    """The reference initialises EASIER's process group here (easier_spmv.py:143); one device, no-op."""


def compile(modules: Sequence[nn.Module], backend: str = "torch", **_ignored) -> List[CompiledModule]:  # noqa: A001
    """``[compiled] = compile([model], backend)`` (easier_spmv.py:144)."""
    return [compile_module(m) for m in modules]
