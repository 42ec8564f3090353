"""Swap a fused fx sub-module of a compiled model for a call into its generated library.

Same surface as the reference (python_wrapper/dynamic_replace_submodule.py): ``get_submodules_wrapper``,
``_coo_rows_to_csr_ptr``, ``_DynamicCudaWrapper`` and ``dynamic_replace_submodule(compiled_eqn, ext,
submodule_name) -> bool``; ``ext`` is any object with ``merged_spmv_launch(<non-gather value tensors in
placeholder order>, <gather sources in order of first use>, <one int32 index tensor per unique selector>,
row_end_offsets, num_rows, num_cols)``.

Deliberate differences:

* selector index tensors are collected in the order in which the fused graph first calls each selector
  module, which is the order the generated binding declares them in (codegen/merged_gen_binding.py:33-38);
  the reference walks ``named_modules()`` and stops at the first Reducer
  (dynamic_replace_submodule.py:65-72), which drops selectors registered after it;
* the reducer's row ids must be sorted for the COO -> CSR conversion to describe them
  (dynamic_replace_submodule.py:20-41 assumes it, and the reference's own toy model draws them unsorted,
  easier_spmv.py:126-127).  ``_coo_rows_to_csr_ptr`` raises on unsorted ids; ``build_wrapper`` handles them:
  it sorts the edges by row once (stable, on the ids' device), permutes the selector index buffers once,
  and per call permutes the streamed edge tensors in and the per-edge results back out;
* outputs are returned in the shapes the fused sub-module itself produces (``[n, 2, 1]`` stays that way).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from .. import formats as _formats
from ..formats import mark_written as _mark_written
from ..frontend.lite import Reducer, Selector
from .edge_order import gather_edges, scatter_edges, stable_sort_by_row


def get_submodules_wrapper(eqn, node_name, run_to_collect=True):
    """``[(fused sub-module, its call_module node)]`` for the node called ``node_name``."""
    if run_to_collect:
        eqn()
    graph = eqn.jit_engine.graph
    found = []
    for node in graph.nodes:
        if node.op == "call_module" and node.name == node_name:
            found.append((eqn.get_submodule(node.target), node))
    return found


def _coo_rows_to_csr_ptr(row_ids: torch.Tensor, num_rows: Optional[int] = None) -> Tuple[torch.Tensor, int]:
    """Sorted COO row ids -> CSR row pointer of length ``num_rows + 1`` (int64, device of ``row_ids``)."""
    if num_rows is None:
        if row_ids.numel() == 0:
            raise RuntimeError("row_ids is empty; cannot infer num_rows")
        num_rows = int(row_ids.max().item()) + 1
    if row_ids.is_cuda:     # the package's own kernel; the reference's int64 result type is kept
        return _formats.coo_rows_to_csr(row_ids, num_rows).to(torch.int64), num_rows
    row_ids = row_ids.to(torch.int64)
    if row_ids.numel() > 1 and bool((row_ids[1:] < row_ids[:-1]).any()):
        raise RuntimeError("Reducer row ids must be sorted ascending for the CSR conversion; sort the edges "
                           "by destination row first (flexspmv_amd.python_wrapper.edge_order)")
    if row_ids.numel() and (int(row_ids.min()) < 0 or int(row_ids.max()) >= num_rows):
        raise RuntimeError("Reducer row ids outside [0, num_rows)")
    counts = torch.bincount(row_ids, minlength=num_rows)
    crow = torch.zeros(num_rows + 1, dtype=torch.int64, device=row_ids.device)
    torch.cumsum(counts, dim=0, out=crow[1:])
    return crow, num_rows


def _iter_placeholders_in_order(gm) -> List[str]:
    return [n.name for n in gm.graph.nodes if n.op == "placeholder"]


def _collect_selector_modules(gm) -> Tuple[List[Tuple[str, nn.Module]], Optional[nn.Module]]:
    """(unique Selector modules in order of first call, the Reducer module or None)."""
    selectors: List[Tuple[str, nn.Module]] = []
    reducer_mod: Optional[nn.Module] = None
    seen = set()
    for node in gm.graph.nodes:
        if node.op != "call_module":
            continue
        mod = gm.get_submodule(node.target)
        if type(mod) is Selector and node.target not in seen:
            seen.add(node.target)
            selectors.append((node.target, mod))
        elif type(mod) is Reducer:
            if reducer_mod is None:
                reducer_mod = mod
            elif mod is not reducer_mod and not (mod.n == reducer_mod.n and torch.equal(mod.idx, reducer_mod.idx)):
                raise RuntimeError("the Reducers of one fused sub-module must share one row structure")
    return selectors, reducer_mod


def _infer_gather_value_inputs(gm, selector_qnames: Iterable[str]) -> List[str]:
    """Placeholders that are gathered through a selector, in order of first use."""
    names: List[str] = []
    wanted = set(selector_qnames)
    for node in gm.graph.nodes:
        if node.op == "call_module" and node.target in wanted:
            for a in node.all_input_nodes:
                if a.op == "placeholder" and a.name not in names:
                    names.append(a.name)
    return names


def _written_inputs(gm) -> List[str]:
    """Placeholders the fused graph stores into (``x[:] = v``, ``x.copy_(v)``, ``x.add_(v)``)."""
    import operator
    out = []
    for node in gm.graph.nodes:
        inplace = (node.op == "call_function" and node.target is operator.setitem) or \
                  (node.op == "call_method" and node.target in ("copy_", "add_"))
        if inplace and node.args and getattr(node.args[0], "op", None) == "placeholder":
            out.append(node.args[0].name)
    return out


def _per_edge_outputs(gm) -> List[bool]:
    """For every returned value: is it a per-edge map result (as opposed to a reducer or an aggregate)?"""
    for node in gm.graph.nodes:
        if node.op == "output":
            returned = node.args[0] if isinstance(node.args[0], (list, tuple)) else [node.args[0]]
            flags = []
            for r in returned:
                reduction = (r.op == "call_module" and type(gm.get_submodule(r.target)) is Reducer) or \
                            (r.op == "call_function" and getattr(r.target, "__name__", "") == "sum")
                flags.append(not reduction)
            return flags
    return []


def _output_shapes(gm) -> List[Tuple[int, ...]]:
    for node in gm.graph.nodes:
        if node.op == "output":
            returned = node.args[0] if isinstance(node.args[0], (list, tuple)) else [node.args[0]]
            return [tuple(r.meta["flex_shape"]) if "flex_shape" in r.meta else () for r in returned]
    return []


class _DynamicCudaWrapper(nn.Module):
    """Callable with the fused sub-module's placeholders; launches the library and returns a list."""

    def __init__(self, ext_module, input_param_names: List[str], non_gather_value_inputs: List[str],
                 gather_value_inputs: List[str], selector_idx_tensors: List[torch.Tensor],
                 row_end_offsets: Optional[torch.Tensor], output_shapes: Optional[List[Tuple[int, ...]]] = None,
                 written_inputs: Iterable[str] = (), edge_permutation: Optional[torch.Tensor] = None,
                 per_edge_outputs: Optional[List[bool]] = None) -> None:
        super().__init__()
        names: List[str] = []
        for i, t in enumerate(selector_idx_tensors):
            t = t.contiguous()
            if t.dtype != torch.int32:
                t = t.to(torch.int32)
            self.register_buffer(f"selector_{i}_idx", t, persistent=False)
            names.append(f"selector_{i}_idx")
        reo = None
        if row_end_offsets is not None:
            reo = row_end_offsets.contiguous()
            if reo.dtype != torch.int32:
                if int(reo[-1]) >= 2 ** 31:
                    raise RuntimeError("row_end_offsets does not fit 32-bit offsets")
                reo = reo.to(torch.int32)
        self.register_buffer("row_end_offsets", reo, persistent=False)
        # edges sorted by row when the model's edge list is not: position k of the kernel's edge order
        # holds the model's edge edge_permutation[k]
        self.register_buffer("edge_permutation", edge_permutation, persistent=False)
        self._per_edge_outputs = list(per_edge_outputs) if per_edge_outputs is not None else None
        self._ext = ext_module
        self._input_param_names = list(input_param_names)
        self._non_gather_value_inputs = list(non_gather_value_inputs)
        self._gather_value_inputs = list(gather_value_inputs)
        self._selector_buf_names = names
        self._output_shapes = list(output_shapes) if output_shapes is not None else None
        self._written_inputs = set(written_inputs)
        self._dummy_ro: Dict[torch.device, torch.Tensor] = {}
        # streamed edge tensors in the kernel's edge order, kept from the previous call: a tensor that has not
        # changed since (same storage, same version counter - a model parameter, a mesh constant) is not
        # permuted again
        self._sorted_inputs: Dict[str, Tuple] = {}

    def _on(self, name: str, device) -> torch.Tensor:
        t = getattr(self, name)
        if t.device != device:       # moved once, then kept: launches must see one unchanged tensor
            t = t.to(device)
            setattr(self, name, t)
        return t

    def _in_edge_order(self, name: str, t: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
        """``t`` permuted into the kernel's edge order; the copy of the previous call when ``t`` is unchanged."""
        if name in self._written_inputs:          # the kernel stores into the copy: always a fresh one
            return gather_edges(t, perm)
        storage = t.untyped_storage()
        key = (storage.data_ptr(), t.storage_offset(), t._version, tuple(t.shape), t.dtype)
        kept = self._sorted_inputs.get(name)
        if kept is not None and kept[0] == key:
            return kept[2]
        out = gather_edges(t, perm)
        # the storage is held so that its address cannot be handed to another tensor while the key is kept
        self._sorted_inputs[name] = (key, storage, out)
        return out

    def __call__(self, *args):
        if len(args) != len(self._input_param_names):
            raise RuntimeError(f"fused sub-module takes {len(self._input_param_names)} tensors, {len(args)} given")
        for n, a in zip(self._input_param_names, args):
            if n in self._written_inputs and not a.is_contiguous():
                raise RuntimeError(f"{n} is written in place by the fused kernel and must be contiguous")
        arg_map = {n: a.contiguous() for n, a in zip(self._input_param_names, args)}
        device = next(iter(arg_map.values())).device

        if self.row_end_offsets is not None:
            ro = self._on("row_end_offsets", device)
            num_rows = int(ro.numel() - 1)
        else:
            ro = self._dummy_ro.get(device)
            if ro is None:          # no reducer: the binding still takes a tensor here
                ro = torch.tensor([42], dtype=torch.int32, device=device)
                self._dummy_ro[device] = ro
            num_rows = None
        gv = self._gather_value_inputs[0] if self._gather_value_inputs else self._non_gather_value_inputs[0]
        num_cols = int(arg_map[gv].shape[0])
        if num_rows is None:
            num_rows = num_cols

        perm = None
        if self.edge_permutation is not None:
            perm = self._on("edge_permutation", device)
            if perm.is_cuda and perm.dtype != torch.int32:      # the permutation kernels take int32
                perm = perm.to(torch.int32)
                self.edge_permutation = perm
            for n in self._non_gather_value_inputs:
                arg_map[n] = self._in_edge_order(n, arg_map[n], perm)
        call_args = [arg_map[n] for n in self._non_gather_value_inputs]
        call_args += [arg_map[n] for n in self._gather_value_inputs]
        call_args += [self._on(b, device) for b in self._selector_buf_names]
        call_args += [ro, num_rows, num_cols]

        outs = self._ext.merged_spmv_launch(*call_args)
        # The kernel stored into the written inputs through raw pointers: their version counters go up as they
        # would after torch's own in-place operations, so that nobody (this class's copies of unchanged edge
        # tensors in another wrapper included) mistakes them for unchanged.
        for n, a in zip(self._input_param_names, args):
            if n in self._written_inputs:
                if perm is not None and n in self._non_gather_value_inputs:
                    scatter_edges(arg_map[n], perm, out=a)      # stores went to the sorted copy: put them back
                _mark_written(a)
        if outs is None:
            return []
        outs = list(outs) if isinstance(outs, (tuple, list)) else [outs]
        if perm is not None and self._per_edge_outputs is not None:
            outs = [scatter_edges(o, perm) if per_edge else o
                    for o, per_edge in zip(outs, self._per_edge_outputs)]
        if self._output_shapes is not None and len(self._output_shapes) == len(outs):
            outs = [o.view(s) if s and o.numel() == _numel(s) else o for o, s in zip(outs, self._output_shapes)]
        return outs


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


def build_wrapper(gm, ext) -> _DynamicCudaWrapper:
    """The wrapper for one fused sub-module ``gm``."""
    input_param_names = _iter_placeholders_in_order(gm)
    selector_modules, reducer_mod = _collect_selector_modules(gm)
    selector_idx_tensors = [mod.idx for _, mod in selector_modules]
    edge_permutation = None
    if reducer_mod is not None:
        row_ids, num_rows = reducer_mod.idx, int(reducer_mod.n)
        if row_ids.is_cuda:         # one pass answers "ascending?" and, if so, already is the row pointer
            row_end_offsets, findings = _formats.coo_rows_to_csr_async(row_ids, num_rows)
            found = int(findings[0])
            if found & _formats.FINDING_OUT_OF_RANGE:
                raise RuntimeError("Reducer row ids outside [0, num_rows)")
            unsorted = bool(found & _formats.FINDING_UNSORTED)
        else:
            unsorted = row_ids.numel() > 1 and bool((row_ids[1:] < row_ids[:-1]).any())
        if unsorted:
            row_ids, edge_permutation = stable_sort_by_row(row_ids, num_rows)
            selector_idx_tensors = [gather_edges(t, edge_permutation) for t in selector_idx_tensors]
        if unsorted or not row_ids.is_cuda:
            row_end_offsets, _ = _coo_rows_to_csr_ptr(row_ids, num_rows)
    else:
        row_end_offsets = None
    gather_value_inputs = _infer_gather_value_inputs(gm, [q for q, _ in selector_modules])
    non_gather_value_inputs = [n for n in input_param_names if n not in gather_value_inputs]
    wrapper = _DynamicCudaWrapper(ext, input_param_names, non_gather_value_inputs, gather_value_inputs,
                                  selector_idx_tensors, row_end_offsets, _output_shapes(gm), _written_inputs(gm),
                                  edge_permutation, _per_edge_outputs(gm))
    names = getattr(ext, "param_names", None)
    if callable(names):             # a library of this package knows its own argument list: cross-check
        expected = non_gather_value_inputs + gather_value_inputs
        declared = names()
        n_idx = len(selector_idx_tensors)
        if declared[:len(expected)] != expected or len(declared) != len(expected) + n_idx + 3:
            raise RuntimeError(f"library arguments {declared} do not match the fused sub-module "
                               f"({expected} + {n_idx} index tensors)")
    return wrapper


def dynamic_replace_submodule(compiled_eqn: nn.Module, ext, submodule_name) -> bool:
    """Replace the fused sub-module called by node ``submodule_name`` with a launch of ``ext``."""
    for gm, node in get_submodules_wrapper(compiled_eqn, submodule_name, run_to_collect=False):
        if node.name != submodule_name:
            continue
        setattr(compiled_eqn, node.target, build_wrapper(gm, ext))
        return True
    return False
