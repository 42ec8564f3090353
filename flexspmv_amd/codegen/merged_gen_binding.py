"""Launch-binding plan and generator for one fused sub-graph.

The Python call contract is the reference's (codegen/merged_gen_binding.py:27-78, identical on the
CPU side, codegen/merged_gen_binding_cpu.py:25-78)::

    merged_spmv_launch(<non-gather value tensors, placeholder order>,
                       <gather-source value tensors, order of first use>,
                       <one int32 index tensor per unique selector module, "<module>_idx">,
                       row_end_offsets, num_rows, num_cols) -> tuple of outputs | None

Outputs follow the ``outputs`` list: reducer outputs ``[num_rows(, Dim)]``, aggregator outputs
``[Dim]``, map outputs ``[ne(, Dim)]`` (merged_gen_binding.py:112-134).  ``ne`` is the element count
of the first index tensor, else ``num_cols`` (:182-187).  The dtype is dispatched on the first
non-gather value input, else the first gather source (:56-62,143-157); int64 values are accepted only
when that input was traced as int64.

What differs underneath: the reference emits a pybind/torch CUDA translation unit per sub-graph; here
the plan below drives (a) the generated HIP library's C entry points (``include/flexspmv.h``) and
(b) the Python launcher in ``flexspmv_amd/binding.py`` that performs the reference's argument
checks and calls those entry points on the current stream.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Tuple

from ..ir import arg_name, dtype_name, get_dim_length


@dataclass
class OutputSpec:
    name: str
    kind: str  # 'reducer' | 'sum' | 'map'
    dim: int
    shape: Tuple[int, ...]


@dataclass
class BindingPlan:
    non_gather_value_inputs: List[str]
    gather_value_inputs: List[str]
    selector_inputs: List[str]          # unique selector module names, first-appearance order
    outputs: List[OutputSpec]
    dispatch_tensor: str
    allow_int64: bool
    value_dims: Dict[str, int] = field(default_factory=dict)

    @property
    def value_inputs(self) -> List[str]:
        return self.non_gather_value_inputs + self.gather_value_inputs

    @property
    def bind_params(self) -> List[Tuple[str, str]]:
        """(name, kind) of every positional argument, kind in value | index | size."""
        params = [(n, "value") for n in self.value_inputs]
        params += [(s + "_idx", "index") for s in self.selector_inputs]
        params += [("row_end_offsets", "index"), ("num_rows", "size"), ("num_cols", "size")]
        return params

    @property
    def has_reducer(self) -> bool:
        return any(o.kind == "reducer" for o in self.outputs)


def output_kind(out: Dict[str, Any]) -> str:
    target = str(out["target"])
    if target == "reducer":
        return "reducer"
    if "sum" in target:
        return "sum"
    return "map"


def binding_plan(inputs, outputs, selector_register) -> BindingPlan:
    """Argument grouping exactly as the reference's binding generator derives it."""
    gather_targets = {s["target"] for s in selector_register if s.get("selector") == 1}
    value_inputs = [i for i in inputs if i["dtype"] != "int"]

    selector_inputs: List[str] = []
    for i in inputs:
        if i["dtype"] == "int" and i["target"] not in selector_inputs:
            selector_inputs.append(i["target"])

    non_gather = [i for i in value_inputs if i["name"] not in gather_targets]
    gather: List[Dict[str, Any]] = []
    seen = set()
    for i in inputs:
        if i["op"] != "call_module":
            continue
        src = arg_name(i["args"][0])
        if src in gather_targets and src not in seen:
            for cand in inputs:
                if cand["name"] == src:
                    gather.append(cand)
                    break
            seen.add(src)

    dispatch = non_gather[0] if non_gather else (gather[0] if gather else value_inputs[0])
    outs = [OutputSpec(o["name"], output_kind(o), get_dim_length(o["shape"]), tuple(o["shape"]))
            for o in outputs]
    return BindingPlan(
        non_gather_value_inputs=[i["name"] for i in non_gather],
        gather_value_inputs=[i["name"] for i in gather],
        selector_inputs=selector_inputs,
        outputs=outs,
        dispatch_tensor=dispatch["name"],
        allow_int64=dtype_name(dispatch.get("dtype_data", "float32")) == "int64",
        value_dims={i["name"]: get_dim_length(i["shape"]) for i in value_inputs},
    )


def generate_binding_code(project_root, inputs, outputs, selector_register) -> Dict[str, Any]:
    """Describe the binding of a sub-graph as plain data (the ``signature`` a generated library
    reports and the launcher checks against).

    Counterpart of ``generate_binding_code`` (codegen/merged_gen_binding.py:9-237).  ``project_root``
    is accepted for call compatibility and unused: nothing is written into the source tree.
    """
    plan = binding_plan(inputs, outputs, selector_register)
    return {
        "params": [{"name": n, "kind": k} for n, k in plan.bind_params],
        "value_inputs": plan.value_inputs,
        "non_gather_value_inputs": plan.non_gather_value_inputs,
        "gather_value_inputs": plan.gather_value_inputs,
        "index_inputs": [s + "_idx" for s in plan.selector_inputs],
        "value_dims": plan.value_dims,
        "outputs": [{"name": o.name, "kind": o.kind, "dim": o.dim, "shape": list(o.shape)}
                    for o in plan.outputs],
        "dispatch_tensor": plan.dispatch_tensor,
        "allow_int64": plan.allow_int64,
        "has_reducer": plan.has_reducer,
    }
