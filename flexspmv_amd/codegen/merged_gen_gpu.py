"""Emit the HIP translation unit (gfx950) for one fused sub-graph.

Counterpart of ``generate_cuda_code_from_graph`` (codegen/merged_gen_gpu.py:17-465).  The reference
pastes per-op statements into CUB-derived agent templates; here the statements are pasted into a graph
type ``Graph<ValueT>`` consumed by the hand-written kernels of ``csrc/flex_agent.hpp``:

* selector statements follow the reference's emitters (codegen/merged_gen_gpu.py:157-181,
  codegen/merged_gen_core.py:91-114): an edge tensor is ``Dim`` contiguous values at ``edge*Dim``, a
  vertex tensor ``Dim`` contiguous values at ``idx[edge]*Dim``;
* map statements cover the reference's op set with its operator spelling
  (codegen/merged_gen_gpu.py:188-298): ``add sub mul pow truediv neg add_ exp norm getitem clone copy_
  setitem abs sign lt gt where`` (``reducer`` / ``sum`` are routed to the reduction machinery);
* a kernel may hold reducers AND aggregators (the reference's templates hold one or the other,
  codegen/merged_gen_gpu.py:394).

What a generated ``Graph`` splits by memory level, because the kernels schedule the levels differently
from the reference's one-statement-after-the-other body:

* ``Fetch``   what is streamed per edge (edge tensors, selector indices): loaded in coalesced order and
  handed through LDS to the thread that owns the edge's row;
* ``Gather``  vertex data addressed through ``Fetch`` - gathered by the row's thread, so that
  neighbouring lanes (neighbouring rows) gather neighbouring vertices;
* ``Row``     sources of ``row_aligned`` selectors (index array == the reducer's row ids): read once
  per row at the row id, the index array is never touched;
* ``edge()``  the whole map for one edge: contributions to the reducers and the aggregators.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

from ..ir import FusedGraphIR, arg_name, dtype_name, get_dim_length
from .merged_gen_binding import BindingPlan, binding_plan, generate_binding_code

VERBOSE_ENV = "EASIER_VERBOSE_CODEGEN"  # same switch as the reference (codegen/merged_gen_gpu.py:140)

# LDS a reducer block may use for the per-edge hand-over (keeps >= 4 blocks per CU: 160 KiB LDS per CU
# on gfx950).
LDS_BUDGET_BYTES = 36 * 1024
BLOCK_THREADS = 256


@dataclass
class Var:
    name: str
    kind: str          # 'tensor' | 'scalar'
    dim: int
    ctype: str         # C++ type name inside Graph<ValueT>


@dataclass
class KernelPlan:
    plan: BindingPlan
    vars: Dict[str, Var]
    fetch_values: List[Tuple[str, str, int, int]]     # (variable, source tensor, dim, first value slot)
    fetch_indices: List[Tuple[str, int]]              # (selector module, index slot)
    gathers: List[Tuple[str, str, str, int]]          # (variable, selector module, source tensor, dim)
    row_sources: List[Tuple[str, str, int, int]]      # (selector var, source tensor, dim, first slot)
    red_slices: List[Tuple[str, int, int]]            # (reducer name, first slot, dim)
    agg_slices: List[Tuple[str, int, int]]
    fetch_value_width: int = 0
    fetch_index_width: int = 0
    red_width: int = 0
    agg_width: int = 0
    row_width: int = 0


def _literal(a: Any) -> str:
    if isinstance(a, bool):
        return "1" if a else "0"
    if isinstance(a, int):
        return str(a)
    if isinstance(a, float):
        return repr(a)
    raise TypeError(f"unsupported literal {a!r}")


def analyse(ir: FusedGraphIR) -> KernelPlan:
    """Variable table and memory-level split of a sub-graph (raises ``ValueError`` for an operation the
    generators cannot express)."""
    inputs, outputs, selector_register, map_ops, red_ops, agg_ops = ir.six()
    plan = binding_plan(inputs, outputs, selector_register)
    has_reducer = bool(red_ops)
    vars: Dict[str, Var] = {}
    fetch_values: List[Tuple[str, str, int, int]] = []
    fetch_indices: List[Tuple[str, int]] = []
    gathers: List[Tuple[str, str, str, int]] = []
    row_sources: List[Tuple[str, str, int, int]] = []
    value_slot = row_slot = 0
    index_slot: Dict[str, int] = {}
    for s in selector_register:
        dim = get_dim_length(s["shape"])
        ctype = f"TensorInput_{s['target']}_T"
        if s["selector"] != 1:
            var = s["selector_name"]
            fetch_values.append((var, s["target"], dim, value_slot))
            value_slot += dim
        elif s.get("row_aligned") and has_reducer:
            var = s["name"]
            row_sources.append((var, s["target"], dim, row_slot))
            row_slot += dim
        else:
            var = s["name"]
            module = s["selector_name"]
            if module not in index_slot:
                index_slot[module] = len(fetch_indices)
                fetch_indices.append((module, index_slot[module]))
            gathers.append((var, module, s["target"], dim))
        vars[var] = Var(var, "tensor", dim, ctype)

    for op in map_ops:
        o = op["op"]
        if o in ("reducer", "sum", "setitem", "copy_", "add_"):
            continue
        dim = get_dim_length(op["shape"])
        if o == "norm":
            vars[op["name"]] = Var(op["name"], "scalar", 1, "ValueT")
        else:
            vars[op["name"]] = Var(op["name"], "tensor", dim, f"TensorOutput_{op['name']}_T")

    red_slices, agg_slices = [], []
    off = 0
    for r in red_ops:
        dim = get_dim_length(r["shape"])
        red_slices.append((r["name"], off, dim))
        off += dim
    red_width = off
    off = 0
    for g in agg_ops:
        dim = get_dim_length(g["shape"])
        agg_slices.append((g["name"], off, dim))
        off += dim
    return KernelPlan(plan, vars, fetch_values, fetch_indices, gathers, row_sources, red_slices, agg_slices,
                      fetch_value_width=value_slot, fetch_index_width=len(fetch_indices), red_width=red_width,
                      agg_width=off, row_width=row_slot)


# ------------------------------------------------------------------------------------------
# statement emitters
# ------------------------------------------------------------------------------------------
def _arg(a: Any) -> str:
    a = arg_name(a)
    return a if isinstance(a, str) else _literal(a)


def _store_loop(ptr: str, edge: str, dim: int, src: str, src_dim: int) -> List[str]:
    return [f"flex::stream_store({ptr} + (size_t){edge} * {dim} + {i}, {src}.values[{i % src_dim}]);"
            for i in range(dim)]


def _emit_map(op: Dict[str, Any], vars: Dict[str, Var], edge: str) -> List[str]:
    o, name = op["op"], op["name"]
    a = [_arg(x) for x in op["args"]] if o not in ("getitem", "setitem") else None
    T = f"TensorOutput_{name}_T"
    binary = {"add": "+", "sub": "-", "mul": "*", "pow": "^", "truediv": "/", "lt": "<", "gt": ">"}
    if o == "pow" and isinstance(op["args"][1], (int, float)) and not isinstance(op["args"][1], bool) \
            and isinstance(arg_name(op["args"][0]), str):
        # literal exponents 0.5 and 1..4 take the direct form (same value to within an ulp of pow)
        e = op["args"][1]
        base = vars.get(a[0])
        scalar = base is not None and base.kind == "scalar"
        if e == 0.5:
            return [f"{T} {name}(flex::v_sqrt({a[0]}));" if scalar else f"{T} {name} = {a[0]}.sqrt();"]
        if float(e).is_integer() and 1 <= int(e) <= 4:
            return [f"{T} {name}(flex::v_ipow<{int(e)}>({a[0]}));" if scalar
                    else f"{T} {name} = {a[0]}.template ipow<{int(e)}>();"]
    if o == "truediv" and isinstance(arg_name(op["args"][0]), str) and isinstance(arg_name(op["args"][1]), str):
        num, den = vars.get(a[0]), vars.get(a[1])
        if num is not None and den is not None and num.kind == "tensor" and num.dim > 1 and den.kind == "scalar":
            # a tensor of several values over a scalar (a vector over its norm): one reciprocal, then products
            return [f"{T} {name} = flex::times_reciprocal({a[0]}, {a[1]});"]
    if o in binary:
        return [f"{T} {name} = {a[0]} {binary[o]} {a[1]};"]
    if o == "neg":
        return [f"{T} {name} = -{a[0]};"]
    if o in ("exp", "abs", "sign"):
        return [f"{T} {name} = {a[0]}.{o}();"]
    if o == "norm":
        return [f"const ValueT {name} = {a[0]}.l2Norm();"]
    if o == "where":
        return [f"{T} {name} = flex::_where({a[0]}, {a[1]}, {a[2]});"]
    if o == "clone":
        return [f"{T} {name}({a[0]});"]
    if o == "getitem":
        var = _arg(op["args"][0])
        index = op["args"][1][1]
        return [f"{T} {name}({var}.values[{int(index)}]);"]
    dim = get_dim_length(op["shape"])
    if o == "copy_":
        dst, src = a[0], a[1]
        return _store_loop(f"q_p.{dst}_ptr", edge, dim, src, vars[src].dim)
    if o == "add_":
        dst = a[0]
        return [f"{dst} = {dst} + {a[1]};"] + _store_loop(f"q_p.{dst}_ptr", edge, dim, dst, vars[dst].dim)
    if o == "setitem":
        dst, src = _arg(op["args"][0]), _arg(op["args"][2])
        sd = vars[src].dim
        lines = _store_loop(f"q_p.{dst}_ptr", edge, dim, src, sd)
        lines += [f"{dst}.values[{i}] = {src}.values[{i % sd}];" for i in range(dim)]
        return lines
    raise ValueError(f"Operation {o} not supported")


def _component(var: Var, c: int) -> str:
    return var.name if var.kind == "scalar" else f"{var.name}.values[{c}]"


def _indent(lines: Sequence[str], n: int = 4) -> str:
    pad = " " * n
    return "".join(pad + l + "\n" for l in lines)


def _choose_ipt(kp: KernelPlan, value_bytes: int) -> int:
    """Items per thread so that one block's LDS stays inside LDS_BUDGET_BYTES."""
    # LDS holds what is fetched per edge of a tile and, in the merge path, one finished total per row
    per_item = max(value_bytes * kp.fetch_value_width + 4 * kp.fetch_index_width, value_bytes * kp.red_width, 1)
    for ipt in (8, 4, 2, 1):
        if BLOCK_THREADS * ipt * per_item <= LDS_BUDGET_BYTES:
            return ipt
    return 1


def generate_hip_source(ir: FusedGraphIR, dtypes: Optional[Sequence[str]] = None,
                        policy: Optional[Dict[str, int]] = None,
                        defines: Sequence[str] = ()) -> Tuple[str, Dict[str, Any]]:
    """Return (translation unit text, signature dict) for a sub-graph.

    ``dtypes`` lists the value types to instantiate (default float32 + float64, plus int64 when the
    dispatch input was traced as int64 - the reference's rule, codegen/merged_gen_binding.py:143-157).
    ``policy`` may override ``block``, ``ipt_f32``, ``ipt_f64`` and ``ipt_flat``.
    ``defines`` are the ``FLEX_TUNE_*`` switches (``NAME`` or ``NAME=VALUE``) the library will be compiled
    with.  A library with a policy override or switches is a measurement variant: both are recorded in the
    signature (``"tuning"``, ``"policy_override"``), and loaders of product libraries refuse it.
    """
    inputs, outputs, selector_register, map_ops, red_ops, agg_ops = ir.six()
    kp = analyse(ir)
    plan = kp.plan
    has_reducer = bool(red_ops)
    if dtypes is None:
        dtypes = ["float32", "float64"] + (["int64"] if plan.allow_int64 else [])
    dtypes = [dtype_name(d) for d in dtypes]
    policy = dict(policy or {})
    defines = sorted(str(d) for d in defines)
    for d in defines:
        if not d.startswith("FLEX_TUNE_"):
            raise ValueError(f"{d!r} is not a tuning switch (FLEX_TUNE_*)")
    block = int(policy.get("block", BLOCK_THREADS))
    ipt = {"float32": int(policy.get("ipt_f32", _choose_ipt(kp, 4))),
           "float64": int(policy.get("ipt_f64", _choose_ipt(kp, 8))),
           "int64": int(policy.get("ipt_f64", _choose_ipt(kp, 8)))}
    if not has_reducer:
        ipt = {k: int(policy.get("ipt_flat", 8)) for k in ipt}

    # ---- Params ---------------------------------------------------------------------------
    params, fill = [], []
    for i, n in enumerate(plan.value_inputs):
        params.append(f"ValueT* __restrict__ {n}_ptr;")
        fill.append(f"q_p.{n}_ptr = static_cast<ValueT*>(a->value_inputs[{i}]);")
    for i, s in enumerate(plan.selector_inputs):
        params.append(f"const OffsetT* __restrict__ {s}_idx_ptr;")
        fill.append(f"q_p.{s}_idx_ptr = a->index_inputs[{i}];")
    for i, o in enumerate(plan.outputs):
        params.append(f"ValueT* __restrict__ output_y_{o.name}_ptr;")
        fill.append(f"q_p.output_y_{o.name}_ptr = static_cast<ValueT*>(a->outputs[{i}]);")

    # ---- typedefs -------------------------------------------------------------------------
    typedefs, seen = [], set()
    for i in inputs:
        if i["dtype"] != "int" and i["target"] not in seen:
            typedefs.append(f"typedef flex::Tensor<ValueT, {get_dim_length(i['shape'])}> TensorInput_{i['target']}_T;")
            seen.add(i["target"])
    for op in map_ops:
        if op["op"] not in ("reducer", "sum", "norm", "setitem", "copy_", "add_"):
            typedefs.append(f"typedef flex::Tensor<ValueT, {get_dim_length(op['shape'])}> TensorOutput_{op['name']}_T;")

    # ---- memory levels --------------------------------------------------------------------
    fetch_members, fetch_body, put_body, get_body = [], [], [], []
    gather_members, gather_body = [], []
    body: List[str] = []          # edge(): prologue, map operations, reducer / aggregator arguments
    for var, target, dim, first in kp.fetch_values:
        T = kp.vars[var].ctype
        fetch_members.append(f"{T} {var};")
        fetch_body += [f"q_f.{var}.values[{i}] = flex::stream_load(q_p.{target}_ptr + (size_t)q_e * {dim} + {i});"
                       for i in range(dim)]
        put_body += [f"q_sv[{first + i} * TILE + q_j] = q_f.{var}.values[{i}];" for i in range(dim)]
        get_body += [f"q_f.{var}.values[{i}] = q_sv[{first + i} * TILE + q_j];" for i in range(dim)]
        body.append(f"{T} {var} = q_f.{var};")
    for module, slot in kp.fetch_indices:
        fetch_members.append(f"OffsetT index_{module};")
        fetch_body.append(f"q_f.index_{module} = flex::stream_load(q_p.{module}_idx_ptr + q_e);")
        put_body.append(f"q_si[{slot} * TILE + q_j] = q_f.index_{module};")
        get_body.append(f"q_f.index_{module} = q_si[{slot} * TILE + q_j];")
    for var, module, target, dim in kp.gathers:
        T = kp.vars[var].ctype
        gather_members.append(f"{T} {var};")
        gather_body.append(f"q_g.{var} = {T}::gathered(q_p.{target}_ptr + (size_t)q_f.index_{module} * {dim});")
        body.append(f"{T} {var} = q_g.{var};")
    # every streamed word an array of its own (edge tensors of width 1, index arrays): a tile's slice of it
    # can then be copied as it lies in memory
    fetch_contiguous = all(dim == 1 for _, _, dim, _ in kp.fetch_values)
    value_streams = [f"if (q_w == {first}) return q_p.{target}_ptr;" for _, target, dim, first in kp.fetch_values
                     if fetch_contiguous]
    index_streams = [f"if (q_w == {slot}) return q_p.{module}_idx_ptr;" for module, slot in kp.fetch_indices]
    load_row = []
    for var, target, dim, first in kp.row_sources:
        load_row += [f"q_rv.v[{first + i}] = q_p.{target}_ptr[(size_t)q_row * {dim} + {i}];" for i in range(dim)]
        body.append(f"{kp.vars[var].ctype} {var};")
        body += [f"{var}.values[{i}] = q_rv.v[{first + i}];" for i in range(dim)]

    map_output_names = {o.name: o for o in plan.outputs if o.kind == "map"}
    for op in map_ops:
        if op["op"] in ("reducer", "sum"):
            continue
        body.extend(_emit_map(op, kp.vars, "q_e"))
        if op["name"] in map_output_names:
            out = map_output_names[op["name"]]
            v = kp.vars[op["name"]]
            if v.kind == "scalar":
                body.append(f"flex::stream_store(q_p.output_y_{out.name}_ptr + (size_t)q_e, {v.name});")
            else:
                body.extend(_store_loop(f"q_p.output_y_{out.name}_ptr", "q_e", out.dim, v.name, v.dim))
    # a map output may also be a selector / input variable
    for name, out in map_output_names.items():
        if not any(op["name"] == name for op in map_ops):
            v = kp.vars[name]
            body.extend(_store_loop(f"q_p.output_y_{out.name}_ptr", "q_e", out.dim, v.name, v.dim))
    for (rname, first, dim), r in zip(kp.red_slices, red_ops):
        v = kp.vars[arg_name(r["args"][0])]
        body += [f"q_tot.v[{first + c}] = {_component(v, c % v.dim)};" for c in range(dim)]
    for (gname, first, dim), g in zip(kp.agg_slices, agg_ops):
        v = kp.vars[arg_name(g["args"][0])]
        body += [f"q_agg.v[{first + c}] = {_component(v, c % v.dim)};" for c in range(dim)]
    edge_pure = not any("stream_store(" in line for line in body)

    store_row, add_row, store_agg = [], [], []
    for (rname, first, dim) in kp.red_slices:
        for c in range(dim):
            store_row.append(f"flex::stream_store(q_p.output_y_{rname}_ptr + (size_t)q_row * {dim} + {c}, q_tot.v[{first + c}]);")
            add_row.append(f"q_p.output_y_{rname}_ptr[(size_t)q_row * {dim} + {c}] += q_tot.v[{first + c}];")
    for (gname, first, dim) in kp.agg_slices:
        for c in range(dim):
            store_agg.append(f"q_p.output_y_{gname}_ptr[{c}] = q_total.v[{first + c}];")

    row_aligned_modules = sorted({s["selector_name"] for s in selector_register
                                  if s["selector"] == 1 and s.get("row_aligned") and has_reducer})
    read_modules = {module for module, _ in kp.fetch_indices}
    signature = generate_binding_code(None, inputs, outputs, selector_register)
    signature.update({
        "graph": ir.name,
        "hash": ir.content_hash(),
        "dtypes": list(dtypes),
        # index arrays the library never dereferences: their selector equals the reducer's row ids
        "row_aligned_index_inputs": [m + "_idx" for m in row_aligned_modules if m not in read_modules],
        # value tensors read at index `row` for every row of a tile: they must hold at least num_rows items
        "row_indexed_value_inputs": sorted({src for _, src, _, _ in kp.row_sources}),
        "policy": {"block": block, "ipt": {k: ipt[k] for k in dtypes}},
        # what makes this library a measurement variant instead of a product library (both empty: product)
        "policy_override": {k: int(v) for k, v in sorted(policy.items())},
        "tuning": defines,
        "widths": {"fetch_values": kp.fetch_value_width, "fetch_indices": kp.fetch_index_width,
                   "reduce": kp.red_width, "aggregate": kp.agg_width, "row": kp.row_width},
    })
    sig_json = json.dumps(signature, sort_keys=True)
    sig_literal = json.dumps(sig_json)  # a C string literal

    ctype = {"float32": "float", "float64": "double", "int64": "long"}
    enum = {"float32": "FLEXSPMV_F32", "float64": "FLEXSPMV_F64", "int64": "FLEXSPMV_I64"}
    cases_run, cases_ws, cases_tiling, cases_static = [], [], [], []
    for d in dtypes:
        disp = f"flex::Dispatch<Graph<{ctype[d]}>, {block}, {ipt[d]}, {'true' if has_reducer else 'false'}>"
        cases_run.append(
            f"    case {enum[d]}: {{ Graph<{ctype[d]}>::Params p; Graph<{ctype[d]}>::fill(p, a); return {disp}::run(p, a); }}\n")
        cases_static.append(
            f"    case {enum[d]}: {{ Graph<{ctype[d]}>::Params p; Graph<{ctype[d]}>::fill(p, a); return {disp}::run_static(p, a); }}\n")
        cases_ws.append(f"    case {enum[d]}: return {disp}::workspace_bytes(num_rows, ne);\n")
        cases_tiling.append(f"    case {enum[d]}: return {disp}::tiling(num_rows, ne, out);\n")

    src = f"""// Generated by flexspmv_amd.codegen.merged_gen_gpu for sub-graph "{ir.name}" ({ir.content_hash()}).
// Do not edit: regenerate from the six-list description instead.
#define FLEX_TUNING_DECLARED {1 if defines else 0}  // tuning switches given to the generator: {" ".join(defines) or "none"}
#include "flex_dispatch.hpp"

namespace {{

template <typename ValueT>
struct Graph {{
  using Value = ValueT;
  using OffsetT = int;
  static constexpr int FETCH_VALUES = {kp.fetch_value_width};   // ValueT words streamed per edge
  static constexpr int FETCH_INDICES = {kp.fetch_index_width};  // index words streamed per edge
  static constexpr int RED_WIDTH = {kp.red_width};
  static constexpr int AGG_WIDTH = {kp.agg_width};
  static constexpr int ROW_WIDTH = {kp.row_width};
  // 32-bit registers that hold one edge's fetched and gathered data
  static constexpr int EDGE_WORDS = ({kp.fetch_value_width} + {sum(d for _, _, _, d in kp.gathers)}) * (int)(sizeof(ValueT) / 4) + {kp.fetch_index_width};
  // edge() has no side effects besides its results, so a kernel may evaluate it for a lane that has no
  // edge and discard the result
  static constexpr bool EDGE_PURE = {'true' if edge_pure else 'false'};

  struct Params {{
{_indent(params)}  }};

{_indent(typedefs, 2)}
  static void fill(Params& q_p, const flexspmv_launch_args* a) {{
{_indent(fill)}  }}

  // streamed per-edge data (edge tensors and selector indices): first memory level
  struct Fetch {{
{_indent(fetch_members)}  }};
  // gathered vertex data: second memory level, addressed through Fetch
  struct Gather {{
{_indent(gather_members)}  }};
  static FLEX_DEV void fetch(const Params& q_p, const int q_e, Fetch& q_f) {{
{_indent(fetch_body)}  }}
  static FLEX_DEV void gather(const Params& q_p, const Fetch& q_f, Gather& q_g) {{
{_indent(gather_body)}  }}
  // the array behind streamed word q_w, where every streamed word is an array of its own
  static constexpr bool FETCH_CONTIGUOUS = {'true' if fetch_contiguous else 'false'};
  static FLEX_DEV const ValueT* value_stream(const Params& q_p, const int q_w) {{
{_indent(value_streams)}    return nullptr;
  }}
  static FLEX_DEV const OffsetT* index_stream(const Params& q_p, const int q_w) {{
{_indent(index_streams)}    return nullptr;
  }}
  // hand-over of a tile's fetched data through LDS: word w of tile edge j sits at [w * TILE + j]
  template <int TILE>
  static FLEX_DEV void put(const Fetch& q_f, ValueT* q_sv, OffsetT* q_si, const int q_j) {{
{_indent(put_body)}  }}
  template <int TILE>
  static FLEX_DEV void get(const ValueT* q_sv, const OffsetT* q_si, const int q_j, Fetch& q_f) {{
{_indent(get_body)}  }}

  // the map for edge q_e: what it contributes to the reducers (q_tot) and to the aggregators (q_agg);
  // both are assigned, the kernel accumulates
  template <class R, class T, class A>
  static FLEX_DEV void edge(const Params& q_p, const int q_e, const Fetch& q_f, const Gather& q_g, const R& q_rv, T& q_tot, A& q_agg) {{
{_indent(body)}  }}

  template <class R>
  static FLEX_DEV void load_row(const Params& q_p, const int q_row, R& q_rv) {{
{_indent(load_row)}  }}
  template <class T>
  static FLEX_DEV void store_row(const Params& q_p, const int q_row, const T& q_tot) {{
{_indent(store_row)}  }}
  template <class T>
  static FLEX_DEV void add_row(const Params& q_p, const int q_row, const T& q_tot) {{
{_indent(add_row)}  }}
  template <class A>
  static FLEX_DEV void store_agg(const Params& q_p, const A& q_total) {{
{_indent(store_agg)}  }}
}};

const char kSignature[] = {sig_literal};

}}  // namespace

extern "C" {{

int flexspmv_abi_version(void) {{ return FLEXSPMV_ABI_VERSION; }}
const char* flexspmv_signature(void) {{ return kSignature; }}
const char* flexspmv_last_error(void) {{ return flex::g_last_error; }}
int flexspmv_last_kernel_ms(float* ms) {{ return flex::last_kernel_ms(ms); }}

size_t flexspmv_workspace_bytes(int32_t dtype, int64_t num_rows, int64_t ne) {{
  switch (dtype) {{
{''.join(cases_ws)}    default: return 0;
  }}
}}

int flexspmv_tiling(int32_t dtype, int64_t num_rows, int64_t ne, int32_t out[6]) {{
  flex::g_last_error[0] = 0;
  switch (dtype) {{
{''.join(cases_tiling)}    default: return flex::fail(FLEXSPMV_ERR_BAD_DTYPE, "Unsupported dtype for ValueT: this library was not generated for it");
  }}
}}

int flexspmv_launch(const flexspmv_launch_args* a) {{
  flex::g_last_error[0] = 0;
  const int bad = flex::check_counts(a, {len(plan.value_inputs)}, {len(plan.selector_inputs)}, {len(plan.outputs)});
  if (bad != FLEXSPMV_OK) return bad;
  switch (a->dtype) {{
{''.join(cases_run)}    default: return flex::fail(FLEXSPMV_ERR_BAD_DTYPE, "Unsupported dtype for ValueT: this library was not generated for it");
  }}
}}

int flexspmv_launch_static(const flexspmv_launch_args* a) {{
  flex::g_last_error[0] = 0;
  const int bad = flex::check_counts(a, {len(plan.value_inputs)}, {len(plan.selector_inputs)}, {len(plan.outputs)});
  if (bad != FLEXSPMV_OK) return bad;
  switch (a->dtype) {{
{''.join(cases_static)}    default: return flex::fail(FLEXSPMV_ERR_BAD_DTYPE, "Unsupported dtype for ValueT: this library was not generated for it");
  }}
}}

}}  // extern "C"
"""
    if os.getenv(VERBOSE_ENV) in ("1", "", "true", "True"):
        for line in body:
            print("Edge code: ", line)
    return src, signature


def generate_cuda_code_from_graph(submodule, traced_model, out_dir: Optional[str] = None):
    """Reference entry-point name kept for drivers: trace a fused fx sub-module and emit its HIP
    source (codegen/merged_gen_gpu.py:17).  Returns (path of the .hip file, signature)."""
    from ..trace.graph_trace import trace_graph
    from ..build import write_generated_source
    six = trace_graph(submodule, traced_model)
    name = getattr(submodule, "_flexspmv_name", None) or type(submodule).__name__
    ir = FusedGraphIR(str(name), *six)
    return write_generated_source(ir, out_dir=out_dir)
