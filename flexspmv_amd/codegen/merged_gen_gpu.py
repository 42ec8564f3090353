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
  codegen/merged_gen_gpu.py:394);
* ops that depend on a ``row_aligned`` selector run in the merge walk, where the row is known; the
  values they need from the coalesced stage travel through LDS next to the reducer arguments.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

from ..ir import FusedGraphIR, arg_name, dtype_name, get_dim_length
from .merged_gen_binding import BindingPlan, binding_plan, generate_binding_code

VERBOSE_ENV = "EASIER_VERBOSE_CODEGEN"  # same switch as the reference (codegen/merged_gen_gpu.py:140)

# LDS a reducer block may use for the per-edge exchange + row offsets; keeps >= 4 blocks per CU
# (160 KiB LDS per CU on gfx950).
LDS_BUDGET_BYTES = 36 * 1024
BLOCK_THREADS = 256


@dataclass
class Var:
    name: str
    kind: str          # 'tensor' | 'scalar'
    dim: int
    ctype: str         # C++ type name inside Graph<ValueT>
    stage: int         # stage that defines it: 1 = coalesced edge stage, 2 = merge-walk stage
    final_stage: int = 1   # stage holding its last value (an in-place op in the walk raises it)


@dataclass
class KernelPlan:
    plan: BindingPlan
    vars: Dict[str, Var]
    exchange: List[Tuple[str, int, int]]      # (variable, component, slot)
    row_sources: List[Tuple[str, str, int, int]]  # (selector var, source tensor, dim, first slot)
    red_slices: List[Tuple[str, int, int]]    # (reducer name, first slot, dim)
    agg_slices: List[Tuple[str, int, int]]
    op_stage: Dict[int, int] = field(default_factory=dict)   # index into map_operations -> stage
    xch_width: int = 0
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
    """Variable table, stage split and LDS slot assignment for a sub-graph.

    A ``row_aligned`` selector may be served from the merge path (no index array read, its dependants
    run in the walk) or like any other selector (index array read, everything runs in the coalesced
    stage).  The first is taken only when it does not widen the per-edge LDS exchange: for ``y = A x``
    with ``x . y`` it saves the 4-byte index per edge for free, for the mesh maps it would push every
    input through LDS and shrink the tile.
    """
    with_rows = _analyse(ir, use_row_aligned=True)
    if with_rows.row_width == 0:
        return with_rows
    plain = _analyse(ir, use_row_aligned=False)
    return with_rows if with_rows.xch_width <= plain.xch_width else plain


def _analyse(ir: FusedGraphIR, use_row_aligned: bool) -> KernelPlan:
    inputs, outputs, selector_register, map_ops, red_ops, agg_ops = ir.six()
    plan = binding_plan(inputs, outputs, selector_register)
    has_reducer = bool(red_ops)
    vars: Dict[str, Var] = {}

    cur_stage: Dict[str, int] = {}   # stage a variable's current value lives in (in-place ops may raise it)
    for s in selector_register:
        dim = get_dim_length(s["shape"])
        stage = 2 if (use_row_aligned and s.get("row_aligned") and has_reducer and s["selector"] == 1) else 1
        var = s["name"] if s["selector"] == 1 else s["selector_name"]
        vars[var] = Var(var, "tensor", dim, f"TensorInput_{s['target']}_T", stage)
        cur_stage[var] = stage

    # values crossing from stage 1 into stage 2 travel through LDS slots
    exchange: List[Tuple[str, int, int]] = []
    slot_of: Dict[Tuple[str, int], int] = {}

    def need(var: str) -> None:
        v = vars[var]
        for c in range(v.dim):
            if (var, c) not in slot_of:
                slot_of[(var, c)] = len(exchange)
                exchange.append((var, c, len(exchange)))

    # reducer arguments take the first slots so that a plain SpMV exchanges exactly its products
    red_arg_names = [arg_name(r["args"][0]) for r in red_ops]

    op_stage: Dict[int, int] = {}
    for op_index, op in enumerate(map_ops):
        o = op["op"]
        if o in ("reducer", "sum"):
            continue
        args = [arg_name(a) for a in (op["args"] if o not in ("getitem", "setitem") else
                                      [op["args"][0]] + ([op["args"][2]] if o == "setitem" else []))]
        used = [a for a in args if isinstance(a, str) and a in vars]
        stage = max([1] + [cur_stage[a] for a in used]) if has_reducer else 1
        op_stage[op_index] = stage
        if stage == 2:
            for a in used:
                if vars[a].stage == 1:
                    need(a)
        if o in ("setitem", "copy_", "add_"):
            if o in ("setitem", "add_"):
                cur_stage[args[0]] = max(cur_stage[args[0]], stage)
            continue
        dim = get_dim_length(op["shape"])
        if o == "norm":
            vars[op["name"]] = Var(op["name"], "scalar", 1, "ValueT", stage)
        else:
            vars[op["name"]] = Var(op["name"], "tensor", dim, f"TensorOutput_{op['name']}_T", stage)
        cur_stage[op["name"]] = stage

    red_slices, agg_slices = [], []
    off = 0
    for r in red_ops:
        a = arg_name(r["args"][0])
        dim = get_dim_length(r["shape"])
        red_slices.append((r["name"], off, dim))
        off += dim
        if vars[a].stage == 1:
            need(a)
    red_width = off
    off = 0
    for g in agg_ops:
        dim = get_dim_length(g["shape"])
        agg_slices.append((g["name"], off, dim))
        off += dim
    agg_width = off
    for g in agg_ops:
        a = arg_name(g["args"][0])
        if has_reducer and cur_stage[a] == 2 and vars[a].stage == 1:
            need(a)
    # put reducer-argument slots first (stable order otherwise)
    order = sorted(range(len(exchange)), key=lambda i: (exchange[i][0] not in red_arg_names, i))
    exchange = [(exchange[i][0], exchange[i][1], n) for n, i in enumerate(order)]
    for var in vars:
        vars[var].final_stage = cur_stage[var]

    row_sources: List[Tuple[str, str, int, int]] = []
    row_width = 0
    for s in selector_register:
        if s["selector"] == 1 and vars[s["name"]].stage == 2 and s.get("row_aligned") and use_row_aligned:
            dim = get_dim_length(s["shape"])
            row_sources.append((s["name"], s["target"], dim, row_width))
            row_width += dim

    return KernelPlan(plan, vars, exchange, row_sources, red_slices, agg_slices, op_stage=op_stage,
                      xch_width=len(exchange), red_width=red_width, agg_width=agg_width,
                      row_width=row_width)


# ------------------------------------------------------------------------------------------
# statement emitters
# ------------------------------------------------------------------------------------------
def _arg(a: Any) -> str:
    a = arg_name(a)
    return a if isinstance(a, str) else _literal(a)


def _emit_selector(s: Dict[str, Any]) -> Tuple[List[str], List[str], List[str], List[str], List[str]]:
    """Statements of one stage-1 selector entry, split by memory level:
    (Fetch members, fetch statements, Gather members, gather statements, stage-1 prologue)."""
    dim = get_dim_length(s["shape"])
    T = f"TensorInput_{s['target']}_T"
    if s["selector"] == 1:
        name, idx = s["name"], f"column_indices_{s['name']}"
        return ([f"OffsetT {idx};"],
                [f"q_f.{idx} = flex::stream_load(q_p.{s['selector_name']}_idx_ptr + q_e);"],
                [f"{T} {name};"],
                [f"q_g.{name} = {T}(q_p.{s['target']}_ptr + (size_t)q_f.{idx} * {dim});"],
                [f"{T} {name} = q_g.{name};"])
    name = s["selector_name"]
    return ([f"{T} {name};"],
            [f"q_f.{name}.values[{i}] = flex::stream_load(q_p.{s['target']}_ptr + (size_t)q_e * {dim} + {i});"
             for i in range(dim)],
            [], [],
            [f"{T} {name} = q_f.{name};"])


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
    # LDS holds the per-edge exchange of a tile and, in the merge path, one finished total per row
    per_item = value_bytes * max(kp.xch_width, kp.red_width, 1)
    for ipt in (8, 4, 2, 1):
        if BLOCK_THREADS * ipt * per_item <= LDS_BUDGET_BYTES:
            return ipt
    return 1


def generate_hip_source(ir: FusedGraphIR, dtypes: Optional[Sequence[str]] = None,
                        policy: Optional[Dict[str, int]] = None) -> Tuple[str, Dict[str, Any]]:
    """Return (translation unit text, signature dict) for a sub-graph.

    ``dtypes`` lists the value types to instantiate (default float32 + float64, plus int64 when the
    dispatch input was traced as int64 - the reference's rule, codegen/merged_gen_binding.py:143-157).
    ``policy`` may override ``block``, ``ipt_f32``, ``ipt_f64`` and ``ipt_flat``.
    """
    inputs, outputs, selector_register, map_ops, red_ops, agg_ops = ir.six()
    kp = analyse(ir)
    plan = kp.plan
    has_reducer = bool(red_ops)
    if dtypes is None:
        dtypes = ["float32", "float64"] + (["int64"] if plan.allow_int64 else [])
    dtypes = [dtype_name(d) for d in dtypes]
    policy = dict(policy or {})
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

    # ---- stage bodies ---------------------------------------------------------------------
    s1: List[str] = []
    s2: List[str] = []
    fetch_members: List[str] = []
    fetch_body: List[str] = []
    gather_members: List[str] = []
    gather_body: List[str] = []
    for s in selector_register:
        var = s["name"] if s["selector"] == 1 else s["selector_name"]
        if kp.vars[var].stage == 1:
            fm, fs, gm, gs, pro = _emit_selector(s)
            fetch_members += fm
            fetch_body += fs
            gather_members += gm
            gather_body += gs
            s1 += pro
    # rebuild crossing variables and row-aligned selector values at the top of stage 2
    rebuilt = set()
    for var, c, slot in kp.exchange:
        v = kp.vars[var]
        if var not in rebuilt:
            s2.append(f"{v.ctype} {var};" if v.kind == "tensor" else f"ValueT {var};")
            rebuilt.add(var)
        s2.append(f"{_component(v, c)} = q_xch.v[{slot}];")
    for sel, src, dim, first in kp.row_sources:
        s2.append(f"TensorInput_{src}_T {sel};")
        s2 += [f"{sel}.values[{i}] = q_rv.v[{first + i}];" for i in range(dim)]

    map_output_names = {o.name: o for o in plan.outputs if o.kind == "map"}
    for op_index, op in enumerate(map_ops):
        o = op["op"]
        if o in ("reducer", "sum"):
            continue
        stage = kp.op_stage.get(op_index, 1) if has_reducer else 1
        body = s1 if stage == 1 else s2
        body.extend(_emit_map(op, kp.vars, "q_e"))
        if op["name"] in map_output_names:
            out = map_output_names[op["name"]]
            v = kp.vars[op["name"]]
            if v.kind == "scalar":
                body.append(f"flex::stream_store(q_p.output_y_{out.name}_ptr + (size_t)q_e, {v.name});")
            else:
                body.extend(_store_loop(f"q_p.output_y_{out.name}_ptr", "q_e", out.dim, v.name, v.dim))
    # a map output may also be a (stage-1) selector / input variable
    for name, out in map_output_names.items():
        if not any(op["name"] == name for op in map_ops):
            v = kp.vars[name]
            (s1 if v.stage == 1 or not has_reducer else s2).extend(
                _store_loop(f"q_p.output_y_{out.name}_ptr", "q_e", out.dim, v.name, v.dim))

    agg2_mask = 0
    stage1_has_agg = False
    # reducer arguments
    for (rname, first, dim), r in zip(kp.red_slices, red_ops):
        v = kp.vars[arg_name(r["args"][0])]
        for c in range(dim):
            s2.append(f"q_tot.v[{first + c}] = {_component(v, c % v.dim)};")
    # aggregator arguments
    for (gname, first, dim), g in zip(kp.agg_slices, agg_ops):
        v = kp.vars[arg_name(g["args"][0])]
        in_walk = has_reducer and v.final_stage == 2
        for c in range(dim):
            if in_walk:
                s2.append(f"q_agg.v[{first + c}] = {_component(v, c % v.dim)};")
                agg2_mask |= 1 << (first + c)
            else:
                s1.append(f"q_agg.v[{first + c}] += {_component(v, c % v.dim)};")
                stage1_has_agg = True
    # exchange writes close stage 1
    if has_reducer:
        for var, c, slot in kp.exchange:
            s1.append(f"q_xch.v[{slot}] = {_component(kp.vars[var], c)};")

    stage2_pure = not any("stream_store(" in line for line in s2)
    stage1_pure = not stage1_has_agg and not any("stream_store(" in line for line in s1)
    load_row, store_row, add_row, store_agg = [], [], [], []
    for sel, src, dim, first in kp.row_sources:
        load_row += [f"q_rv.v[{first + i}] = q_p.{src}_ptr[(size_t)q_row * {dim} + {i}];" for i in range(dim)]
    for (rname, first, dim) in kp.red_slices:
        for c in range(dim):
            store_row.append(f"flex::stream_store(q_p.output_y_{rname}_ptr + (size_t)q_row * {dim} + {c}, q_tot.v[{first + c}]);")
            add_row.append(f"q_p.output_y_{rname}_ptr[(size_t)q_row * {dim} + {c}] += q_tot.v[{first + c}];")
    for (gname, first, dim) in kp.agg_slices:
        for c in range(dim):
            store_agg.append(f"q_p.output_y_{gname}_ptr[{c}] = q_total.v[{first + c}];")

    signature = generate_binding_code(None, inputs, outputs, selector_register)
    signature.update({
        "graph": ir.name,
        "hash": ir.content_hash(),
        "dtypes": list(dtypes),
        "row_aligned_index_inputs": sorted({s["selector_name"] + "_idx" for s in selector_register
                                            if s["selector"] == 1 and kp.vars[s["name"]].stage == 2}),
        # value tensors read at index `row` for every row of a tile (served from the merge path): they
        # must hold at least num_rows items
        "row_indexed_value_inputs": sorted({src for _, src, _, _ in kp.row_sources}),
        "policy": {"block": block, "ipt": {k: ipt[k] for k in dtypes}},
        "widths": {"exchange": kp.xch_width, "reduce": kp.red_width, "aggregate": kp.agg_width,
                   "row": kp.row_width},
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
#include "flex_dispatch.hpp"

namespace {{

template <typename ValueT>
struct Graph {{
  using Value = ValueT;
  using OffsetT = int;
  static constexpr int XCH_WIDTH = {kp.xch_width};
  static constexpr int RED_WIDTH = {kp.red_width};
  static constexpr int AGG_WIDTH = {kp.agg_width};
  static constexpr int ROW_WIDTH = {kp.row_width};
  // stage 2 has no side effects besides its accumulators, so the walk may run it unconditionally
  static constexpr bool STAGE2_PURE = {'true' if stage2_pure else 'false'};
  // likewise stage 1 (no stores, no aggregator fed from the coalesced stage)
  static constexpr bool STAGE1_PURE = {'true' if stage1_pure else 'false'};
  // aggregator slots fed from the merge walk (the others are summed in stage 1)
  static constexpr unsigned AGG2_MASK = {agg2_mask}u;

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

  // coalesced edge stage: the map on fetched + gathered data
  template <class X, class A>
  static FLEX_DEV void stage1(const Params& q_p, const int q_e, const Fetch& q_f, const Gather& q_g, X& q_xch, A& q_agg) {{
{_indent(s1)}  }}

  // merge-walk stage (row known): what edge e contributes to the reducers (tot) and to the
  // aggregators fed from the walk (agg); both are assigned, the kernel accumulates
  template <class X, class R, class T, class A>
  static FLEX_DEV void contrib(const Params& q_p, const int q_e, const int q_row, const X& q_xch, const R& q_rv, T& q_tot, A& q_agg) {{
{_indent(s2)}  }}

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
        for line in s1:
            print("Stage-1 code: ", line)
        for line in s2:
            print("Stage-2 code: ", line)
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
