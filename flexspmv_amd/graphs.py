"""Six-list descriptions of the fused sub-graphs this package ships prebuilt.

Each function returns what ``trace_graph`` (trace/graph_trace.py:32-328) would produce for the
corresponding EASIER module, written node by node with :class:`GraphBuilder`.  They cover the five
benchmark workloads and the generated instances the reference keeps in its tree, so the kernels do
not depend on a tracer being installed.
"""
from __future__ import annotations

from typing import Callable, Dict, List

from .ir import FusedGraphIR, GraphBuilder

SLICE_ALL = slice(None, None, None)
GRAVITY = 9.81


def csr_spmv(dtype="float32") -> FusedGraphIR:
    """y = A @ x for CSR A: ``y = reducer(vals * selector(x))`` (the reference's plain-SpMV slot
    set: one edge tensor, one selector, ``mul``, one reducer)."""
    b = GraphBuilder("csr_spmv", dtype, doc=csr_spmv.__doc__)
    b.placeholder("vals", (1,))
    b.placeholder("x", (1,))
    b.select("selector", "x")
    b.map("mul", "mul", ["vals", "selector"])
    b.reduce("reducer", "mul")
    b.output("reducer")
    return b.build()


def spmv_dot(dtype="float64") -> FusedGraphIR:
    """One CG-style iteration: ``y = A @ x`` and ``dot = x . y`` in a single pass.  The dot is the
    edge-level aggregator ``sum(x[row(e)] * a_e * x[col(e)])``; the row selector's index array equals
    the reducer's row ids, so the kernel takes the row from the merge path."""
    b = GraphBuilder("spmv_dot", dtype, doc=spmv_dot.__doc__)
    b.placeholder("vals", (1,))
    b.placeholder("x", (1,))
    b.select("selector_col", "x")
    b.select("selector_row", "x", row_aligned=True)
    b.map("mul", "mul", ["vals", "selector_col"])
    b.reduce("reducer", "mul")
    b.map("mul", "mul_1", ["selector_row", "mul"])
    b.aggregate("sum_1", "mul_1")
    b.output("reducer", "sum_1")
    return b.build()


def spring_mass(dtype="float32") -> FusedGraphIR:
    """Spring forces on a half-edge list sorted by destination vertex:
    ``d = x_dst - x_src; r = |d|; f = k (r - L) d / r`` reduced per destination vertex, plus the
    potential energy ``sum(0.25 k (r - L)^2)`` (each spring appears as two half-edges)."""
    b = GraphBuilder("spring_mass", dtype, doc=spring_mass.__doc__)
    b.placeholder("pos", (3,))
    b.placeholder("k", (1,))
    b.placeholder("rest", (1,))
    b.select("gather_src", "pos")
    b.select("gather_dst", "pos", row_aligned=True)
    b.map("sub", "sub", ["gather_dst", "gather_src"])          # d (3)
    b.map("norm", "norm", ["sub"])                             # r (scalar)
    b.map("sub", "sub_1", ["norm", "rest"], shape=(1,))        # r - L
    b.map("mul", "mul", ["k", "sub_1"])                         # k (r - L)
    b.map("mul", "mul_1", ["mul", "sub"], shape=(3,))           # k (r - L) d
    b.map("truediv", "truediv", ["mul_1", "norm"], shape=(3,))  # / r
    b.reduce("scatter", "truediv")
    b.map("pow", "pow_1", ["sub_1", 2])
    b.map("mul", "mul_2", ["k", "pow_1"])
    b.map("mul", "mul_3", ["mul_2", 0.25])
    b.aggregate("sum_1", "mul_3")
    b.output("scatter", "sum_1")
    return b.build()


def swe_rusanov(dtype="float64") -> FusedGraphIR:
    """Rusanov flux of the shallow-water equations over half-edges sorted by destination cell.
    State ``U = (h, uh, vh)`` per cell, unit normal and length per half-edge; three reducers (mass and
    the two momentum fluxes) share the row structure.  ``max(a, b)`` is ``where(a > b, a, b)`` and
    ``sqrt`` is ``pow(., 0.5)``."""
    g = GRAVITY
    b = GraphBuilder("swe_rusanov", dtype, doc=swe_rusanov.__doc__)
    b.placeholder("U", (3,))
    b.placeholder("nrm", (2,))
    b.placeholder("length", (1,))
    b.select("gather_src", "U")
    b.select("gather_dst", "U", row_aligned=True)
    b.map("getitem", "nx", ["nrm", (SLICE_ALL, 0)])
    b.map("getitem", "ny", ["nrm", (SLICE_ALL, 1)])
    for side, src in (("l", "gather_dst"), ("r", "gather_src")):
        b.map("getitem", f"h_{side}", [src, (SLICE_ALL, 0)])
        b.map("getitem", f"uh_{side}", [src, (SLICE_ALL, 1)])
        b.map("getitem", f"vh_{side}", [src, (SLICE_ALL, 2)])
        b.map("truediv", f"u_{side}", [f"uh_{side}", f"h_{side}"])
        b.map("truediv", f"v_{side}", [f"vh_{side}", f"h_{side}"])
        b.map("mul", f"unx_{side}", [f"u_{side}", "nx"])
        b.map("mul", f"vny_{side}", [f"v_{side}", "ny"])
        b.map("add", f"un_{side}", [f"unx_{side}", f"vny_{side}"])       # normal velocity
        b.map("mul", f"hh_{side}", [f"h_{side}", f"h_{side}"])
        b.map("mul", f"pr_{side}", [f"hh_{side}", 0.5 * g])               # 0.5 g h^2
        b.map("mul", f"gh_{side}", [f"h_{side}", g])
        b.map("pow", f"c_{side}", [f"gh_{side}", 0.5])                    # sqrt(g h)
        b.map("abs", f"aun_{side}", [f"un_{side}"])
        b.map("add", f"lam_{side}", [f"aun_{side}", f"c_{side}"])
        b.map("mul", f"fh_{side}", [f"h_{side}", f"un_{side}"])           # mass flux
        b.map("mul", f"fu0_{side}", [f"uh_{side}", f"un_{side}"])
        b.map("mul", f"prx_{side}", [f"pr_{side}", "nx"])
        b.map("add", f"fu_{side}", [f"fu0_{side}", f"prx_{side}"])        # x-momentum flux
        b.map("mul", f"fv0_{side}", [f"vh_{side}", f"un_{side}"])
        b.map("mul", f"pry_{side}", [f"pr_{side}", "ny"])
        b.map("add", f"fv_{side}", [f"fv0_{side}", f"pry_{side}"])        # y-momentum flux
    b.map("gt", "gt", ["lam_l", "lam_r"])
    b.map("where", "lam", ["gt", "lam_l", "lam_r"])
    for comp, q in (("h", "h"), ("u", "uh"), ("v", "vh")):
        b.map("add", f"fs_{comp}", [f"f{comp}_l", f"f{comp}_r"])
        b.map("sub", f"jump_{comp}", [f"{q}_r", f"{q}_l"])
        b.map("mul", f"diss_{comp}", ["lam", f"jump_{comp}"])
        b.map("sub", f"num_{comp}", [f"fs_{comp}", f"diss_{comp}"])
        b.map("mul", f"half_{comp}", [f"num_{comp}", 0.5])
        b.map("mul", f"flux_{comp}", [f"half_{comp}", "length"])
    b.reduce("scatter_h", "flux_h")
    b.reduce("scatter_uh", "flux_u")
    b.reduce("scatter_vh", "flux_v")
    b.output("scatter_h", "scatter_uh", "scatter_vh")
    return b.build()


def mass_sum(dtype="float64") -> FusedGraphIR:
    """Total mass ``sum(h * area)`` over cells: an aggregator-only sub-graph (``ne`` = cells)."""
    b = GraphBuilder("mass_sum", dtype, doc=mass_sum.__doc__)
    b.placeholder("h", (1,))
    b.placeholder("area", (1,))
    b.map("mul", "mul", ["h", "area"])
    b.aggregate("sum_1", "mul")
    b.output("sum_1")
    return b.build()


def system_two_selectors(dtype="float64") -> FusedGraphIR:
    """The toy ``System`` module of the reference (easier_spmv.py:17-69): two selectors on one
    ``vector_x``, edge tensors of width 2 and 6, two in-place stores and one reducer.  Node order as
    in the generated instance the reference keeps (include/merged_agent_spmv.cuh:124-137,407-446,
    include/merged_utils.cuh:249-256)."""
    b = GraphBuilder("system_two_selectors", dtype, doc=system_two_selectors.__doc__)
    b.placeholder("vector_x", (2, 1))
    b.placeholder("spm_1", (2, 1))
    b.placeholder("y_add_1", (2, 1))
    b.placeholder("spm_2", (2, 3))
    b.placeholder("y_add_2", (2, 3))
    b.select("selector_1", "vector_x")
    b.select("selector_2", "vector_x")
    b.map("add", "add", ["selector_1", "selector_2"], shape=(2, 1))
    b.map("add", "add_1", ["add", "spm_1"], shape=(2, 1))
    b.map("add", "add_2", ["selector_1", "selector_2"], shape=(2, 1))
    b.map("add", "add_3", ["add_2", "spm_2"], shape=(2, 3))
    b.map("setitem", "setitem", ["y_add_1", (SLICE_ALL,), "add_1"], shape=(2, 1))
    b.map("setitem", "setitem_1", ["y_add_2", (SLICE_ALL,), "add_3"], shape=(2, 3))
    b.reduce("reducer_1", "add_1")
    b.output("reducer_1")
    return b.build()


def bpoints_copy(dtype="int64") -> FusedGraphIR:
    """The map-only instance the reference keeps generated for its CPU path (merged_spmv.h:92-151):
    ``bp_1[:] = bpoints[:, 1].clone()`` on int64 index data."""
    b = GraphBuilder("bpoints_copy", dtype, doc=bpoints_copy.__doc__)
    b.placeholder("bpoints", (2,))
    b.placeholder("bp_1", (1,))
    b.map("getitem", "getitem_10", ["bpoints", (SLICE_ALL, 1)])
    b.map("clone", "clone_10", ["getitem_10"])
    b.map("copy_", "copy__10", ["bp_1", "clone_10"], shape=(1,))
    return b.build()


def index_spmv(dtype="int64") -> FusedGraphIR:
    """Integer SpMV with a total: ``y = reducer(w * selector(ids))`` and ``sum(w * selector(ids))`` on int64
    data, the value type the reference dispatches for sub-graphs traced on int64 tensors
    (codegen/merged_gen_binding.py:143-157).  Integer sums have one right answer whatever the order, so
    this sub-graph holds the reducer, the carry fix-up and the aggregator to bit-exactness."""
    b = GraphBuilder("index_spmv", dtype, doc=index_spmv.__doc__)
    b.placeholder("w", (1,))
    b.placeholder("ids", (1,))
    b.select("selector", "ids")
    b.map("mul", "mul", ["w", "selector"])
    b.reduce("reducer", "mul")
    b.aggregate("sum_1", "mul")
    b.output("reducer", "sum_1")
    return b.build()


def index_sums(dtype="int64") -> FusedGraphIR:
    """Integer sub-graph with a row-aligned source, two reducers of widths 2 and 1 on one row structure
    and an aggregator of width 2, on int64 data (mesh bookkeeping such as per-cell sums of neighbour ids
    and weighted degrees; assemble_shallow_water.py:62-77 shuffles indices the same way)."""
    b = GraphBuilder("index_sums", dtype, doc=index_sums.__doc__)
    b.placeholder("w", (1,))
    b.placeholder("ids", (2,))
    b.select("sel", "ids")
    b.select("sel_row", "ids", row_aligned=True)
    b.map("mul", "mul", ["sel", "w"], shape=(2,))
    b.map("sub", "sub", ["mul", "sel_row"])
    b.reduce("red", "sub")
    b.reduce("weight", "w", module="red")
    b.aggregate("sum_1", "mul")
    b.output("red", "weight", "sum_1")
    return b.build()


def op_zoo(dtype="float32") -> FusedGraphIR:
    """Every element-wise op of the reference's emitters in one reducer sub-graph, including the
    corner cases of the value type: guarded and unguarded division, modulo broadcast between widths
    6 / 3 / 2, pow with tensor and literal exponents, comparisons, ``where`` with tensor and literal
    branches, in-place ``add_`` / ``setitem`` / ``copy_``, a map output, a scalar (``norm``) mixed with
    tensors."""
    b = GraphBuilder("op_zoo", dtype, doc=op_zoo.__doc__)
    b.placeholder("a6", (6,))
    b.placeholder("b3", (3,))
    b.placeholder("c2", (2,))
    b.placeholder("acc", (3,))
    b.placeholder("dst6", (6,))
    b.placeholder("vx", (3,))
    b.select("sel_p", "vx")
    b.select("sel_q", "vx", module="sel_q")
    b.map("add", "add", ["a6", "b3"])                        # 6 + 3 -> modulo broadcast
    b.map("sub", "sub", ["sel_p", "sel_q"])                  # 3
    b.map("mul", "mul", ["a6", "c2"])                        # 6 * 2
    b.map("truediv", "truediv", ["b3", "sub"])               # same width: guarded
    b.map("truediv", "truediv_1", ["a6", "b3"])              # 6 / 3: unguarded
    b.map("neg", "neg", ["truediv"])
    b.map("abs", "abs_1", ["sub"])
    b.map("pow", "pow_1", ["abs_1", 0.5])
    b.map("pow", "pow_2", ["abs_1", "c2"], shape=(3,))       # tensor exponent, widths 3 ^ 2
    b.map("exp", "exp", ["sub"])
    b.map("sign", "sign", ["sub"])
    b.map("norm", "norm", ["b3"])
    b.map("truediv", "truediv_2", ["sub", "norm"], shape=(3,))   # tensor / scalar: unguarded
    b.map("truediv", "truediv_3", [1, "b3"])                 # literal / tensor: guarded
    b.map("lt", "lt", ["sub", 0])
    b.map("gt", "gt", ["a6", "b3"])
    b.map("where", "where", ["lt", "pow_1", "exp"])
    b.map("where", "where_1", ["gt", "add", 0.0])
    b.map("where", "where_2", ["lt", 1.5, "truediv_3"])
    b.map("getitem", "getitem", ["a6", (SLICE_ALL, 4)])
    b.map("clone", "clone", ["getitem"])
    b.map("mul", "mul_1", ["clone", "sign"], shape=(3,))
    b.map("add_", "add_", ["acc", "mul_1"], shape=(3,))
    b.map("mul", "mul_2", ["where_1", "mul"])
    b.map("add", "add_1", ["mul_2", "truediv_1"])
    b.map("setitem", "setitem", ["dst6", (SLICE_ALL,), "add_1"], shape=(6,))
    b.map("add", "add_2", ["where", "where_2"])
    b.map("add", "add_3", ["add_2", "pow_2"])
    b.map("mul", "mul_3", ["neg", 0.001])
    b.map("add", "add_6", ["add_3", "mul_3"])
    b.map("add", "add_4", ["add_6", "truediv_2"])
    b.map("add", "add_5", ["add_4", "acc"])
    b.reduce("reducer", "add_5")
    b.reduce("reducer_6", "dst6", module="reducer")
    b.aggregate("sum_1", "mul_1")
    b.output("reducer", "reducer_6", "sum_1", "add_4")
    return b.build()


def map_store(dtype="float32") -> FusedGraphIR:
    """Map-only sub-graph with a fresh per-edge output and an aggregator over a width-3 value."""
    b = GraphBuilder("map_store", dtype, doc=map_store.__doc__)
    b.placeholder("w", (3,))
    b.placeholder("vx", (3,))
    b.select("sel", "vx")
    b.map("mul", "mul", ["w", "sel"])
    b.map("add", "add", ["mul", 1.0])
    b.aggregate("sum_1", "mul")
    b.output("add", "sum_1")
    return b.build()


REGISTRY: Dict[str, Callable[..., FusedGraphIR]] = {
    "csr_spmv": csr_spmv,
    "spmv_dot": spmv_dot,
    "spring_mass": spring_mass,
    "swe_rusanov": swe_rusanov,
    "mass_sum": mass_sum,
    "system_two_selectors": system_two_selectors,
    "bpoints_copy": bpoints_copy,
    "index_spmv": index_spmv,
    "index_sums": index_sums,
    "op_zoo": op_zoo,
    "map_store": map_store,
}


def get(name: str) -> FusedGraphIR:
    """The description of a prebuilt sub-graph (dtype dispatch happens at launch, so one description
    serves float32 and float64)."""
    return REGISTRY[name]()


def all_graphs() -> List[FusedGraphIR]:
    return [f() for f in REGISTRY.values()]
