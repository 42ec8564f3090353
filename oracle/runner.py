"""TEST INFRASTRUCTURE ONLY -- run the CPU oracle of a sub-graph on numpy arrays.

Mirrors what the reference's CPU binding does around its kernel
(cpu_template/merged_binding_template_cpu.cpp:8-33): outputs are zero-initialised, ``ne`` is the
element count of the first index array (else ``num_cols``), the thread count is explicit here
(the reference takes ``at::get_num_threads()``, :27).
"""
from __future__ import annotations

import ctypes
import os
import sys
from typing import Any, Dict, List, Optional, Sequence, Tuple

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from flexspmv_amd.codegen.merged_gen_binding import binding_plan  # noqa: E402
from flexspmv_amd.ir import FusedGraphIR  # noqa: E402
from oracle.build_oracle import build_graph_oracle, oracle_library_path  # noqa: E402

_DTYPE_CODE = {np.dtype("float32"): 0, np.dtype("float64"): 1, np.dtype("int64"): 2}
_LIBS: Dict[str, ctypes.CDLL] = {}


def _library(ir: FusedGraphIR) -> ctypes.CDLL:
    path = oracle_library_path(ir)
    if path not in _LIBS:
        if not os.path.exists(path):
            build_graph_oracle(ir)
        lib = ctypes.CDLL(path)
        lib.oracle_run.restype = ctypes.c_int
        lib.oracle_run.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                   ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p),
                                   ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        _LIBS[path] = lib
    return _LIBS[path]


def run_oracle(ir: FusedGraphIR, tensors: Dict[str, np.ndarray], row_end_offsets: Optional[np.ndarray],
               num_rows: int, num_cols: int, num_threads: int = 8,
               copy_inputs: bool = True) -> Tuple[List[np.ndarray], Dict[str, np.ndarray]]:
    """Run the oracle.  ``tensors`` maps binding names (value inputs by name, index inputs as
    ``<module>_idx``) to arrays.  Returns (outputs in binding order, the value inputs after the run -
    in-place map ops write through them)."""
    plan = binding_plan(ir.inputs, ir.outputs, ir.selector_register)
    lib = _library(ir)
    values = []
    for n in plan.value_inputs:
        a = np.ascontiguousarray(tensors[n])
        values.append(a.copy() if copy_inputs else a)
    dtype = values[0].dtype if values else np.dtype("float32")
    dispatch = tensors[plan.dispatch_tensor].dtype
    if any(v.dtype != dispatch for v in values):
        raise RuntimeError("value dtype mismatch")
    indices = [np.ascontiguousarray(tensors[s + "_idx"], dtype=np.int32) for s in plan.selector_inputs]
    ne = int(indices[0].size) if indices else int(num_cols)
    if ne <= 0:
        raise RuntimeError("selector index must be non-empty (ne > 0)")
    outs = []
    for o in plan.outputs:
        lead = {"reducer": num_rows, "sum": None, "map": ne}[o.kind]
        shape = (o.dim,) if lead is None else ((lead,) if o.dim == 1 else (lead, o.dim))
        outs.append(np.zeros(shape, dtype=dispatch))

    def parr(arrs):
        p = (ctypes.c_void_p * max(1, len(arrs)))()
        for i, a in enumerate(arrs):
            p[i] = a.ctypes.data
        return p

    ro = None
    if row_end_offsets is not None:
        ro = np.ascontiguousarray(row_end_offsets, dtype=np.int32)
    rc = lib.oracle_run(_DTYPE_CODE[np.dtype(dispatch)], int(num_threads), parr(values), parr(indices),
                        parr(outs), ro.ctypes.data if ro is not None else None, int(num_rows), ne)
    if rc != 0:
        raise RuntimeError(f"oracle_run failed ({rc})")
    return outs, dict(zip(plan.value_inputs, values))
