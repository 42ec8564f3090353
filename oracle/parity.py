"""TEST INFRASTRUCTURE ONLY -- the parity criterion between a device result and the CPU oracle.

Used by ``tests/``, by ``bench.py``'s CPU leg and by ``__graft_entry__.smoke()``; the product never imports it.

Tolerances: float32 1e-5, float64 1e-12, integers and structure exact.  A reducer output is held to the
tolerance **row by row**::

    |device - oracle| <= tol * max(|oracle|, sum over the row of |contribution of an edge|) + floor(row)

    floor(row) = FLOOR_ULPS * eps * largest |contribution| of the row
                 + MOVE_FACTOR * sum over the row of |change of an edge's contribution when the
                                 floating-point inputs move by a unit or two in the last place|

Every term is the row's own: a row of small terms gets no slack from a large edge elsewhere in the launch.
The contributions come from the oracle itself, run on the same edges with every edge as a row of its own
(single-term sums: no rounding of a sum is involved).  The second term of the floor is the row's
conditioning: a map with a cancellation inside (the spring's ``r - L``, the flux differences of the
shallow-water map) cannot be evaluated more precisely than its intermediate values allow, and two
floating-point evaluations of it (fused multiply-adds, another sqrt or division sequence) differ by a few
ulps of those intermediates however small the contribution comes out - which is what moving the inputs by
an ulp shows.  The inputs are moved several times and the changes added: every value tensor on its own,
all its values scaled by (1 + 2 eps) (deterministic; intermediates are homogeneous in the inputs, so this
shows their size even where random moves of two operands happen to cancel), and once all of them by one
ulp up or down at random.  For products (SpMV) the sum is a few ulps of the contribution itself and changes
nothing.  A wrong kernel - a dropped or doubled edge, a wrong index, a wrong operand - moves a row by whole
contributions, not by ulps of them, and fails.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import numpy as np

from oracle.runner import run_oracle

TOL = {np.dtype("float32"): 1e-5, np.dtype("float64"): 1e-12}
FLOOR_ULPS = 8
MOVE_FACTOR = 2


def nudge(a: np.ndarray, rng: np.random.Generator) -> np.ndarray:
    """Every element of a floating-point array moved by one unit in the last place, up or down at random."""
    if a.dtype.kind != "f":
        return a
    up = rng.integers(0, 2, a.shape).astype(bool)
    inf = np.array(np.inf, dtype=a.dtype)
    return np.where(up, np.nextafter(a, inf), np.nextafter(a, -inf)).astype(a.dtype)


def reducer_row_scales(ir, tensors: Dict[str, np.ndarray], row_ptr: np.ndarray, num_cols: int,
                       threads: int = 8) -> Dict[int, Tuple[np.ndarray, np.ndarray]]:
    """Per reducer output (keyed by its position among the outputs): ``(scale, floor)`` as float64 arrays of
    shape [num_rows][Dim] - the sum over each row of |contribution| and the row's floor (module docstring)."""
    ne = int(row_ptr[-1])
    one_per_row = np.arange(ne + 1, dtype=np.int32)
    per_edge, _ = run_oracle(ir, tensors, one_per_row, ne, num_cols, threads)
    moves = [{k: nudge(np.asarray(v), np.random.default_rng(ne)) for k, v in tensors.items()}]
    for name, v in tensors.items():
        v = np.asarray(v)
        if v.dtype.kind == "f" and not name.endswith("_idx"):
            scaled = (v * v.dtype.type(1.0 + 2.0 * float(np.finfo(v.dtype).eps))).astype(v.dtype)
            moves.append({**tensors, name: scaled})
    change = [None] * len(per_edge)
    for moved in moves:
        per_edge_moved, _ = run_oracle(ir, moved, one_per_row, ne, num_cols, threads)
        for i, (a, b) in enumerate(zip(per_edge, per_edge_moved)):
            if a.dtype.kind == "f" and ir.outputs[i]["target"] == "reducer":
                d = np.abs(b.astype(np.float64).reshape(ne, -1) - a.astype(np.float64).reshape(ne, -1))
                change[i] = d if change[i] is None else change[i] + d
    starts = np.minimum(np.asarray(row_ptr[:-1], dtype=np.int64), ne)   # reduceat needs valid start indices
    empty = np.diff(row_ptr) == 0
    pad = lambda a: np.vstack([a, np.zeros((1, a.shape[1]))])
    out = {}
    for i, spec in enumerate(ir.outputs):
        if spec["target"] != "reducer" or per_edge[i].dtype.kind != "f":
            continue
        eps = float(np.finfo(per_edge[i].dtype).eps)
        c = np.abs(per_edge[i].astype(np.float64)).reshape(ne, -1)
        d = change[i]
        scale = np.add.reduceat(pad(c), starts, axis=0)
        largest = np.maximum.reduceat(pad(c), starts, axis=0)
        moved_sum = np.add.reduceat(pad(d), starts, axis=0)
        floor = FLOOR_ULPS * eps * largest + MOVE_FACTOR * moved_sum
        scale[empty] = 0.0
        floor[empty] = 0.0
        out[i] = (scale, floor)
    return out


def row_excess(got: np.ndarray, ref: np.ndarray, tol: float, scale: np.ndarray, floor: np.ndarray) -> np.ndarray:
    """|got - ref| divided by what the row criterion allows (<= 1 everywhere: within the criterion)."""
    ref64 = ref.astype(np.float64)
    allowed = tol * np.maximum(np.abs(ref64), scale.reshape(ref.shape)) + floor.reshape(ref.shape)
    diff = np.abs(got.astype(np.float64) - ref64)
    return np.where(diff == 0.0, 0.0, diff / np.maximum(allowed, 1e-300))


def aggregator_bounds(ir, tensors, row_ptr, num_rows: int, num_cols: int, index: int, tol: float,
                      threads_fine: int = 256) -> Optional[dict]:
    """What a float32 aggregator output is compared with.

    The reference adds every edge of a thread's share sequentially, so its own float32 result drifts from the
    exact sum by up to (edges per thread) * eps * sum|terms| and depends on the thread count (spring-mass
    100^3: 0.7 % at one thread).  The centre of the comparison is therefore the same oracle evaluated in
    float64 on the same float32 inputs (``centre``, tolerance ``tol``).  Beside it the float32 oracle itself is
    run at ``threads_fine`` threads - the most the reference's carry arrays allow, so the shortest chains it
    can have - and the device result has to be within ``bound_fine`` = (chain * eps + tol) * sum|terms| of it,
    chain = ceil(items / threads_fine): a bound a wrong kernel fails at test sizes (a few hundred terms per
    chain).  Returns None for outputs that are not float32 aggregators."""
    spec = ir.outputs[index]
    dispatch = next(v for k, v in tensors.items() if not k.endswith("_idx"))
    if spec["target"] != "sum" or dispatch.dtype != np.float32:
        return None
    hi = {k: (v.astype(np.float64) if v.dtype == np.float32 else v) for k, v in tensors.items()}
    centre, _ = run_oracle(ir, hi, row_ptr, num_rows, num_cols, 8)
    fine, _ = run_oracle(ir, tensors, row_ptr, num_rows, num_cols, threads_fine)
    ne = int(row_ptr[-1]) if row_ptr is not None else int(num_cols)
    # sum of |terms|: the aggregator of the absolute per-edge values, from the per-edge oracle run in float64
    items = ne + (int(num_rows) if row_ptr is not None else ne)   # the reference splits rows + edges over its threads
    chain = -(-items // threads_fine)
    magnitude = float(np.abs(centre[index]).max())
    return {"centre": centre[index], "fine": fine[index], "chain": chain,
            "bound_fine": (chain * float(np.finfo(np.float32).eps) + tol) * magnitude}
