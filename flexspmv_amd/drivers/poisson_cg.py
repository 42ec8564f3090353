"""Conjugate gradients on the 3-D Poisson operator, the solver loop the fused ``y = A p`` and ``p . y``
launch is made for (the reference drives its Poisson model through EASIER's CG solver,
test_modules/utils.py:74-85).  One iteration is one fused launch plus vector updates; the sparsity pattern
never changes, so every launch after the first reuses the tile table."""
from __future__ import annotations

from typing import Callable, Tuple

import torch

from .. import workloads as W
from ..binding import load_named


def fused_operator(n: int, device="cuda", dtype=torch.float64) -> Tuple[Callable, int]:
    """``apply(p) -> (A p, p . A p)`` for the 7-point Laplacian on an n^3 grid, and the vector length."""
    w = W.poisson_3d_spmv_dot(n, dtype=str(dtype).replace("torch.", ""))
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    args = W.launch_arguments(w, names, device)
    xi = names.index("x")

    def apply(p: torch.Tensor):
        args[xi] = p
        y, dot = ext.merged_spmv_launch(*args)
        return y, dot

    return apply, w.num_rows


def conjugate_gradients(apply: Callable, b: torch.Tensor, tol: float = 1e-10, maxiter: int = 1000):
    """Solve ``A x = b``; returns (x, iterations, relative residual).  All scalars stay on the device."""
    x = torch.zeros_like(b)
    r = b.clone()
    p = r.clone()
    rr = torch.dot(r, r)
    stop = (tol * tol) * rr
    it = 0
    for it in range(1, maxiter + 1):
        ap, pap = apply(p)
        alpha = rr / pap[0]
        x.add_(p * alpha)
        r.sub_(ap * alpha)
        rr_new = torch.dot(r, r)
        if it % 8 == 0 and bool(rr_new <= stop):      # one host synchronisation every 8 iterations
            rr = rr_new
            break
        p = r + p * (rr_new / rr)
        rr = rr_new
    return x, it, float(torch.sqrt(rr / torch.dot(b, b)))
