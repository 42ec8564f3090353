"""Edge ordering in front of the kernel: the merge-path reducer needs the edges grouped by row.

The reference converts the Reducer's COO row ids with ``torch._convert_indices_from_coo_to_csr``
(python_wrapper/dynamic_replace_submodule.py:20-41), which is only meaningful when the ids are already
sorted.  These helpers produce that order on the device the ids live on (torch's sort is a device radix
sort), once, at model set-up time.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import torch


def sort_edges_by_row(row_ids: torch.Tensor, *edge_tensors: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """Stable sort of the edges by destination row.

    Returns ``(sorted_row_ids, permutation, *edge_tensors reordered)``; ``permutation[k]`` is the old
    position of the edge now at position ``k``.  Ties keep their original order, so the per-row summation
    order of the original edge list is preserved."""
    if row_ids.dim() != 1:
        raise ValueError("row_ids must be 1-D")
    sorted_ids, perm = torch.sort(row_ids, stable=True)
    moved = []
    for t in edge_tensors:
        if t.shape[0] != row_ids.shape[0]:
            raise ValueError("every edge tensor must have one leading entry per edge")
        moved.append(t.index_select(0, perm).contiguous())
    return (sorted_ids, perm, *moved)


def half_edges(src: torch.Tensor, dst: torch.Tensor, *edge_tensors: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """Directed half-edges of an undirected edge list, sorted by destination.

    "Scatter into both endpoints" is expressed as one reducer over the destinations of the doubled list
    ``(src -> dst)`` followed by ``(dst -> src)``.  Returns ``(src2, dst2, sign, origin, *edge_tensors
    doubled)`` sorted by ``dst2``; ``sign`` is +1 for an edge in its original direction and -1 for its
    mirror; ``origin`` is the index of the undirected edge."""
    ne = src.shape[0]
    s2 = torch.cat([src, dst])
    d2 = torch.cat([dst, src])
    sign = torch.cat([torch.ones(ne, device=src.device), -torch.ones(ne, device=src.device)])
    origin = torch.arange(ne, device=src.device).repeat(2)
    doubled = [torch.cat([t, t]) for t in edge_tensors]
    d_sorted, perm, s_sorted, sign_s, origin_s, *rest = sort_edges_by_row(d2, s2, sign, origin, *doubled)
    return (s_sorted, d_sorted, sign_s, origin_s, *rest)


def coo_to_csr(row_ids: torch.Tensor, num_rows: int) -> torch.Tensor:
    """int32 CSR row pointer of sorted row ids (histogram + inclusive scan on the ids' device)."""
    if row_ids.numel() > 1 and bool((row_ids[1:] < row_ids[:-1]).any()):
        raise ValueError("row ids are not sorted; use sort_edges_by_row first")
    counts = torch.bincount(row_ids.to(torch.int64), minlength=num_rows)
    if counts.numel() != num_rows:
        raise ValueError("row ids outside [0, num_rows)")
    ptr = torch.zeros(num_rows + 1, dtype=torch.int64, device=row_ids.device)
    torch.cumsum(counts, dim=0, out=ptr[1:])
    if int(ptr[-1]) >= 2 ** 31:
        raise ValueError("edge count does not fit 32-bit offsets")
    return ptr.to(torch.int32)


def morton_order(xy) -> "numpy.ndarray":
    """Permutation that sorts 2-D points of the unit square (numpy ``[n, 2]``) along a Morton curve.

    Numbering mesh cells in this order gives neighbouring cells nearby numbers, which keeps the gathers
    of a face loop inside a few cache lines; triangulators number cells without any locality."""
    import numpy as np
    lo = xy.min(axis=0)
    span = np.maximum(xy.max(axis=0) - lo, 1e-300)
    q = np.minimum(((xy - lo) / span * 65536.0).astype(np.uint64), 65535)

    def spread(v):
        v = (v | (v << np.uint64(8))) & np.uint64(0x00FF00FF)
        v = (v | (v << np.uint64(4))) & np.uint64(0x0F0F0F0F)
        v = (v | (v << np.uint64(2))) & np.uint64(0x33333333)
        return (v | (v << np.uint64(1))) & np.uint64(0x55555555)
    return np.argsort(spread(q[:, 0]) | (spread(q[:, 1]) << np.uint64(1)), kind="stable")
