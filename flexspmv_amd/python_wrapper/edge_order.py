"""Edge ordering in front of the kernel: the merge-path reducer needs the edges grouped by row.

The reference converts the Reducer's COO row ids with ``torch._convert_indices_from_coo_to_csr``
(python_wrapper/dynamic_replace_submodule.py:20-41), which is only meaningful when the ids are already
sorted.  These helpers produce that order, once, at model set-up time.  Tensors on the GPU go through the
package's own kernels (``flexspmv_amd.formats``: radix sort by row, row pointer from the ids, permutation
of per-edge tensors); tensors in host memory, which only model set-up on a machine without a GPU sees, go
through the equivalent torch calls.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import torch

from .. import formats


def stable_sort_by_row(row_ids: torch.Tensor, num_rows: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(sorted ids, permutation)``; on the GPU both are int32, in host memory int64."""
    if row_ids.is_cuda:
        return formats.sort_edges_by_row(row_ids, num_rows)
    return torch.sort(row_ids.to(torch.int64), stable=True)


def gather_edges(t: torch.Tensor, permutation: torch.Tensor) -> torch.Tensor:
    """``t[permutation]`` along the leading dimension, contiguous."""
    if t.is_cuda and t.element_size() * (t.numel() // max(t.shape[0], 1)) % 4 == 0 and t.shape[0] > 0:
        return formats.gather_rows(t, permutation.to(device=t.device, dtype=torch.int32))
    return t.index_select(0, permutation.to(device=t.device, dtype=torch.int64)).contiguous()


def scatter_edges(src: torch.Tensor, permutation: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """``out[permutation[k]] = src[k]`` along the leading dimension (``out`` is created when not given)."""
    if out is None:
        out = torch.empty_like(src, memory_format=torch.contiguous_format)
    if (src.is_cuda and out.is_contiguous() and src.shape[0] > 0
            and src.element_size() * (src.numel() // src.shape[0]) % 4 == 0):
        return formats.scatter_rows(src.reshape(out.shape), permutation.to(device=src.device, dtype=torch.int32),
                                    out=out)
    return out.index_copy_(0, permutation.to(device=src.device, dtype=torch.int64), src.reshape(out.shape))


def sort_edges_by_row(row_ids: torch.Tensor, *edge_tensors: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """Stable sort of the edges by destination row.

    Returns ``(sorted_row_ids, permutation, *edge_tensors reordered)``; ``permutation[k]`` is the old
    position of the edge now at position ``k``.  Ties keep their original order, so the per-row summation
    order of the original edge list is preserved."""
    if row_ids.dim() != 1:
        raise ValueError("row_ids must be 1-D")
    num_rows = int(row_ids.max()) + 1 if row_ids.numel() else 1
    sorted_ids, perm = stable_sort_by_row(row_ids, num_rows)
    moved = []
    for t in edge_tensors:
        if t.shape[0] != row_ids.shape[0]:
            raise ValueError("every edge tensor must have one leading entry per edge")
        moved.append(gather_edges(t, perm))
    return (sorted_ids.to(row_ids.dtype), perm.to(torch.int64), *moved)


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
    """int32 CSR row pointer of sorted row ids."""
    if row_ids.is_cuda:
        try:
            return formats.coo_rows_to_csr(row_ids, num_rows)
        except RuntimeError as e:
            if "sorted" in str(e):
                raise ValueError("row ids are not sorted; use sort_edges_by_row first") from e
            if "outside" in str(e):
                raise ValueError("row ids outside [0, num_rows)") from e
            raise
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
