"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of the edge-list preparation in front of a launch.

``coo_rows_to_csr`` follows the reference's fallback branch of ``_coo_rows_to_csr_ptr``
(python_wrapper/dynamic_replace_submodule.py:35-39): ``bincount`` of the row ids with ``minlength =
num_rows``, a leading zero, then the inclusive running sum.  Pinned in tests/test_formats.py by a
brute-force count of ids smaller than r on small inputs, by ``searchsorted`` on larger ones and by the
invariants of a row pointer (first entry 0, last entry ne, differences = row lengths).

``sort_edges_by_row`` has no counterpart in the reference (it assumes ascending ids); the definition is
"stable sort by row id", restated with numpy's stable argsort and pinned against Python's ``sorted`` (stable
by specification) on (row, position) pairs.

``gather_rows`` / ``scatter_rows`` are the two directions of applying that permutation.
"""
from __future__ import annotations

import numpy as np


def coo_rows_to_csr(row_ids: np.ndarray, num_rows: int) -> np.ndarray:
    """int32 row pointer of ascending row ids; raises like the product on unsorted / out-of-range ids."""
    ids = np.asarray(row_ids).astype(np.int64)
    if ids.size and (ids.min() < 0 or ids.max() >= num_rows):
        raise RuntimeError("Reducer row ids outside [0, num_rows)")
    if ids.size > 1 and np.any(ids[1:] < ids[:-1]):
        raise RuntimeError("Reducer row ids must be sorted ascending")
    counts = np.bincount(ids, minlength=num_rows)
    ptr = np.zeros(num_rows + 1, dtype=np.int64)
    ptr[1:] = np.cumsum(counts)
    return ptr.astype(np.int32)


def sort_edges_by_row(row_ids: np.ndarray):
    """(sorted ids int32, permutation int32) of a stable sort by row id."""
    ids = np.asarray(row_ids).astype(np.int64)
    perm = np.argsort(ids, kind="stable")
    return ids[perm].astype(np.int32), perm.astype(np.int32)


def gather_rows(src: np.ndarray, permutation: np.ndarray) -> np.ndarray:
    return np.asarray(src)[np.asarray(permutation, dtype=np.int64)]


def scatter_rows(src: np.ndarray, permutation: np.ndarray) -> np.ndarray:
    out = np.empty_like(np.asarray(src))
    out[np.asarray(permutation, dtype=np.int64)] = src
    return out
