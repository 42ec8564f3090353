"""Host side of the edge-list preparation library (``include/flexspmv_formats.h``).

The reference turns a reducer's COO row ids into a CSR row pointer with torch
(``_coo_rows_to_csr_ptr``, python_wrapper/dynamic_replace_submodule.py:20-41) and assumes that the ids are
ascending.  Here that step, the stable sort by row an unordered edge list needs first, and the
permutation of per-edge tensors are HIP kernels behind a C interface; this module is the thin layer that
hands torch's device memory and current stream to them.  There is no CPU or eager fallback: tensors must
live on the GPU and the library must be built.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

from . import build as _build

ABI_VERSION = 1
FINDING_UNSORTED = 1
FINDING_OUT_OF_RANGE = 2
EXPORTED_SYMBOLS = ("flexspmv_coo_rows_to_csr", "flexspmv_sort_workspace_bytes", "flexspmv_sort_edges_by_row",
                    "flexspmv_gather_rows", "flexspmv_scatter_rows", "flexspmv_formats_last_error",
                    "flexspmv_formats_abi_version")

_lib: Optional[ctypes.CDLL] = None


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """dlopen the formats library and type its entry points."""
    path = path or _build.FORMATS_LIBRARY
    if not os.path.exists(path):
        raise RuntimeError(f"FlexSpmv formats library {path} is not built (run __graft_entry__.build())")
    try:
        import torch  # noqa: F401  (torch's HIP runtime has to be the one in the process)
    except ImportError:
        pass
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
    vp, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    lib.flexspmv_coo_rows_to_csr.argtypes = [vp, i32, i64, i64, vp, vp, vp]
    lib.flexspmv_coo_rows_to_csr.restype = ctypes.c_int
    lib.flexspmv_sort_workspace_bytes.argtypes = [i64, i64]
    lib.flexspmv_sort_workspace_bytes.restype = sz
    lib.flexspmv_sort_edges_by_row.argtypes = [vp, i32, i64, i64, vp, vp, vp, sz, vp]
    lib.flexspmv_sort_edges_by_row.restype = ctypes.c_int
    for fn in (lib.flexspmv_gather_rows, lib.flexspmv_scatter_rows):
        fn.argtypes = [vp, vp, vp, i64, i64, vp]
        fn.restype = ctypes.c_int
    lib.flexspmv_formats_last_error.argtypes = []
    lib.flexspmv_formats_last_error.restype = ctypes.c_char_p
    lib.flexspmv_formats_abi_version.argtypes = []
    lib.flexspmv_formats_abi_version.restype = ctypes.c_int
    if lib.flexspmv_formats_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path} was built against formats ABI {lib.flexspmv_formats_abi_version()}, "
                           f"this package expects {ABI_VERSION}; rebuild it")
    return lib


def library() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = load_library()
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(f"flexspmv formats call failed ({rc}): "
                           f"{library().flexspmv_formats_last_error().decode() or 'HIP error'}")


def _stream(t) -> int:
    import torch
    return torch.cuda.current_stream(t.device).cuda_stream


def _ids(row_ids):
    import torch
    if not row_ids.is_cuda:
        raise RuntimeError("row ids must live on the GPU: the formats kernels have no CPU path")
    if row_ids.dim() != 1:
        raise RuntimeError("row ids must be 1-D")
    if row_ids.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"row ids must be int32 or int64, got {row_ids.dtype}")
    return row_ids.contiguous()


def coo_rows_to_csr_async(row_ids, num_rows: int):
    """``(row_ptr int32[num_rows + 1], findings int32[4])`` without waiting for the GPU; ``findings[0]``
    holds FINDING_* bits once the stream has run."""
    import torch
    row_ids = _ids(row_ids)
    with torch.cuda.device(row_ids.device):
        row_ptr = torch.empty(int(num_rows) + 1, dtype=torch.int32, device=row_ids.device)
        findings = torch.empty(4, dtype=torch.int32, device=row_ids.device)
        _check(library().flexspmv_coo_rows_to_csr(row_ids.data_ptr(), row_ids.element_size(), row_ids.numel(),
                                                  int(num_rows), row_ptr.data_ptr(), findings.data_ptr(),
                                                  _stream(row_ids)))
    return row_ptr, findings


def coo_rows_to_csr(row_ids, num_rows: int):
    """CSR row pointer (int32) of ascending row ids; raises on unsorted or out-of-range ids."""
    row_ptr, findings = coo_rows_to_csr_async(row_ids, num_rows)
    found = int(findings[0].item())
    if found & FINDING_OUT_OF_RANGE:
        raise RuntimeError("Reducer row ids outside [0, num_rows)")
    if found & FINDING_UNSORTED:
        raise RuntimeError("Reducer row ids must be sorted ascending for the CSR conversion; sort the edges "
                           "by destination row first (flexspmv_amd.formats.sort_edges_by_row)")
    return row_ptr


def sort_edges_by_row(row_ids, num_rows: int) -> Tuple["torch.Tensor", "torch.Tensor"]:
    """Stable sort by row: ``(sorted_rows int32, permutation int32)``, ``permutation[k]`` = old position
    of the edge now at ``k``."""
    import torch
    row_ids = _ids(row_ids)
    ne = row_ids.numel()
    with torch.cuda.device(row_ids.device):
        sorted_rows = torch.empty(ne, dtype=torch.int32, device=row_ids.device)
        permutation = torch.empty(ne, dtype=torch.int32, device=row_ids.device)
        lib = library()
        need = lib.flexspmv_sort_workspace_bytes(ne, int(num_rows))
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=row_ids.device)
        _check(lib.flexspmv_sort_edges_by_row(row_ids.data_ptr(), row_ids.element_size(), ne, int(num_rows),
                                              sorted_rows.data_ptr(), permutation.data_ptr(),
                                              workspace.data_ptr(), workspace.numel(), _stream(row_ids)))
    return sorted_rows, permutation


def mark_written(t) -> None:
    """Tell torch that ``t`` was written through its raw pointer (a kernel of this package, not a torch
    operation): the tensor's version counter goes up, as it does for torch's own in-place operations, so
    that whoever keys a cache on it (autograd's saved-tensor check, the wrapper's copies of unchanged edge
    tensors) sees the change."""
    import torch
    bump = getattr(torch.autograd.graph, "increment_version", None)
    if bump is not None:
        bump(t)
    else:                      # older torch: an in-place no-op on an empty slice bumps the counter too
        t[:0].zero_()


def _permute(fn_name: str, src, permutation, out=None):
    import torch
    if not (src.is_cuda and permutation.is_cuda):
        raise RuntimeError("tensors must live on the GPU: the formats kernels have no CPU path")
    if permutation.dtype != torch.int32 or permutation.dim() != 1:
        raise RuntimeError("permutation must be a 1-D int32 tensor")
    n = permutation.numel()
    if src.shape[0] != n:
        raise RuntimeError(f"tensor has {src.shape[0]} leading entries, the permutation {n}")
    src = src.contiguous()
    row_bytes = (src.numel() // max(n, 1)) * src.element_size()
    if n and row_bytes % 4 != 0:
        raise RuntimeError("one entry of the tensor must be a multiple of 4 bytes")
    given = out is not None
    if out is None:
        out = torch.empty_like(src)
    elif not (out.is_contiguous() and out.shape == src.shape and out.dtype == src.dtype and out.device == src.device):
        raise RuntimeError("out must be a contiguous tensor of the source's shape, dtype and device")
    with torch.cuda.device(src.device):
        _check(getattr(library(), fn_name)(src.data_ptr(), out.data_ptr(), permutation.contiguous().data_ptr(), n,
                                           row_bytes, _stream(src)))
    if given:
        mark_written(out)      # the caller's tensor changed behind torch's back
    return out


def gather_rows(src, permutation, out=None):
    """``out[k] = src[permutation[k]]`` along the leading dimension."""
    return _permute("flexspmv_gather_rows", src, permutation, out)


def scatter_rows(src, permutation, out=None):
    """``out[permutation[k]] = src[k]`` along the leading dimension."""
    return _permute("flexspmv_scatter_rows", src, permutation, out)
