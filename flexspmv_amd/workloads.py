"""Seeded synthetic inputs for the five benchmark workloads (numpy, host side).

Every generator returns a :class:`Workload`: the name of the prebuilt sub-graph it feeds, the tensors
in the binding's argument names, the CSR row pointer, and the algorithmic byte / flop counts used for
the roofline (every streamed array once, every gathered source once, every output once; index arrays
are int32; zero fills, scratch and re-fetches of gathered data are not counted).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np


@dataclass
class Workload:
    name: str
    graph: str                       # key into flexspmv_amd.graphs.REGISTRY
    tensors: Dict[str, np.ndarray]   # binding name -> array
    row_end_offsets: Optional[np.ndarray]
    num_rows: int
    num_cols: int
    ne: int
    algorithmic_bytes: int
    flops: int
    seed: int
    notes: str = ""
    extra: Dict[str, np.ndarray] = field(default_factory=dict)


def _rows_from_ptr(ptr: np.ndarray) -> np.ndarray:
    return np.repeat(np.arange(len(ptr) - 1, dtype=np.int32), np.diff(ptr)).astype(np.int32)


# ---------------------------------------------------------------------------------------------
# structured Laplacians
# ---------------------------------------------------------------------------------------------
def _laplacian(shape, dtype, diag):
    """CSR of the (2d+1)-point Laplacian on a grid with Dirichlet boundary; columns ascending."""
    dims = len(shape)
    n = int(np.prod(shape))
    idx = np.arange(n, dtype=np.int64)
    coords = np.unravel_index(idx, shape)
    strides = [int(np.prod(shape[d + 1:])) for d in range(dims)]
    # neighbour order that keeps columns ascending: -stride (largest first) ... self ... +stride
    offsets, valid = [], []
    for d in range(dims):
        offsets.append(-strides[d]); valid.append(coords[d] > 0)
    offsets.append(0); valid.append(np.ones(n, dtype=bool))
    for d in reversed(range(dims)):
        offsets.append(strides[d]); valid.append(coords[d] < shape[d] - 1)
    mask = np.stack(valid, axis=1)
    cols = (idx[:, None] + np.asarray(offsets, dtype=np.int64)[None, :])[mask].astype(np.int32)
    vals_row = np.full(len(offsets), -1.0, dtype=dtype)
    vals_row[dims] = diag
    vals = np.broadcast_to(vals_row, mask.shape)[mask].astype(dtype)
    ptr = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(mask.sum(axis=1), out=ptr[1:])
    return ptr, cols, vals


def laplacian_2d_spmv(n: int = 256, dtype="float32", seed: int = 1) -> Workload:
    """Workload 1: y = A x, A the 2-D 5-point Laplacian on an n x n grid (diag 4, off-diag -1)."""
    dtype = np.dtype(dtype)
    ptr, cols, vals = _laplacian((n, n), dtype, 4.0)
    N, nnz = n * n, len(cols)
    x = np.random.default_rng(seed).uniform(-1.0, 1.0, N).astype(dtype)
    b = dtype.itemsize
    return Workload("laplacian2d_%d" % n, "csr_spmv", {"vals": vals, "x": x, "selector_idx": cols}, ptr,
                    N, N, nnz, algorithmic_bytes=(4 + b) * nnz + 4 * (N + 1) + b * N + b * N,
                    flops=2 * nnz, seed=seed)


def poisson_3d_spmv_dot(n: int = 256, dtype="float64", seed: int = 5) -> Workload:
    """Workload 5: y = A x and x.y for the 3-D 7-point Laplacian on an n^3 grid (diag 6, off-diag -1)."""
    dtype = np.dtype(dtype)
    ptr, cols, vals = _laplacian((n, n, n), dtype, 6.0)
    N, nnz = n ** 3, len(cols)
    x = np.random.default_rng(seed).uniform(-1.0, 1.0, N).astype(dtype)
    b = dtype.itemsize
    return Workload("poisson3d_%d" % n, "spmv_dot",
                    {"vals": vals, "x": x, "selector_col_idx": cols, "selector_row_idx": _rows_from_ptr(ptr)},
                    ptr, N, N, nnz,
                    algorithmic_bytes=(4 + b) * nnz + 4 * (N + 1) + b * N + b * N + b,
                    flops=2 * nnz + 2 * N, seed=seed,
                    notes="selector_row_idx equals the row ids and is not read by the kernel")


# ---------------------------------------------------------------------------------------------
# R-MAT
# ---------------------------------------------------------------------------------------------
def rmat_spmv(scale: int = 22, degree: int = 16, dtype="float32", seed: int = 4,
              a: float = 0.57, b: float = 0.19, c: float = 0.19) -> Workload:
    """Workload 4: y = A x for an R-MAT graph (duplicates merged, rows in natural order)."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(seed)
    n = 1 << scale
    m = degree * n
    keys = np.zeros(m, dtype=np.int64)
    chunk = 1 << 24
    for lo in range(0, m, chunk):
        hi = min(lo + chunk, m)
        r = np.zeros(hi - lo, dtype=np.int64)
        cidx = np.zeros(hi - lo, dtype=np.int64)
        for _ in range(scale):
            u = rng.random(hi - lo)
            right = (u >= a) & (u < a + b) | (u >= a + b + c)   # quadrants b and d: column bit set
            down = u >= a + b                                    # quadrants c and d: row bit set
            r = (r << 1) | down
            cidx = (cidx << 1) | right
        keys[lo:hi] = (r << scale) | cidx
    keys = np.unique(keys)
    rows = (keys >> scale).astype(np.int64)
    cols = (keys & (n - 1)).astype(np.int32)
    del keys
    U = len(cols)
    ptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=n), out=ptr[1:])
    ptr = ptr.astype(np.int32)
    vals = rng.random(U).astype(dtype)
    x = rng.random(n).astype(dtype)
    bsz = dtype.itemsize
    return Workload("rmat_s%d_d%d" % (scale, degree), "csr_spmv",
                    {"vals": vals, "x": x, "selector_idx": cols}, ptr, n, n, U,
                    algorithmic_bytes=(4 + bsz) * U + 4 * (n + 1) + bsz * n + bsz * n,
                    flops=2 * U, seed=seed)


# ---------------------------------------------------------------------------------------------
# spring-mass on a jittered grid
# ---------------------------------------------------------------------------------------------
def spring_mass_grid(n: int = 100, dtype="float32", seed: int = 2) -> Workload:
    """Workload 2: n^3 vertices displaced by U(-0.1, 0.1) h from a regular lattice, 6-neighbour springs
    (rest length = lattice spacing h) as half-edges sorted by destination vertex."""
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(seed)
    V = n ** 3
    h = 1.0 / n
    grid = np.stack(np.meshgrid(*([np.arange(n)] * 3), indexing="ij"), axis=-1).reshape(V, 3)
    pos = ((grid + rng.uniform(-0.1, 0.1, (V, 3))) * h).astype(dtype)
    vid = np.arange(V, dtype=np.int64).reshape(n, n, n)
    a_list, b_list = [], []
    for axis in range(3):
        sl_lo = [slice(None)] * 3; sl_hi = [slice(None)] * 3
        sl_lo[axis] = slice(0, n - 1); sl_hi[axis] = slice(1, n)
        a_list.append(vid[tuple(sl_lo)].ravel()); b_list.append(vid[tuple(sl_hi)].ravel())
    sa, sb = np.concatenate(a_list), np.concatenate(b_list)
    S = len(sa)
    k_spring = rng.uniform(0.5, 2.0, S).astype(dtype)
    # springs are at rest on the regular lattice (length h); the jitter above is the displacement
    rest = np.full(S, h, dtype=dtype)
    dst = np.concatenate([sa, sb]); src = np.concatenate([sb, sa])
    kk = np.concatenate([k_spring, k_spring]); ll = np.concatenate([rest, rest])
    order = np.lexsort((src, dst))
    dst, src, kk, ll = dst[order], src[order], kk[order], ll[order]
    ptr = np.zeros(V + 1, dtype=np.int64)
    np.cumsum(np.bincount(dst, minlength=V), out=ptr[1:])
    D = len(dst)
    b = dtype.itemsize
    return Workload("spring_mass_%d" % n, "spring_mass",
                    {"pos": pos, "k": kk, "rest": ll, "gather_src_idx": src.astype(np.int32),
                     "gather_dst_idx": dst.astype(np.int32)},
                    ptr.astype(np.int32), V, V, D,
                    algorithmic_bytes=D * (4 + b + b) + 4 * (V + 1) + 3 * b * V + 3 * b * V + b,
                    flops=25 * D, seed=seed,
                    notes="gather_dst_idx equals the row ids and is not read by the kernel")


# ---------------------------------------------------------------------------------------------
# shallow water on a Delaunay mesh
# ---------------------------------------------------------------------------------------------
def shallow_water_mesh(points: int = 1_000_000, dtype="float64", seed: int = 3) -> Workload:
    """Workload 3: Rusanov flux over interior half-edges of a Delaunay triangulation of the unit
    square, sorted by destination cell.  ``extra`` holds ``area`` and ``h`` for the mass aggregator."""
    from scipy.spatial import Delaunay
    dtype = np.dtype(dtype)
    rng = np.random.default_rng(seed)
    pts = rng.random((points, 2))
    tri = Delaunay(pts)
    cells = tri.simplices                      # [C, 3]
    nbr = tri.neighbors                        # nbr[c, k] = cell opposite vertex k, -1 on the hull
    C = len(cells)
    # Cells are numbered along a Morton curve through their centroids, as mesh generators and
    # partitioners do: neighbouring cells get nearby numbers (the triangulation itself numbers them in
    # an order without locality, which turns every gather into a random access).
    from .python_wrapper.edge_order import morton_order
    order_c = morton_order(pts[cells].mean(axis=1))
    new_id = np.empty(C, dtype=np.int64)
    new_id[order_c] = np.arange(C)
    cells = cells[order_c]
    nbr = nbr[order_c]
    nbr = np.where(nbr >= 0, new_id[np.maximum(nbr, 0)], -1)
    cc, kk = np.nonzero(nbr >= 0)
    dst = cc.astype(np.int64)                  # the cell being updated
    src = nbr[cc, kk].astype(np.int64)
    # the shared edge is opposite vertex kk of cell dst
    va = cells[cc, (kk + 1) % 3]; vb = cells[cc, (kk + 2) % 3]
    ex = pts[vb] - pts[va]
    length = np.linalg.norm(ex, axis=1)
    nrm = np.stack([ex[:, 1], -ex[:, 0]], axis=1) / length[:, None]
    centroid = pts[cells].mean(axis=1)
    mid = 0.5 * (pts[va] + pts[vb])
    flip = ((mid - centroid[dst]) * nrm).sum(axis=1) < 0     # outward from dst
    nrm[flip] *= -1.0
    order = np.lexsort((src, dst))
    dst, src, nrm, length = dst[order], src[order], nrm[order], length[order]
    p0, p1, p2 = pts[cells[:, 0]], pts[cells[:, 1]], pts[cells[:, 2]]
    area = 0.5 * np.abs((p1[:, 0] - p0[:, 0]) * (p2[:, 1] - p0[:, 1]) - (p2[:, 0] - p0[:, 0]) * (p1[:, 1] - p0[:, 1]))
    hh = 1.0 + 0.1 * np.exp(-100.0 * ((centroid[:, 0] - 0.5) ** 2 + (centroid[:, 1] - 0.5) ** 2))
    U = np.zeros((C, 3), dtype=dtype)
    U[:, 0] = hh
    ptr = np.zeros(C + 1, dtype=np.int64)
    np.cumsum(np.bincount(dst, minlength=C), out=ptr[1:])
    D = len(dst)
    b = dtype.itemsize
    return Workload("swe_delaunay_%d" % points, "swe_rusanov",
                    {"U": U, "nrm": nrm.astype(dtype), "length": length.astype(dtype),
                     "gather_src_idx": src.astype(np.int32), "gather_dst_idx": dst.astype(np.int32)},
                    ptr.astype(np.int32), C, C, D,
                    algorithmic_bytes=D * (4 + 2 * b + b) + 4 * (C + 1) + 3 * b * C + 3 * b * C,
                    flops=60 * D, seed=seed,
                    notes="gather_dst_idx equals the row ids and is not read by the kernel",
                    extra={"area": area.astype(dtype), "h": np.ascontiguousarray(U[:, 0])})


def mass_sum_of(swe: Workload) -> Workload:
    """The cell-level total-mass aggregator that accompanies workload 3."""
    h, area = swe.extra["h"], swe.extra["area"]
    C = len(h)
    b = h.dtype.itemsize
    return Workload("mass_sum_%d" % C, "mass_sum", {"h": h, "area": area}, None, C, C, C,
                    algorithmic_bytes=2 * b * C + b, flops=2 * C, seed=swe.seed)


def matrix_market_spmv(path: str, dtype="float64", seed: int = 7, fused_dot: bool = False) -> Workload:
    """SpMV on a matrix read from a MatrixMarket file (the reference's CUDA harness takes one with
    ``--mtx``, src/flex_spmv_full_red.cu:643): CSR with sorted columns, duplicate entries summed,
    symmetric storage expanded; pattern matrices get unit values.  ``x`` is random in [-1, 1)."""
    import os

    import scipy.io
    import scipy.sparse as sp
    dtype = np.dtype(dtype)
    a = sp.csr_matrix(scipy.io.mmread(path))
    a.sum_duplicates()
    a.sort_indices()
    if a.nnz == 0:
        raise ValueError(f"{path}: matrix has no entries")
    if a.shape[0] + a.nnz >= 2 ** 31:
        raise ValueError(f"{path}: rows + non-zeros do not fit 32-bit offsets")
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1.0, 1.0, a.shape[1]).astype(dtype)
    vals = np.ascontiguousarray(a.data.astype(dtype))
    cols = np.ascontiguousarray(a.indices.astype(np.int32))
    ptr = np.ascontiguousarray(a.indptr.astype(np.int32))
    n, m, nnz, b = a.shape[0], a.shape[1], a.nnz, dtype.itemsize
    name = "mtx_" + os.path.splitext(os.path.basename(path))[0]
    if fused_dot:
        if n != m:
            raise ValueError("x . (A x) needs a square matrix")
        rows = np.repeat(np.arange(n, dtype=np.int32), np.diff(ptr))
        return Workload(name, "spmv_dot", {"vals": vals, "x": x, "selector_col_idx": cols, "selector_row_idx": rows},
                        ptr, n, m, nnz, algorithmic_bytes=nnz * (4 + b) + 4 * (n + 1) + b * m + b * n + b,
                        flops=2 * nnz + 2 * n, seed=seed, notes="selector_row_idx equals the row ids and is not read")
    return Workload(name, "csr_spmv", {"vals": vals, "x": x, "selector_idx": cols}, ptr, n, m, nnz,
                    algorithmic_bytes=nnz * (4 + b) + 4 * (n + 1) + b * m + b * n, flops=2 * nnz, seed=seed)


WORKLOADS = {
    "laplacian2d": laplacian_2d_spmv,
    "spring_mass": spring_mass_grid,
    "shallow_water": shallow_water_mesh,
    "rmat": rmat_spmv,
    "poisson3d": poisson_3d_spmv_dot,
}


def launch_arguments(w: Workload, param_names, device):
    """Positional arguments of ``merged_spmv_launch`` for a workload, as torch tensors on ``device``,
    in the order a library's signature lists them."""
    import torch
    args = []
    for name in param_names:
        if name == "row_end_offsets":
            ro = w.row_end_offsets if w.row_end_offsets is not None else np.array([42], dtype=np.int32)
            args.append(torch.from_numpy(np.ascontiguousarray(ro)).to(device))
        elif name == "num_rows":
            args.append(int(w.num_rows))
        elif name == "num_cols":
            args.append(int(w.num_cols))
        else:
            args.append(torch.from_numpy(np.ascontiguousarray(w.tensors[name])).to(device))
    return args
