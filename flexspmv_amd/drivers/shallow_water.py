"""Shallow-water equations on an unstructured triangular mesh, fourth-order Runge-Kutta in time.

The model is the one the reference accelerates end to end (shallow_water_equation/swe_main.py:13-140):
cell-centred height ``h`` and momenta ``uh, vh``; every interior face is a directed half-edge
``src -> dst`` sorted by ``dst``; face values are interpolated with weight ``alpha``; fluxes through the
scaled face normals ``(sx, sy)`` are summed per destination cell by one ``Reducer``; wall faces add the
pressure term through a second ``Reducer`` over the boundary cells.  The reference reads its mesh from
HDF5 files; here the same arrays come from a Delaunay triangulation of a jittered lattice of points, or from
a file written by ``save_mesh`` (``.npz`` everywhere, ``.hdf5`` where h5py exists) and read dataset by
dataset like the reference's."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from .. import frontend as esr
from ..python_wrapper.edge_order import morton_order


def synthetic_mesh(points: int = 2000, seed: int = 3, dtype=torch.float64, device="cpu") -> Dict[str, torch.Tensor]:
    """Arrays of the reference's mesh / initial-state files for a Delaunay mesh of the unit square
    (about ``points`` vertices)."""
    from scipy.spatial import Delaunay
    rng = np.random.default_rng(seed)
    m = max(3, int(round(points ** 0.5)))                 # jittered lattice: well-shaped triangles
    gx, gy = np.meshgrid(np.arange(m), np.arange(m), indexing="ij")
    jitter = rng.uniform(-0.25, 0.25, (m * m, 2))
    edge = (gx.ravel() == 0) | (gx.ravel() == m - 1) | (gy.ravel() == 0) | (gy.ravel() == m - 1)
    jitter[edge] = 0.0                                    # a straight hull: no sliver cells along the walls
    pts = (np.stack([gx.ravel(), gy.ravel()], axis=1) + jitter) / (m - 1)
    tri = Delaunay(pts)
    cells, nbr = tri.simplices, tri.neighbors           # nbr[c, k]: cell opposite vertex k (-1: wall)
    nc = len(cells)
    order_c = morton_order(pts[cells].mean(axis=1))     # number the cells with spatial locality
    new_id = np.empty(nc, dtype=np.int64)
    new_id[order_c] = np.arange(nc)
    cells, nbr = cells[order_c], nbr[order_c]
    nbr = np.where(nbr >= 0, new_id[np.maximum(nbr, 0)], -1)
    centroid = pts[cells].mean(axis=1)
    p0, p1, p2 = pts[cells[:, 0]], pts[cells[:, 1]], pts[cells[:, 2]]
    area = 0.5 * np.abs((p1[:, 0] - p0[:, 0]) * (p2[:, 1] - p0[:, 1]) - (p2[:, 0] - p0[:, 0]) * (p1[:, 1] - p0[:, 1]))

    def faces(mask):
        c, k = np.nonzero(mask)
        va, vb = cells[c, (k + 1) % 3], cells[c, (k + 2) % 3]
        e = pts[vb] - pts[va]
        n = np.stack([e[:, 1], -e[:, 0]], axis=1)                 # |n| = face length
        mid = 0.5 * (pts[va] + pts[vb])
        n[((mid - centroid[c]) * n).sum(axis=1) < 0] *= -1.0      # outward from cell c
        return c, k, n, mid

    dst, k, n_in, mid = faces(nbr >= 0)
    src = nbr[dst, k]
    d_dst = np.linalg.norm(mid - centroid[dst], axis=1)
    d_src = np.linalg.norm(mid - centroid[src], axis=1)
    alpha = d_src / (d_src + d_dst)                                # weight of the dst value at the face
    order = np.lexsort((src, dst))
    dst, src, n_in, alpha = dst[order], src[order], n_in[order], alpha[order]
    bcells, _, n_b, _ = faces(nbr < 0)
    order_b = np.argsort(bcells, kind="stable")
    bcells, n_b = bcells[order_b], n_b[order_b]
    h0 = 1.0 + 0.1 * np.exp(-100.0 * ((centroid[:, 0] - 0.5) ** 2 + (centroid[:, 1] - 0.5) ** 2))

    def val(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(device)

    def idx(a):
        return torch.from_numpy(np.ascontiguousarray(a).astype(np.int64)).to(device)

    return {"src": idx(src), "dst": idx(dst), "bcells": idx(bcells), "nc": nc,
            "x": val(centroid[:, 0]), "y": val(centroid[:, 1]), "area": val(area),
            "sx": val(n_in[:, 0]), "sy": val(n_in[:, 1]), "bsx": val(n_b[:, 0]), "bsy": val(n_b[:, 1]),
            "alpha": val(alpha), "h": val(h0)}


MESH_INDEX_ARRAYS = ("src", "dst", "bcells")
MESH_VALUE_ARRAYS = ("x", "y", "area", "sx", "sy", "bsx", "bsy", "alpha", "h")


def save_mesh(mesh: Dict[str, torch.Tensor], path: str) -> None:
    """Write the arrays of ``synthetic_mesh`` (or any mesh with the same names) to ``path``."""
    esr.save_arrays(path, {k: mesh[k] for k in MESH_INDEX_ARRAYS + MESH_VALUE_ARRAYS + ("nc",)})


def load_mesh(path: str, dtype=torch.float64, device="cpu") -> Dict[str, torch.Tensor]:
    """The mesh dict of a file, read one dataset at a time (the reference's ``esr.hdf5(path, name, dtype=...)``
    calls, swe_main.py:19-71); ``nc`` is taken from the file or, failing that, from the cell arrays."""
    mesh: Dict[str, torch.Tensor] = {}
    for name in MESH_INDEX_ARRAYS:
        mesh[name] = esr.hdf5(path, name, dtype=torch.long, device=device)
    for name in MESH_VALUE_ARRAYS:
        mesh[name] = esr.hdf5(path, name, dtype=dtype, device=device)
    mesh["nc"] = int(esr.hdf5(path, "nc")) if "nc" in esr.datasets(path) else int(mesh["x"].shape[0])
    ne, nb = mesh["src"].shape[0], mesh["bcells"].shape[0]
    for name, n in (("dst", ne), ("sx", ne), ("sy", ne), ("alpha", ne), ("bsx", nb), ("bsy", nb),
                    ("y", mesh["nc"]), ("area", mesh["nc"]), ("h", mesh["nc"]), ("x", mesh["nc"])):
        if mesh[name].shape[0] != n:
            raise ValueError(f"{path}: array {name!r} has {mesh[name].shape[0]} entries, expected {n}")
    for name in MESH_INDEX_ARRAYS:
        if mesh[name].numel() and (int(mesh[name].min()) < 0 or int(mesh[name].max()) >= mesh["nc"]):
            raise ValueError(f"{path}: {name!r} refers to cells outside [0, {mesh['nc']})")
    return mesh


class ShallowWaterEquation(esr.Module):
    def __init__(self, mesh: Dict[str, torch.Tensor], dt: float = 0.005) -> None:
        super().__init__()
        self.dt = dt
        nc = int(mesh["nc"])
        self.nc = nc
        self.scatter = esr.Reducer(mesh["dst"], nc)
        self.gather_src = esr.Selector(mesh["src"])
        self.gather_dst = esr.Selector(mesh["dst"])
        self.scatter_b = esr.Reducer(mesh["bcells"], nc)
        self.gather_b = esr.Selector(mesh["bcells"])
        for name in ("x", "y", "area", "sx", "sy", "bsx", "bsy", "h", "alpha"):
            setattr(self, name, esr.Tensor(mesh[name].clone(), mode="partition"))
        self.uh = esr.Tensor(torch.zeros_like(mesh["h"]), mode="partition")
        self.vh = esr.Tensor(torch.zeros_like(mesh["h"]), mode="partition")

    def face_reconstruct(self, phi):
        return (1.0 - self.alpha) * self.gather_src(phi) + self.alpha * self.gather_dst(phi)

    def delta(self, h, uh, vh):
        h_f, uh_f, vh_f = self.face_reconstruct(h), self.face_reconstruct(uh), self.face_reconstruct(vh)
        u_f, v_f = uh_f / h_f, vh_f / h_f
        pressure_f = 0.5 * h_f * h_f
        flux_x, flux_y = uh_f * self.sx, vh_f * self.sy
        wall_pressure = 0.5 * self.gather_b(h) ** 2

        d_h = -(self.scatter(flux_x + flux_y)) / self.area
        d_uh = -(self.scatter((u_f * uh_f + pressure_f) * self.sx + u_f * flux_y)
                 + self.scatter_b(wall_pressure * self.bsx)) / self.area
        d_vh = -(self.scatter(v_f * flux_x + (v_f * vh_f + pressure_f) * self.sy)
                 + self.scatter_b(wall_pressure * self.bsy)) / self.area
        return d_h, d_uh, d_vh

    def forward(self):
        dt = self.dt
        k1 = self.delta(self.h, self.uh, self.vh)
        k2 = self.delta(*[q + 0.5 * dt * k for q, k in zip((self.h, self.uh, self.vh), k1)])
        k3 = self.delta(*[q + 0.5 * dt * k for q, k in zip((self.h, self.uh, self.vh), k2)])
        k4 = self.delta(*[q + dt * k for q, k in zip((self.h, self.uh, self.vh), k3)])
        for q, a, b, c, d in zip((self.h, self.uh, self.vh), k1, k2, k3, k4):
            q.add_(dt / 6 * (a + b + c + d))
