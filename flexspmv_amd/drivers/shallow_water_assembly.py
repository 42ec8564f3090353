"""Mesh pre-processing models of the shallow-water pipeline.

The reference prepares the inputs of its shallow-water model with two more models
(shallow_water_equation/assemble_shallow_water.py): a *components collector* that only shuffles int64
index data (per face, the three point ids of both neighbouring cells; per wall face, its two point
ids), and an *initializer* that derives the geometry (face normals scaled by face length, interpolation
weights, cell areas and centroids, the initial height) with a mix of ``sign / where / lt / abs / exp``.
They are the second and third pipelines of its A/B driver (test_full/easier_full.py:48-56).  Here they
take the mesh arrays directly instead of HDF5 paths."""
from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from .. import frontend as esr
from ..python_wrapper.edge_order import morton_order


def synthetic_topology(points: int = 900, seed: int = 3, device="cpu") -> Dict[str, torch.Tensor]:
    """points [np, 2] float64, cells [nc, 3], src/dst [ne] (directed interior faces sorted by dst),
    bcells [nbc], bpoints [nbc, 2] of a Delaunay mesh of a jittered lattice on the unit square."""
    from scipy.spatial import Delaunay
    rng = np.random.default_rng(seed)
    m = max(3, int(round(points ** 0.5)))
    gx, gy = np.meshgrid(np.arange(m), np.arange(m), indexing="ij")
    jitter = rng.uniform(-0.25, 0.25, (m * m, 2))
    edge = (gx.ravel() == 0) | (gx.ravel() == m - 1) | (gy.ravel() == 0) | (gy.ravel() == m - 1)
    jitter[edge] = 0.0
    pts = (np.stack([gx.ravel(), gy.ravel()], axis=1) + jitter) / (m - 1) - 0.5
    tri = Delaunay(pts)
    cells, nbr = tri.simplices.astype(np.int64), tri.neighbors
    order_c = morton_order(pts[cells].mean(axis=1))     # number the cells with spatial locality
    new_id = np.empty(len(cells), dtype=np.int64)
    new_id[order_c] = np.arange(len(cells))
    cells, nbr = cells[order_c], nbr[order_c]
    nbr = np.where(nbr >= 0, new_id[np.maximum(nbr, 0)], -1)
    dst, k = np.nonzero(nbr >= 0)
    src = nbr[dst, k]
    order = np.lexsort((src, dst))
    bc, bk = np.nonzero(nbr < 0)
    ob = np.argsort(bc, kind="stable")
    bc, bk = bc[ob], bk[ob]
    bpoints = np.stack([cells[bc, (bk + 1) % 3], cells[bc, (bk + 2) % 3]], axis=1)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)   # noqa: E731
    return {"points": t(pts), "cells": t(cells), "src": t(src[order].astype(np.int64)),
            "dst": t(dst[order].astype(np.int64)), "bcells": t(bc.astype(np.int64)), "bpoints": t(bpoints)}


class MeshComponentsCollector(esr.Module):
    """Per-face and per-cell point ids as separate int64 vectors."""

    def __init__(self, mesh: Dict[str, torch.Tensor]) -> None:
        super().__init__()
        ne, nc, nbc = mesh["src"].shape[0], mesh["cells"].shape[0], mesh["bcells"].shape[0]
        dev = mesh["cells"].device
        self.cells = esr.Tensor(mesh["cells"].clone())
        self.bpoints = esr.Tensor(mesh["bpoints"].clone())
        self.selector_src = esr.Selector(mesh["src"])
        self.selector_dst = esr.Selector(mesh["dst"])

        def zeros(n, count):
            return torch.nn.ParameterList([esr.Tensor(torch.zeros(n, dtype=torch.long, device=dev))
                                           for _ in range(count)])
        self.src_p, self.dst_p, self.cells_p, self.bp = zeros(ne, 3), zeros(ne, 3), zeros(nc, 3), zeros(nbc, 2)

    def forward(self):
        src_p = self.selector_src(self.cells)
        dst_p = self.selector_dst(self.cells)
        for i in range(3):
            self.src_p[i].copy_(src_p[:, i].clone())
            self.dst_p[i].copy_(dst_p[:, i].clone())
            self.cells_p[i].copy_(self.cells[:, i].clone())
        for i in range(2):
            self.bp[i].copy_(self.bpoints[:, i].clone())


class Initializer(esr.Module):
    """Geometry and initial state from the point coordinates and the collected point ids."""

    def __init__(self, mesh: Dict[str, torch.Tensor], components: MeshComponentsCollector,
                 dtype=torch.float64) -> None:
        super().__init__()
        dev = mesh["points"].device
        self.points = esr.Tensor(mesh["points"].to(dtype))
        sel = lambda plist: torch.nn.ModuleList([esr.Selector(p.data) for p in plist])   # noqa: E731
        self.selector_src_p = sel(components.src_p)
        self.selector_dst_p = sel(components.dst_p)
        self.selector_cells_p = sel(components.cells_p)
        self.selector_bp = sel(components.bp)
        self.bselector = esr.Selector(mesh["bcells"])
        ne, nc, nbc = mesh["src"].shape[0], mesh["cells"].shape[0], mesh["bcells"].shape[0]
        for name, n in (("x", nc), ("y", nc), ("area", nc), ("h", nc), ("sx", ne), ("sy", ne), ("alpha", ne),
                        ("bsx", nbc), ("bsy", nbc)):
            setattr(self, name, esr.Tensor(torch.zeros(n, dtype=dtype, device=dev)))
        self.centroid = esr.Tensor(torch.zeros(nc, 2, dtype=dtype, device=dev))

    @staticmethod
    def crossing_weight(sc, dc, p0, p1):
        """Where the segment src centroid -> dst centroid crosses the face p0-p1, as a fraction of it."""
        x1, y1, x2, y2 = sc[:, 0].clone(), sc[:, 1].clone(), dc[:, 0].clone(), dc[:, 1].clone()
        x3, y3, x4, y4 = p0[:, 0].clone(), p0[:, 1].clone(), p1[:, 0].clone(), p1[:, 1].clone()
        return ((x3 - x1) * (y4 - y3) - (y3 - y1) * (x4 - x3)) / ((x2 - x1) * (y4 - y3) - (y2 - y1) * (x4 - x3))

    @staticmethod
    def face_normal(inside, p1, p2):
        """Normal of face p1-p2 scaled by its length, pointing away from ``inside``."""
        a1, a2 = inside[:, 0].clone(), inside[:, 1].clone()
        b1, b2, c1, c2 = p1[:, 0].clone(), p1[:, 1].clone(), p2[:, 0].clone(), p2[:, 1].clone()
        s = torch.sign((b1 - c1) * (a2 - c2) - (b2 - c2) * (a1 - c1))
        return s * (b2 - c2), -s * (b1 - c1)

    def forward(self):
        sp = [s(self.points) for s in self.selector_src_p]
        dp = [s(self.points) for s in self.selector_dst_p]
        src_cent = (sp[0] + sp[1] + sp[2]) / 3.
        dst_cent = (dp[0] + dp[1] + dp[2]) / 3.
        first = True
        for a, b, c in ((0, 1, 2), (1, 2, 0), (2, 0, 1)):       # face a-b of the src cell, c opposite
            nx, ny = self.face_normal(sp[c], sp[a], sp[b])
            mx, my = self.face_normal(dst_cent, sp[a], sp[b])
            shared = (nx * mx + ny * my) < 0                     # the dst centroid lies beyond this face
            weight = self.crossing_weight(src_cent, dst_cent, sp[a], sp[b])
            self.sx[:] = torch.where(shared, nx, 0. if first else self.sx)
            self.sy[:] = torch.where(shared, ny, 0. if first else self.sy)
            self.alpha[:] = torch.where(shared, weight, 0. if first else self.alpha)
            first = False

        cp = [s(self.points) for s in self.selector_cells_p]
        x0, y0, x1, y1, x2, y2 = (cp[0][:, 0].clone(), cp[0][:, 1].clone(), cp[1][:, 0].clone(),
                                  cp[1][:, 1].clone(), cp[2][:, 0].clone(), cp[2][:, 1].clone())
        self.area[:] = 0.5 * torch.abs(x0 * (y1 - y2) + x1 * (y2 - y0) + x2 * (y0 - y1))
        self.centroid[:] = (cp[0] + cp[1] + cp[2]) / 3.
        self.x[:] = self.centroid[:, 0].clone()
        self.y[:] = self.centroid[:, 1].clone()
        self.h[:] = 1 + 0.1 * torch.exp(-100 * ((self.x - 0.0) ** 2 + (self.y - 0.0) ** 2))

        wall_inside = self.bselector(self.centroid)
        bnx, bny = self.face_normal(wall_inside, self.selector_bp[0](self.points), self.selector_bp[1](self.points))
        self.bsx[:] = -bnx          # like the interior normals, wall normals point into the receiving cell
        self.bsy[:] = -bny


def mesh_for_model(topology: Dict[str, torch.Tensor], init: "Initializer") -> Dict[str, torch.Tensor]:
    """The arrays :class:`flexspmv_amd.drivers.shallow_water.ShallowWaterEquation` takes."""
    out = {k: topology[k] for k in ("src", "dst", "bcells")}
    out["nc"] = topology["cells"].shape[0]
    for k in ("x", "y", "area", "sx", "sy", "bsx", "bsy", "alpha", "h"):
        out[k] = getattr(init, k).data
    return out


def assemble(points: int = 900, seed: int = 3, device="cpu", dtype=torch.float64):
    """(topology, collector after its run, initializer after its run): the two pre-processing models
    run on their torch sub-modules."""
    mesh = synthetic_topology(points, seed, device)
    collector = MeshComponentsCollector(mesh)
    collector()
    init = Initializer(mesh, collector, dtype)
    init()
    return mesh, collector, init
