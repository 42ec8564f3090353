"""Mass-spring lattice: per-spring Hooke force from gathered end points, summed per node by a reducer,
total elastic energy by an aggregator, then a symplectic Euler update of velocity and position.  It is
the map + reducer + aggregator mix of the spring-mass benchmark workload, as a steppable model."""
from __future__ import annotations

import numpy as np
import torch

from .. import frontend as esr
from ..python_wrapper.edge_order import half_edges


class SpringMass(esr.Module):
    def __init__(self, pos: torch.Tensor, springs: torch.Tensor, stiffness: float = 50.0, dt: float = 1e-3) -> None:
        """``pos`` [n, 3]; ``springs`` [m, 2] undirected node pairs; rest lengths are the initial ones."""
        super().__init__()
        a, b = springs[:, 0], springs[:, 1]
        rest = (pos[a] - pos[b]).norm(dim=1)
        src, dst, _sign, _origin, rest2 = half_edges(a, b, rest)
        self.k, self.dt = stiffness, dt
        self.pos = esr.Tensor(pos.clone())
        self.vel = esr.Tensor(torch.zeros_like(pos))
        self.force = esr.Tensor(torch.zeros_like(pos))
        self.energy = esr.Tensor(torch.zeros(1, dtype=pos.dtype, device=pos.device))
        self.rest = esr.Tensor(rest2.reshape(-1, 1).contiguous())
        self.at_src = esr.Selector(src)
        self.at_dst = esr.Selector(dst)
        self.to_dst = esr.Reducer(dst, pos.shape[0])

    def forward(self):
        d = self.at_src(self.pos) - self.at_dst(self.pos)           # [2m, 3]
        length = esr.norm(d)                                        # [2m, 1]
        stretch = length - self.rest
        pull = self.k * stretch * d / length                        # on dst, towards src when stretched
        self.force[:] = self.to_dst(pull)
        self.energy[:] = esr.sum(0.25 * self.k * stretch * stretch)  # every spring appears twice
        self.vel.add_(self.dt * self.force)
        self.pos.add_(self.dt * self.vel)


def lattice(n: int = 12, jitter: float = 0.1, seed: int = 2, dtype=torch.float32, device="cpu"):
    """(positions [n^3, 3], springs [m, 2]) of a cubic lattice with nearest-neighbour springs."""
    rng = np.random.default_rng(seed)
    ii, jj, kk = np.meshgrid(np.arange(n), np.arange(n), np.arange(n), indexing="ij")
    node = (ii * n + jj) * n + kk
    pos = np.stack([ii, jj, kk], axis=-1).reshape(-1, 3).astype(np.float64)
    pos += rng.uniform(-jitter, jitter, pos.shape)
    pairs = []
    for axis in range(3):
        lo = [slice(None)] * 3
        hi = [slice(None)] * 3
        lo[axis], hi[axis] = slice(0, n - 1), slice(1, n)
        pairs.append(np.stack([node[tuple(lo)].ravel(), node[tuple(hi)].ravel()], axis=1))
    springs = np.concatenate(pairs)
    return (torch.from_numpy(pos).to(dtype).to(device), torch.from_numpy(springs.astype(np.int64)).to(device))
