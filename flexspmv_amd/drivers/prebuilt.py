"""The fused sub-graphs of the driver models, for building their libraries ahead of time.

Sub-graph descriptions do not depend on mesh or lattice size (item shapes only), so the libraries built
from small instances serve instances of any size."""
from __future__ import annotations

from typing import Callable, Dict, List

import torch

from .. import frontend as esr
from ..ir import FusedGraphIR


def _system(device="cpu", dtype=torch.float64, num_nnz=64, sorted_rows=True):
    from .system_model import make_system
    return make_system(num_nnz, 17, 13, device=device, dtype=dtype, sorted_rows=sorted_rows)


def _swe(device="cpu", dtype=torch.float64, points=900, dt=0.0005, mesh=None):
    """``dt`` is a literal of the generated kernels (as every Python number of a model is): another value
    means other libraries.  0.0005 is stable up to about 250k mesh points (gravity wave speed is ~1).
    ``mesh``: a file written by ``shallow_water.save_mesh`` instead of a generated mesh."""
    from .shallow_water import ShallowWaterEquation, load_mesh, synthetic_mesh
    if mesh is not None:
        return ShallowWaterEquation(load_mesh(mesh, dtype=dtype, device=device), dt=dt)
    return ShallowWaterEquation(synthetic_mesh(points, dtype=dtype, device=device), dt=dt)


def _spring(device="cpu", dtype=torch.float32, n=8):
    from .spring_mass import SpringMass, lattice
    pos, springs = lattice(n, dtype=dtype, device=device)
    model = SpringMass(pos, springs)
    with torch.no_grad():
        model.pos.mul_(1.05)          # start 5 % stretched: the lattice breathes
    return model


def _swe_parts(device="cpu", points=900):
    from .shallow_water_assembly import MeshComponentsCollector, synthetic_topology
    return MeshComponentsCollector(synthetic_topology(points, device=device))


def _swe_init(device="cpu", dtype=torch.float64, points=900):
    from .shallow_water_assembly import Initializer, MeshComponentsCollector, synthetic_topology
    mesh = synthetic_topology(points, device=device)
    parts = MeshComponentsCollector(mesh)
    parts()
    return Initializer(mesh, parts, dtype)


MODELS: Dict[str, Callable[..., torch.nn.Module]] = {"system": _system, "swe": _swe, "spring": _spring,
                                                     "swe_parts": _swe_parts, "swe_init": _swe_init}


def model_graphs() -> List[FusedGraphIR]:
    """Every sub-graph of every driver model that the generators implement."""
    from ..python_wrapper.accelerate import lower_submodules
    out: List[FusedGraphIR] = []
    for name, factory in MODELS.items():
        [compiled] = esr.compile([factory()], "torch")
        irs, _ = lower_submodules(compiled, prefix=name)
        out.extend(irs.values())
    return out
