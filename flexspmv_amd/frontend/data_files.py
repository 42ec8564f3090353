"""Named arrays from a file: the stand-in for EASIER's ``esr.hdf5(path, dataset, dtype=...)``.

The reference's drivers read their mesh and initial state dataset by dataset from HDF5 files
(shallow_water_equation/swe_main.py:19-71).  Two containers are understood here:

* ``.npz`` - numpy's own archive, always available (``numpy.load`` with ``allow_pickle=False``);
* ``.hdf5`` / ``.h5`` - through ``h5py`` when it can be imported; where it cannot, the call fails and says so
  (there is no partial HDF5 reader in this package).

``save_arrays`` writes either container from a dict of arrays, so a mesh assembled on one machine can be
handed to a run on another.
"""
from __future__ import annotations

import os
from typing import Dict, Mapping, Optional

import numpy as np
import torch

_HDF5_SUFFIXES = (".hdf5", ".h5", ".hdf")


def _h5py(path: str):
    try:
        import h5py  # type: ignore
    except ImportError as e:
        raise RuntimeError(f"{path}: reading or writing HDF5 needs the h5py package, which cannot be imported "
                           "here; convert the file to .npz (numpy.savez) on a machine that has it") from e
    return h5py


def hdf5(path: str, dataset: str, dtype: Optional[torch.dtype] = None, device=None) -> torch.Tensor:
    """The array stored under ``dataset`` in ``path`` as a tensor (same call as ``esr.hdf5``)."""
    if not os.path.exists(path):
        raise FileNotFoundError(path)
    if path.lower().endswith(_HDF5_SUFFIXES):
        with _h5py(path).File(path, "r") as f:
            if dataset not in f:
                raise KeyError(f"{path} has no dataset {dataset!r}")
            arr = np.asarray(f[dataset][...])
    elif path.lower().endswith(".npz"):
        with np.load(path, allow_pickle=False) as f:
            if dataset not in f.files:
                raise KeyError(f"{path} has no array {dataset!r} (it has {sorted(f.files)})")
            arr = f[dataset]
    else:
        raise RuntimeError(f"{path}: unknown container (expected .npz, .hdf5 or .h5)")
    t = torch.from_numpy(np.ascontiguousarray(arr))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(device) if device is not None else t


def datasets(path: str):
    """Names of the arrays in ``path``."""
    if path.lower().endswith(_HDF5_SUFFIXES):
        with _h5py(path).File(path, "r") as f:
            return sorted(f.keys())
    with np.load(path, allow_pickle=False) as f:
        return sorted(f.files)


def save_arrays(path: str, arrays: Mapping[str, object]) -> None:
    """Write ``{name: tensor or array or number}`` to ``path`` (.npz, or .hdf5 / .h5 with h5py)."""
    host: Dict[str, np.ndarray] = {}
    for name, a in arrays.items():
        host[name] = a.detach().cpu().numpy() if isinstance(a, torch.Tensor) else np.asarray(a)
    if path.lower().endswith(_HDF5_SUFFIXES):
        with _h5py(path).File(path, "w") as f:
            for name, a in host.items():
                f.create_dataset(name, data=a)
    elif path.lower().endswith(".npz"):
        np.savez(path, **host)
    else:
        raise RuntimeError(f"{path}: unknown container (expected .npz, .hdf5 or .h5)")
