"""Stand-ins for the few EASIER names the reference's models are written against.

The reference's drivers build their models from ``easier.Module``, ``easier.Tensor``,
``easier.Selector``, ``easier.Reducer``, ``easier.sum`` and ``easier.zeros`` (easier_spmv.py:17-69,
shallow_water_equation/swe_main.py:13-140) and hand them to ``easier.compile``.  EASIER is not a
dependency of this package; these classes give the same modelling surface on plain ``torch`` so that
such a model can be traced, fused and accelerated here, on one device.  Their eager semantics are the
ones the fused kernels are checked against:

* ``Selector(idx)(x)``     ``x[idx]``                       (gather rows of a vertex tensor per edge)
* ``Reducer(idx, n)(x)``   ``zeros(n, ...).index_add_(0, idx, x)``   (sum edge values per row)
* ``sum(x)``               ``x.sum(dim=0, keepdim=True)``   (aggregate over all edges)
* ``norm(x)``              2-norm of every item, ``[n, 1]``
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch
import torch.fx
import torch.nn as nn


class Tensor(nn.Parameter):
    """A distributed tensor of the model in the reference (``esr.Tensor(data, mode='partition')``);
    here simply a parameter without gradient whose storage the fused kernels read and write."""

    def __new__(cls, data: torch.Tensor, mode: str = "partition"):
        t = torch.Tensor._make_subclass(cls, data.detach(), False)
        t.mode = mode
        return t

    def __deepcopy__(self, memo):
        out = type(self)(self.data.clone(memory_format=torch.preserve_format), getattr(self, "mode", "partition"))
        memo[id(self)] = out
        return out

    def collect(self) -> torch.Tensor:
        """The whole tensor (the reference gathers the partitions of every rank; one device here)."""
        return self.data

    def __repr__(self) -> str:  # pragma: no cover - cosmetic
        return "frontend.Tensor(" + repr(self.data) + ")"


def zeros(size: Sequence[int], dtype: Optional[torch.dtype] = None, device=None) -> torch.Tensor:
    return torch.zeros(tuple(size), dtype=dtype, device=device)


class Selector(nn.Module):
    """``y[e] = x[idx[e]]``."""

    def __init__(self, idx: torch.Tensor) -> None:
        super().__init__()
        if idx.dim() != 1 or idx.dtype not in (torch.int32, torch.int64):
            raise TypeError("Selector index must be a 1-D int32/int64 tensor")
        self.register_buffer("idx", idx.clone(), persistent=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return x[self.idx.long()]


class Reducer(nn.Module):
    """``y[r] = sum of x[e] over the edges e with idx[e] == r``, for ``r`` in ``[0, n)``."""

    def __init__(self, idx: torch.Tensor, n: int) -> None:
        super().__init__()
        if idx.dim() != 1 or idx.dtype not in (torch.int32, torch.int64):
            raise TypeError("Reducer index must be a 1-D int32/int64 tensor")
        self.register_buffer("idx", idx.clone(), persistent=False)
        self.n = int(n)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.zeros((self.n,) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
        return out.index_add_(0, self.idx.long(), x)


def sum(x: torch.Tensor) -> torch.Tensor:  # noqa: A001 - the reference's name
    """Aggregate over the leading (edge) dimension; the result keeps it with length 1.  Under symbolic
    tracing the call is recorded as one node whose target is this function."""
    if isinstance(x, torch.fx.Proxy):
        return x.tracer.create_proxy("call_function", sum, (x,), {})
    return torch.sum(x, dim=0, keepdim=True)


def norm(x: torch.Tensor) -> torch.Tensor:
    """2-norm of every item over all of its trailing dimensions, shape ``[n, 1]``; one node under
    symbolic tracing."""
    if isinstance(x, torch.fx.Proxy):
        return x.tracer.create_proxy("call_function", norm, (x,), {})
    return torch.linalg.vector_norm(x.reshape(x.shape[0], -1), dim=1, keepdim=True)


class Module(nn.Module):
    """Base class of a model: ``forward()`` takes no arguments and updates ``Tensor`` attributes in
    place (easier_spmv.py:58-69)."""

    def forward(self):  # pragma: no cover - abstract
        raise NotImplementedError
