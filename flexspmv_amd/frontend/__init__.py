"""Modelling front end on plain ``torch``: the few EASIER names the reference's models use, and a
``compile`` that fuses a traced model into select -> map -> reduce / aggregate sub-modules."""
from .data_files import datasets, hdf5, save_arrays  # noqa: F401
from .fusion import CompiledModule, compile, compile_module, init  # noqa: F401,A004
from .lite import Module, Reducer, Selector, Tensor, norm, sum, zeros  # noqa: F401,A004

__all__ = ["CompiledModule", "Module", "Reducer", "Selector", "Tensor", "compile", "compile_module", "datasets",
           "hdf5", "init", "norm", "save_arrays", "sum", "zeros"]
