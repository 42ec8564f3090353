"""Modelling front end on plain ``torch``: the few EASIER names the reference's models use, and a
``compile`` that fuses a traced model into select -> map -> reduce / aggregate sub-modules."""
from .fusion import CompiledModule, compile, compile_module, init  # noqa: F401,A004
from .lite import Module, Reducer, Selector, Tensor, norm, sum, zeros  # noqa: F401,A004

__all__ = ["CompiledModule", "Module", "Reducer", "Selector", "Tensor", "compile", "compile_module", "init",
           "norm", "sum", "zeros"]
