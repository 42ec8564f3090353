"""FlexSpmv for MI355X: the fused merge-path SpMV / map + reducer + aggregator path as generated
HIP (gfx950) libraries behind the reference's ``merged_spmv_launch`` call surface."""
from .ir import FusedGraphIR, GraphBuilder  # noqa: F401

__all__ = ["FusedGraphIR", "GraphBuilder"]
