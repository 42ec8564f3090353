"""Shape helper shared by the generators (codegen/utils.py:5-12 of the reference)."""
from ..ir import get_dim_length  # noqa: F401
