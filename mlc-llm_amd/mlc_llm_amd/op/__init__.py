"""Mirrors of python/mlc_llm/op/{moe_matmul,moe_misc}.py of the reference."""
from . import moe_matmul, moe_misc  # noqa: F401
