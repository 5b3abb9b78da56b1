"""MoE matmuls on group-quantized experts (mirror of python/mlc_llm/op/moe_matmul.py).

Only the two dequantizing operators the quantized Mixtral path uses are provided:
dequantize_gemv (:77-176) and dequantize_group_gemm (:562-768).
"""

from __future__ import annotations

import torch

from .. import ops

_BITS = {"int3": 3, "int4": 4}


def dequantize_gemv(x: torch.Tensor, w: torch.Tensor, scale: torch.Tensor, indptr: torch.Tensor,
                    quantize_dtype: str, group_size: int) -> torch.Tensor:
    """x [1|k, K], w [Ne, N, nw], scale [Ne, N, ng], indptr int32 [1, k] (expert ids) -> [k, N]."""
    (x_leading_dim, _) = x.shape
    _, experts_per_tok = indptr.shape
    assert indptr.shape == (1, experts_per_tok) and indptr.dtype == torch.int32
    assert x_leading_dim in [1, experts_per_tok]
    return ops.moe_gemv(x, w, scale, indptr, _BITS[quantize_dtype], group_size)


def dequantize_group_gemm(x: torch.Tensor, w: torch.Tensor, scale: torch.Tensor,
                          indptr: torch.Tensor, quantize_dtype: str, indptr_dtype: str,
                          group_size: int) -> torch.Tensor:
    """x [rows, K] in expert order, indptr [Ne + 1] -> [rows, N].

    With indptr_dtype "int64" the reference receives the inclusive form [Ne] and pads a
    leading zero itself (:629-630); the same is done here.
    """
    if indptr_dtype == "int64" and indptr.shape[0] == w.shape[0]:
        indptr = torch.cat([torch.zeros(1, dtype=indptr.dtype, device=indptr.device), indptr])
    return ops.moe_group_gemm(x, w, scale, indptr.contiguous(), _BITS[quantize_dtype], group_size)
