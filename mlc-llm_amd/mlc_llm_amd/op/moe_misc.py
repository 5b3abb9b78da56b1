"""MoE routing operators (mirror of python/mlc_llm/op/moe_misc.py of the reference)."""

from __future__ import annotations

from typing import Tuple

import torch

from .. import ops


def moe_sum(x: torch.Tensor, dim: int) -> torch.Tensor:
    """:14-32.  x [T, k, H] -> [T, H]; fp16 adds left to right."""
    assert dim == 1 and x.dim() == 3
    if x.shape[1] == 1:
        return x.reshape(x.shape[0], x.shape[2])
    ones = torch.ones((x.shape[0], x.shape[1]), dtype=torch.float16, device=x.device)
    return ops.moe_combine(x.contiguous(), ones)


def gating_softmax_topk(x: torch.Tensor, k: int, norm_topk_prob: bool = True
                        ) -> Tuple[torch.Tensor, torch.Tensor]:
    """:135-235.  Returns (expert_weights [T, k] in x's dtype, expert_indices int32 [T, k]).
    norm_topk_prob=False is the branch of :234-235 (softmax over all experts, cast, then gating_topk)."""
    return ops.gating_softmax_topk(x, k, norm_topk_prob)


def gating_topk(scores: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """:63-132.  Returns (the k largest scores as they are [T, k], their expert indices int32 [T, k])."""
    return ops.gating_topk(scores, k)


def moe_cumsum(expert_indices: torch.Tensor, num_local_experts: int) -> torch.Tensor:
    """:371-450."""
    return ops.moe_cumsum(expert_indices, num_local_experts)


def get_indices(cumsum: torch.Tensor, expert_indices: torch.Tensor
                ) -> Tuple[torch.Tensor, torch.Tensor]:
    """:453-525.  Returns (reverse_indices, token_indices)."""
    return ops.get_indices(cumsum, expert_indices)


def get_indptr(cumsum: torch.Tensor, num_local_experts: int, batch_size: int, inclusive: bool,
               out_dtype: str) -> torch.Tensor:
    """:528-605."""
    return ops.get_indptr(cumsum, num_local_experts, batch_size, inclusive,
                          torch.int64 if out_dtype == "int64" else torch.int32)


def scatter_output(x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """:608-645."""
    return ops.scatter_output(x, indices)
