"""MixtralMoE.forward over group-quantized experts.

Mirror of python/mlc_llm/model/mixtral/mixtral_model.py:32-117 of the reference, with the
router logits supplied by the caller (the router `gate` is an unquantized nn.Linear there,
quantization/utils.py:57-59, and is outside this path).
"""

from __future__ import annotations

import torch
from torch import nn

from .. import _lib, ops
from ..op import moe_misc
from ..quantization import GroupQuantize, GroupQuantizeMixtralExperts


class MixtralMoE(nn.Module):
    """Mixture of experts with group-quantized e1_e3 / e2 expert stacks."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_local_experts: int,
                 num_experts_per_tok: int, config: GroupQuantize, device=None):
        super().__init__()
        self.num_experts_per_tok = num_experts_per_tok
        self.num_local_experts = num_local_experts
        self.intermediate_size = intermediate_size
        self.e1_e3 = GroupQuantizeMixtralExperts(num_local_experts, hidden_size,
                                                 2 * intermediate_size, config, device=device)
        self.e2 = GroupQuantizeMixtralExperts(num_local_experts, intermediate_size, hidden_size,
                                              config, device=device)
        # Which fused forms the library has for this module is a property of its dtype, expert count, top-k and
        # shapes: each is tried until the library first answers "unsupported", then never again (a failing call
        # formats a message and raises on every forward otherwise).
        self._fused = {"route": True, "routed_gemv": True, "gemv_combine": True}

    def _try(self, name, fn, *args, **kwargs):
        """fn(*args) if the fused form `name` is (still) believed to exist, else None; a first ERR_UNSUPPORTED
        switches the form off for this module."""
        if not self._fused[name]:
            return None
        try:
            return fn(*args, **kwargs)
        except _lib.Mi355gqError as err:
            if err.code != _lib.ERR_UNSUPPORTED:
                raise
            self._fused[name] = False
            return None

    def _route_fits(self, num_tokens: int) -> bool:
        """The batch sizes mi355gq_moe_route scans in one workgroup (it answers "unsupported" beyond them, which says
        nothing about smaller batches, so that answer is not remembered)."""
        slots, experts = num_tokens * self.num_experts_per_tok, self.num_local_experts
        if slots <= 8192 and experts * -(-slots // 64) <= 8192:
            return True
        return experts <= 64 and num_tokens <= 8192 and experts * -(-num_tokens // 1024) <= 64

    def _expert_forward(self, x: torch.Tensor, indptr: torch.Tensor) -> torch.Tensor:
        # x1, x3 = split(e1_e3(x)); e2(silu(x1) * x3): the activation rides in the e1_e3 kernel
        return self.e2(self.e1_e3(x, indptr, silu_mul_halves=True), indptr)

    def forward(self, x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """x [batch, seq, hidden]; gate [batch * seq, num_local_experts] router logits, both in the model dtype."""
        experts_per_tok = self.num_experts_per_tok
        local_experts = self.num_local_experts
        batch_size, seq_len, hidden_size = x.shape
        num_tokens = batch_size * seq_len
        x = x.reshape(num_tokens, hidden_size).contiguous()
        if num_tokens > 1:
            # routing in one launch; the gather rides in e1_e3's row addressing, the scatter in the
            # combine's: four launches where the op-by-op sequence below takes nine
            routed = self._try("route", ops.moe_route, gate, experts_per_tok) if self._route_fits(num_tokens) else None
            if routed is not None:
                weights, _, token_indices, _, slot_positions, indptr = routed
                cfg = self.e1_e3.config
                if num_tokens * experts_per_tok > 128:
                    # the GEMM's workgroups would each start with one more dependent load (index, then
                    # rows): measured slower than a separate gather once the few-row kernels are left
                    x, token_indices = ops.take_rows(x, token_indices), None
                h = ops.moe_experts(x, token_indices, self.e1_e3.q_weight, self.e1_e3.q_scale, indptr, cfg.bits,
                                    self.e1_e3.group_size, silu_mul_halves=True)
                y = self.e2(h, indptr)
                return ops.moe_combine_sorted(y, slot_positions, weights).reshape(batch_size, seq_len, hidden_size)
        if num_tokens == 1:
            # the token routes itself inside the e1_e3 kernel: one launch where the two operators take two
            cfg = self.e1_e3.config
            first = self._try("routed_gemv", ops.moe_gemv_routed_silu_mul, x, gate, experts_per_tok, self.e1_e3.q_weight,
                              self.e1_e3.q_scale, cfg.bits, self.e1_e3.group_size)
            if first is not None:
                h, expert_weights, expert_indices = first
                # e2 and the weighted sum over the experts in one launch as well
                cfg2 = self.e2.config
                out = self._try("gemv_combine", ops.moe_gemv_combine, h, self.e2.q_weight, self.e2.q_scale, expert_indices,
                                expert_weights, cfg2.bits, self.e2.group_size)
                if out is None:
                    out = self.e2(h, expert_indices)
                    out = ops.moe_combine(out.reshape(1, experts_per_tok, hidden_size), expert_weights)
                return out.reshape(batch_size, seq_len, hidden_size)
        expert_weights, expert_indices = moe_misc.gating_softmax_topk(gate, experts_per_tok)
        if num_tokens == 1:
            x = self._expert_forward(x, expert_indices)
        else:
            cumsum = moe_misc.moe_cumsum(expert_indices, local_experts)
            reverse_indices, token_indices = moe_misc.get_indices(cumsum, expert_indices)
            indptr = moe_misc.get_indptr(cumsum, local_experts, num_tokens, inclusive=False,
                                         out_dtype="int32")
            x = ops.take_rows(x, token_indices)
            x = self._expert_forward(x, indptr)
            x = moe_misc.scatter_output(x, reverse_indices)
        x = ops.moe_combine(x.reshape(num_tokens, experts_per_tok, hidden_size), expert_weights)
        return x.reshape(batch_size, seq_len, hidden_size)
