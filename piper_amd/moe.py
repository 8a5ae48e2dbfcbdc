"""Module-level mirror of the reference's MoE layer (examples/models/qwen3.py:225-289 and
examples/models/qwen3_bmm_experts_patch.py:90-110), backed by the HIP kernels.

Parameter names and shapes follow the reference (``router.gate.weight`` [E,H],
``experts.w1/w3`` [E,I,H], ``experts.w2`` [E,H,I]) so a state dict moves across unchanged.
The router gate is kept in float32 (the "fp32 router" of the benchmark configuration).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import nn

from . import functional as F_
from .annotate import EP_TAG, annotate


@dataclass
class MoEArgs:
    """The fields of torchtitan's MoEArgs that the reference sets (qwen3.py:36-50,167-176)."""

    num_experts: int = 8
    top_k: int = 2
    score_func: str = "softmax"
    route_norm: bool = False
    route_scale: float = 1.0
    gate_bias: bool = False
    score_before_experts: bool = False
    num_shared_experts: int = 0
    load_balance_coeff: float | None = None


class TokenChoiceTopKRouter(nn.Module):
    """``self.router(x, expert_bias)`` -> (top_scores, selected_experts_indices, num_tokens_per_expert)."""

    def __init__(self, dim: int, num_experts: int, top_k: int, route_norm: bool, route_scale: float, gate_bias: bool):
        super().__init__()
        self.gate = nn.Linear(dim, num_experts, bias=gate_bias, dtype=torch.float32)
        self.num_experts, self.top_k = num_experts, top_k
        self.route_norm, self.route_scale = route_norm, route_scale

    def forward(self, x: torch.Tensor, expert_bias: torch.Tensor | None = None):
        if expert_bias is not None:
            raise NotImplementedError(
                "selection-only expert_bias (load_balance_coeff) is not part of the reference configurations "
                "(qwen3.py:48,175 set load_balance_coeff=None); use gate_bias for a logit bias"
            )
        return F_.router(x, self.gate.weight, self.gate.bias, top_k=self.top_k,
                         route_norm=self.route_norm, route_scale=self.route_scale)


class TokenReorderer(nn.Module):
    """``self.reorderer(top_scores, selected_experts_indices)``."""

    def __init__(self, num_experts: int, top_k: int):
        super().__init__()
        self.num_experts, self.top_k = num_experts, top_k

    def forward(self, top_scores, selected_experts_indices):
        return F_.reorder(top_scores, selected_experts_indices, self.num_experts)


class BmmExperts(nn.Module):
    """Same parameters and call as the reference BmmExperts (qwen3_bmm_experts_patch.py:90-110);
    the input must be sorted by expert and ``num_tokens_per_expert`` gives each expert's row count."""

    def __init__(self, dim: int, hidden_dim: int, num_experts: int, dtype: torch.dtype | None = None):
        super().__init__()
        self.num_experts = num_experts
        self.w1 = nn.Parameter(torch.empty(num_experts, hidden_dim, dim, dtype=dtype))
        self.w2 = nn.Parameter(torch.empty(num_experts, dim, hidden_dim, dtype=dtype))
        self.w3 = nn.Parameter(torch.empty(num_experts, hidden_dim, dim, dtype=dtype))

    def forward(self, x: torch.Tensor, num_tokens_per_expert: torch.Tensor) -> torch.Tensor:
        return F_.bmm_experts(self.w1, self.w2, self.w3, x, num_tokens_per_expert)


class AnnotatedMoE(nn.Module):
    """The MoE block of the reference model.  ``fused=True`` (default) runs the whole region as one
    autograd node; ``fused=False`` follows the reference's op-by-op data flow (router, reorderer,
    gather, EP-annotated experts, scatter+combine) through the piecewise HIP operators."""

    def __init__(self, moe_args: MoEArgs, dim: int, hidden_dim: int, dtype: torch.dtype | None = None, fused: bool = True):
        super().__init__()
        if moe_args.score_func != "softmax":
            raise NotImplementedError("only score_func='softmax' is used by the reference configurations")
        if moe_args.score_before_experts:
            raise NotImplementedError("score_before_experts=True is not used by the reference configurations")
        if moe_args.num_shared_experts:
            raise NotImplementedError("shared experts are not used by the reference configurations")
        self.router = TokenChoiceTopKRouter(dim, moe_args.num_experts, moe_args.top_k, moe_args.route_norm,
                                            moe_args.route_scale, moe_args.gate_bias)
        self.reorderer = TokenReorderer(moe_args.num_experts, moe_args.top_k)
        self.experts = BmmExperts(dim, hidden_dim, moe_args.num_experts, dtype=dtype)
        self.expert_bias = None
        self.shared_experts = None
        self.score_before_experts = False
        self.fused = fused

    def init_weights(self, std: float = 0.02, generator: torch.Generator | None = None) -> None:
        for p in (self.router.gate.weight, self.experts.w1, self.experts.w3, self.experts.w2):
            nn.init.normal_(p, mean=0.0, std=std, generator=generator)
        if self.router.gate.bias is not None:
            nn.init.zeros_(self.router.gate.bias)

    def forward(self, x: torch.Tensor, residual: torch.Tensor | None = None) -> torch.Tensor:
        """``residual`` (same shape as x; fused path only) is added in the combine kernel."""
        bs, slen, dim = x.shape
        x2 = x.reshape(-1, dim)
        top_k = self.router.top_k
        if self.fused:
            with annotate(EP_TAG):
                out = F_.expert_region(x2, self.router.gate.weight, self.router.gate.bias, self.experts.w1,
                                       self.experts.w2, self.experts.w3, top_k=top_k,
                                       route_norm=self.router.route_norm, route_scale=self.router.route_scale,
                                       residual=None if residual is None else residual.reshape(-1, dim))
            return out.reshape(bs, slen, dim)
        if residual is not None:
            return residual + self.forward(x)

        top_scores, selected_experts_indices, num_tokens_per_expert = self.router(x2, self.expert_bias)
        _scores_sorted, token_indices_experts_sorted, num_tokens_per_expert = self.reorderer(
            top_scores, selected_experts_indices)
        routed_input = F_.permute(x2, token_indices_experts_sorted, top_k)
        with annotate(EP_TAG):
            gathered_output = self.experts(routed_input, num_tokens_per_expert)
        out_experts = F_.combine(gathered_output.reshape(-1, dim), token_indices_experts_sorted, top_scores)
        return out_experts.reshape(bs, slen, dim)


class RMSNorm(nn.Module):
    """The norm module torchtitan's TransformerBlock builds as ``ffn_norm`` (RMSNorm(dim, eps))."""

    def __init__(self, dim: int, eps: float = 1e-6, dtype: torch.dtype | None = None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F_.rmsnorm(x, self.weight, self.eps)


class MoEFeedForwardBlock(nn.Module):
    """The MoE half of AnnotatedQwen3TransformerBlock.forward (qwen3.py:313-314):
    ``x = x + self.moe(self.ffn_norm(x))`` with the parameter names of the reference block
    (``ffn_norm.weight``, ``moe.router.gate.weight``, ``moe.experts.w1/w2/w3``)."""

    def __init__(self, moe_args: MoEArgs, dim: int, hidden_dim: int, norm_eps: float = 1e-6,
                 dtype: torch.dtype | None = None):
        super().__init__()
        self.ffn_norm = RMSNorm(dim, norm_eps, dtype=dtype)
        self.moe = AnnotatedMoE(moe_args, dim, hidden_dim, dtype=dtype, fused=True)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.moe(self.ffn_norm(x), residual=x)
