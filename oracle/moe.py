"""CPU restatement of the MoE expert region (TEST INFRASTRUCTURE, see oracle/__init__.py).

Follows examples/models/qwen3.py:225-289 (AnnotatedMoE.forward) and
examples/models/qwen3_bmm_experts_patch.py:11-50,90-110 (_run_bmm_experts, BmmExperts).
The router and the reorderer live in torchtitan, which is not vendored in the reference and has
no version pin (pyproject.toml:13); their restatement follows the benchmark's wording
("Linear then softmax and top-k with renormalised weights", ties to the lower expert index) and
torchtitan's published TokenChoiceTopKRouter / TokenReorderer algorithm.

Pinning status (tests/test_oracle_*.py):
  gate_logits / softmax        closed form, checked against float64 evaluation
  route_topk selection         brute force on tiny inputs incl. all-equal / pairwise-equal rows
  renormalisation              invariant sum(w) == route_scale
  sort_by_expert               bijection, expert ids non-decreasing, ascending slots per expert,
                               equality with numpy's stable argsort
  grouped_swiglu               equals the reference's literal padded-bmm algorithm
                               (padded_bmm_experts below) and a per-row float64 evaluation
  unpermute_combine            float64 evaluation of sum_k s[t,k] * y[t,k,:]
  backward                     torch.autograd over this forward; gradcheck in float64
  rmsnorm / moe_block          library routine torch.nn.functional.rms_norm (present on CPU) and the
                               closed form x / sqrt(mean(x^2) + eps) * w in float64; gradcheck
  torchtitan op order/dtypes   PARITY UNPINNED: cannot be pinned offline (library absent); this
                               covers the router, the reorderer and the block's ffn_norm module
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def gate_logits(x: torch.Tensor, w_gate: torch.Tensor, gate_bias: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 router gate: Linear(H -> E) on the token rows (router call, qwen3.py:237-241)."""
    logits = x.float() @ w_gate.float().t()
    if gate_bias is not None:
        logits = logits + gate_bias.float()
    return logits


def route_topk(logits: torch.Tensor, top_k: int, route_norm: bool, route_scale: float = 1.0, top_idx=None):
    """softmax over experts (fp32), top-k with ties to the LOWER expert index, optional
    renormalisation of the selected scores (MoEArgs score_func="softmax", route_norm,
    route_scale: qwen3.py:41-44,170-173).

    The selection key is the fp32 logit: softmax is monotone, so this is the order of the scores
    wherever the scores differ, and it does not depend on the exp() implementation.
    torch.topk is NOT used: its tie order on CPU is unspecified (an all-equal row of 4 returns
    [2, 3]); a stable descending sort returns equal keys in ascending index order."""
    logits = logits.float()
    scores = torch.softmax(logits, dim=-1)
    if top_idx is None:
        order = torch.sort(logits, dim=-1, descending=True, stable=True).indices
        top_idx = order[:, :top_k].contiguous()
    else:
        # a selection made elsewhere (a test hands over the device's indices so that a token on a
        # near-tie, which bf16 activations can tip either way, is routed alike on both sides)
        top_idx = top_idx.long()
    top_scores = scores.gather(1, top_idx)
    if route_norm:
        top_scores = top_scores / (top_scores.sum(dim=-1, keepdim=True) + 1e-20)
    top_scores = top_scores * route_scale
    return top_scores, top_idx


def sort_by_expert(top_idx: torch.Tensor, num_experts: int):
    """Reorderer (qwen3.py:243-247): stable argsort of the flattened expert ids.
    Returns counts [E], starts [E+1] (starts[:E] = cumsum(counts) - counts,
    qwen3_bmm_experts_patch.py:27), perm [A] (sorted position -> flat slot t*K+k) and inv_perm."""
    flat = top_idx.reshape(-1).long()
    counts = torch.bincount(flat, minlength=num_experts)
    starts = torch.zeros(num_experts + 1, dtype=torch.long)
    starts[1:] = torch.cumsum(counts, 0)
    perm = torch.argsort(flat, stable=True)
    inv_perm = torch.empty_like(perm)
    inv_perm[perm] = torch.arange(perm.numel())
    return counts, starts, perm, inv_perm


def permute(x: torch.Tensor, perm: torch.Tensor, top_k: int) -> torch.Tensor:
    """routed_input = x[token_indices_experts_sorted // top_k]  (qwen3.py:250)."""
    return x[perm // top_k]


def grouped_swiglu(w1, w2, w3, x_sorted, counts, compute_dtype=None):
    """Un-padded per-expert loop: y[rows_e] = (silu(x w1[e]^T) * (x w3[e]^T)) w2[e]^T on the row
    slice [starts[e], starts[e]+counts[e]).  Same mathematics as _run_bmm_experts
    (qwen3_bmm_experts_patch.py:27-49), whose padded rows contribute exact zeros
    (silu(0) * 0 == 0).  compute_dtype=None keeps x's dtype; torch.float32 gives the
    fp32-accumulate evaluation used to judge bf16 results."""
    dt = compute_dtype or x_sorted.dtype
    x_ = x_sorted.to(dt)
    outs = []
    start = 0
    for e in range(w1.shape[0]):
        n = int(counts[e])
        xe = x_[start:start + n]
        h = F.silu(xe @ w1[e].to(dt).t()) * (xe @ w3[e].to(dt).t())
        outs.append(h @ w2[e].to(dt).t())
        start += n
    return torch.cat(outs, 0) if outs else x_.new_zeros(x_.shape)


def padded_bmm_experts(w1, w2, w3, x, num_tokens_per_expert):
    """The reference's literal algorithm (qwen3_bmm_experts_patch.py:11-50): pad every expert to
    capacity = all routed rows, three dense bmm, scatter_add back.  E-fold memory: small shapes only."""
    dim = x.shape[-1]
    num_experts = w1.shape[0]
    counts = num_tokens_per_expert.long()
    capacity = x.shape[0]
    starts = torch.cumsum(counts, 0) - counts
    positions = torch.arange(capacity)
    zero = x.new_zeros((capacity, dim))
    rows = []
    for e in range(num_experts):
        valid = positions < counts[e]
        safe = torch.where(valid, starts[e] + positions, torch.zeros((), dtype=torch.long))
        rows.append(torch.where(valid[:, None], x[safe], zero))
    packed = torch.stack(rows, 0)
    h = F.silu(torch.bmm(packed, w1.transpose(-2, -1))) * torch.bmm(packed, w3.transpose(-2, -1))
    expert_out = torch.bmm(h, w2.transpose(-2, -1))
    out = x.new_zeros(x.shape)
    for e in range(num_experts):
        valid = positions < counts[e]
        safe = torch.where(valid, starts[e] + positions, torch.zeros((), dtype=torch.long))
        src = torch.where(valid[:, None], expert_out[e], zero)
        out = out.scatter_add(0, safe[:, None].expand(-1, dim), src)
    return out


def unpermute_combine(y_sorted: torch.Tensor, perm: torch.Tensor, top_scores: torch.Tensor, out_dtype=None):
    """Scatter back to (token, k) order and weight in fp32 (qwen3.py:265-283):
    out[t] = sum_k top_scores[t,k] * y[t,k,:], accumulated in fp32, cast to the activation dtype."""
    T, K = top_scores.shape
    H = y_sorted.shape[1]
    unsorted = torch.zeros((T * K, H), dtype=y_sorted.dtype)
    unsorted = unsorted.index_put((perm,), y_sorted)
    unsorted = unsorted.reshape(T, K, H)
    acc = torch.float64 if y_sorted.dtype == torch.float64 else torch.float32  # fp32 in the reference
    out = torch.bmm(top_scores.reshape(T, 1, K).to(acc), unsorted.to(acc)).squeeze(1)
    return out.to(out_dtype or y_sorted.dtype)


def moe_forward(x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale=1.0, compute_dtype=None, top_idx=None):
    """AnnotatedMoE.forward on x [T,H] (qwen3.py:233-289).  Returns (out, aux) where aux holds the
    routing tables.  Differentiable w.r.t. x, w_gate, gate_bias, w1, w2, w3."""
    E = w1.shape[0]
    logits = gate_logits(x, w_gate, gate_bias)
    top_scores, top_idx = route_topk(logits, top_k, route_norm, route_scale, top_idx=top_idx)
    counts, starts, perm, inv_perm = sort_by_expert(top_idx, E)
    routed = permute(x, perm, top_k)
    y = grouped_swiglu(w1, w2, w3, routed, counts, compute_dtype=compute_dtype)
    out = unpermute_combine(y, perm, top_scores, out_dtype=compute_dtype or x.dtype)
    aux = dict(logits=logits, top_scores=top_scores, top_idx=top_idx, counts=counts, starts=starts,
               perm=perm, inv_perm=inv_perm, y_sorted=y)
    return out, aux


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """The block's ffn_norm (qwen3.py:313-314; built by torchtitan as RMSNorm(dim, eps=norm_eps),
    qwen3.py:28): x * rsqrt(mean(x^2) + eps) * weight over the last dimension, evaluated in the
    dtype of x (float32 / float64 in the tests)."""
    ms = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * weight


def moe_block(h, norm_weight, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale=1.0, norm_eps=1e-6,
              compute_dtype=None, top_idx=None):
    """h + moe(ffn_norm(h)) (qwen3.py:313-314) on h [T,H]."""
    out, aux = moe_forward(rmsnorm(h, norm_weight, norm_eps), w_gate, gate_bias, w1, w2, w3, top_k, route_norm,
                           route_scale, compute_dtype=compute_dtype, top_idx=top_idx)
    return h + out, aux
