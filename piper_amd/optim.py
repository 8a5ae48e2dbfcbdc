"""Fused AdamW over a flat bucket, satisfying the optimizer-factory contract of the reference's
actor: ``optim_class([shard_param])`` / ``optim_class(params, fused=True)`` returns an object whose
``.step()`` consumes ``p.grad`` (src/actor.py:573,600; src/runtime.py:470-473).

Every parameter handed in is treated as one flat buffer and updated by ONE kernel launch that
reads grad/master/exp_avg/exp_avg_sq and writes master/exp_avg/exp_avg_sq (28 B/element) plus,
for a bf16 parameter, the bf16 value the model reads (+2 B/element).  bf16 parameters get an fp32
master copy; fp32 parameters are their own master.
"""
from __future__ import annotations

import torch

from . import ops


class FusedAdamW(torch.optim.Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2, fused: bool = True, zero_grad_in_step: bool = False):
        if lr < 0 or eps < 0 or not (0 <= betas[0] < 1) or not (0 <= betas[1] < 1) or weight_decay < 0:
            raise ValueError("invalid AdamW hyper-parameters")
        defaults = dict(lr=lr, betas=tuple(betas), eps=eps, weight_decay=weight_decay)
        super().__init__(params, defaults)
        self.zero_grad_in_step = zero_grad_in_step

    def _init_state(self, p: torch.Tensor) -> dict:
        st = self.state[p]
        if not st:
            flat = p.detach().reshape(-1)
            st["step"] = 0
            st["master"] = flat if p.dtype == torch.float32 else flat.float()
            st["exp_avg"] = torch.zeros_like(st["master"])
            st["exp_avg_sq"] = torch.zeros_like(st["master"])
        return st

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            b1, b2 = group["betas"]
            for p in group["params"]:
                if p.grad is None:
                    continue
                if not p.is_contiguous():
                    raise RuntimeError("FusedAdamW needs contiguous parameters (flatten them into a bucket)")
                st = self._init_state(p)
                st["step"] += 1
                grad = p.grad.detach().reshape(-1)
                owns_grad = grad.dtype == torch.float32 and grad.is_contiguous()
                if not owns_grad:
                    grad = grad.float().contiguous()
                shadow = None if p.dtype == torch.float32 else p.detach().reshape(-1)
                ops.adamw_fused(st["master"], st["exp_avg"], st["exp_avg_sq"], grad, step=st["step"],
                                lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"],
                                weight_decay=group["weight_decay"], shadow=shadow,
                                zero_grad=self.zero_grad_in_step and owns_grad)
        return loss

    @torch.no_grad()
    def step_packed(self, p: torch.Tensor, grads, offsets, numels, flat_grad: torch.Tensor | None = None) -> None:
        """One step for the flat parameter `p` (a bucket) whose last gradients have not been packed:
        tensor i of the bucket (elements offsets[i] .. +numels[i]) has the gradient flat_grad[...] (what
        earlier microbatches packed, optional) + grads[i] (optional).  Same result as packing
        grads into flat_grad and calling step() with p.grad = flat_grad, in one launch that
        neither writes nor re-reads the fp32 gradient bucket."""
        group = next(g for g in self.param_groups if any(q is p for q in g["params"]))
        if not p.is_contiguous():
            raise RuntimeError("FusedAdamW needs contiguous parameters (flatten them into a bucket)")
        st = self._init_state(p)
        st["step"] += 1
        b1, b2 = group["betas"]
        shadow = None if p.dtype == torch.float32 else p.detach().reshape(-1)
        ops.adamw_fused_packed(st["master"], st["exp_avg"], st["exp_avg_sq"], flat_grad, list(grads), list(offsets),
                               list(numels), step=st["step"], lr=group["lr"], beta1=b1, beta2=b2, eps=group["eps"],
                               weight_decay=group["weight_decay"], shadow=shadow,
                               zero_grad=self.zero_grad_in_step and flat_grad is not None)
