"""CPU restatement of the ZeRO bucket path (TEST INFRASTRUCTURE, see oracle/__init__.py).

Follows src/actor.py:517-601 (flatten, view re-pointing, offsets), src/runtime.py:223-229
(zero), :249-282 (gradient pack), :312-371 (unflatten = views), :454-484 and
src/executors.py:1005-1034 (optimizer step).  AdamW, its hyper-parameters, the fp32 master
bucket and the 256-byte alignment come from the benchmark definition, not from the reference
(which runs torch.optim.Adam on the param-dtype shard with unaligned offsets).

Pinning status (tests/test_oracle_bucket.py):
  plan_offsets     closed form; align=1 reproduces the reference's running numel sum
  pack             bit-exact definition flat[o:o+n] += g.float()
  adamw_step       torch.optim.AdamW (library routine) == closed-form step 1 == float64 evaluation
  unflatten        views alias the bucket; round trip equals the input
"""
from __future__ import annotations

import math

import torch


def plan_offsets(numels, elem_size: int, align_bytes: int = 256):
    """off_0 = 0, off_i = align_up(off_{i-1} + numel_{i-1}); offsets in ELEMENTS, alignment in bytes.
    align_bytes = 1 is the reference rule (src/actor.py:545-554).  Returns (offsets, padded_total)."""
    a = max(1, align_bytes // elem_size)
    offsets, cur = [], 0
    for n in numels:
        cur = (cur + a - 1) // a * a
        offsets.append(cur)
        cur += int(n)
    return offsets, (cur + a - 1) // a * a


def flatten(tensors, offsets, total, dtype):
    """torch.cat flatten with aligned starts (src/actor.py:534 plus padding)."""
    flat = torch.zeros(total, dtype=dtype)
    for t, o in zip(tensors, offsets):
        flat[o:o + t.numel()] = t.reshape(-1).to(dtype)
    return flat


def pack(flat_grads: torch.Tensor, grads, offsets) -> torch.Tensor:
    """flat[o:o+n].add_(grad.reshape(-1).to(flat.dtype)) per tensor (src/runtime.py:275-282)."""
    for g, o in zip(grads, offsets):
        if g is None:
            continue
        flat_grads[o:o + g.numel()].add_(g.detach().reshape(-1).to(flat_grads.dtype))
    return flat_grads


def unflatten(flat: torch.Tensor, shapes, offsets):
    """Views of the bucket (src/runtime.py:337-339)."""
    return [flat[o:o + math.prod(s)].view(s) for s, o in zip(shapes, offsets)]


def adamw_step_torch(master, grad, exp_avg, exp_avg_sq, step, lr, betas, eps, weight_decay):
    """One step of torch.optim.AdamW on fp32 CPU tensors, state injected so any step can be taken."""
    p = master.clone().requires_grad_(True)
    opt = torch.optim.AdamW([p], lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, foreach=False)
    opt.state[p] = {"step": torch.tensor(float(step - 1)), "exp_avg": exp_avg.clone(), "exp_avg_sq": exp_avg_sq.clone()}
    p.grad = grad.clone()
    opt.step()
    st = opt.state[p]
    return p.detach(), st["exp_avg"], st["exp_avg_sq"]


def adamw_step_formula(master, grad, exp_avg, exp_avg_sq, step, lr, betas, eps, weight_decay, dtype=torch.float64):
    """Textbook decoupled-weight-decay Adam, evaluated in `dtype` (float64 for the reference value)."""
    b1, b2 = betas
    p, g, m, v = (t.to(dtype) for t in (master, grad, exp_avg, exp_avg_sq))
    p = p * (1 - lr * weight_decay)
    m = b1 * m + (1 - b1) * g
    v = b2 * v + (1 - b2) * g * g
    mhat = m / (1 - b1 ** step)
    vhat = v / (1 - b2 ** step)
    p = p - lr * mhat / (vhat.sqrt() + eps)
    return p, m, v
