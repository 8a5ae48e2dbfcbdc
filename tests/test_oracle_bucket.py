"""Pins the CPU oracle of the bucket path: closed forms, library routine, float64 evaluation."""
import math

import pytest
import torch

from oracle import bucket as OB
from piper_amd.configs import ADAMW, bucket_manifest_cfg2, manifest_numel


def test_plan_offsets_closed_form_and_reference_rule():
    numels = [5, 128, 1, 300, 0, 7]
    # align 1 byte == the reference's running numel sum (src/actor.py:545-554)
    offs, total = OB.plan_offsets(numels, 2, 1)
    assert offs == [0, 5, 133, 134, 434, 434] and total == 441
    # 256-byte alignment with 2-byte elements == 128-element alignment
    offs, total = OB.plan_offsets(numels, 2, 256)
    assert offs == [0, 128, 256, 384, 768, 768] and total == 896
    for o in offs:
        assert (o * 2) % 256 == 0
    # brute force: smallest aligned offset not overlapping the previous tensor
    a = 256 // 4
    offs4, _ = OB.plan_offsets(numels, 4, 256)
    end = 0
    for n, o in zip(numels, offs4):
        assert o % a == 0 and o >= end and o - end < a
        end = o + n


def test_cfg2_manifest():
    m = bucket_manifest_cfg2()
    assert len(m) == 96
    assert manifest_numel(m) == 2 * (2 * 4096 * 2048 + 2 * 512 * 2048 + 2 * 2048 + 14 * 3 * 768 * 2048)
    offs, total = OB.plan_offsets([math.prod(s) for _, s in m], 2, 256)
    assert all((o * 2) % 256 == 0 for o in offs) and total >= manifest_numel(m)


def test_pack_is_exact_and_accumulates():
    g = torch.Generator().manual_seed(0)
    shapes = [(3, 5), (7,), (2, 2, 2)]
    grads = [torch.randn(s, generator=g).bfloat16() for s in shapes]
    offs, total = OB.plan_offsets([t.numel() for t in grads], 2, 256)
    flat = torch.zeros(total)
    OB.pack(flat, grads, offs)
    OB.pack(flat, [grads[0], None, grads[2]], offs)
    for i, (t, o) in enumerate(zip(grads, offs)):
        mult = 1.0 if i == 1 else 2.0
        assert torch.equal(flat[o:o + t.numel()], t.float().reshape(-1) * mult)
    views = OB.unflatten(flat, shapes, offs)
    assert all(v.data_ptr() == flat.data_ptr() + 4 * o for v, o in zip(views, offs))


def test_adamw_torch_equals_closed_form_step1_and_float64_multistep():
    g = torch.Generator().manual_seed(1)
    n = 1000
    p0 = torch.randn(n, generator=g) * 0.02
    lr, (b1, b2), eps, wd = ADAMW["lr"], ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"]
    grad = torch.randn(n, generator=g) * 1e-3
    z = torch.zeros(n)
    p1, m1, v1 = OB.adamw_step_torch(p0, grad, z, z, 1, lr, (b1, b2), eps, wd)
    # step 1 closed form: m/(1-b1) = g, sqrt(v/(1-b2)) = |g|
    closed = p0.double() * (1 - lr * wd) - lr * grad.double() / (grad.double().abs() + eps)
    assert torch.allclose(p1.double(), closed, rtol=0, atol=1e-8)
    # several steps against the float64 textbook recurrence
    p, m, v = p0, z, z
    p64, m64, v64 = p0.double(), z.double(), z.double()
    for step in range(1, 6):
        gk = torch.randn(n, generator=g) * 1e-3
        p, m, v = OB.adamw_step_torch(p, gk, m, v, step, lr, (b1, b2), eps, wd)
        p64, m64, v64 = OB.adamw_step_formula(p64, gk, m64, v64, step, lr, (b1, b2), eps, wd)
    assert torch.allclose(p.double(), p64, rtol=0, atol=1e-7)
    assert torch.allclose(m.double(), m64, rtol=1e-5, atol=1e-10)
    assert torch.allclose(v.double(), v64, rtol=1e-5, atol=1e-12)
