"""RMSNorm in front of the region and the residual added in the combine kernel (qwen3.py:313-314),
through the C ABI, against the CPU oracle."""
import pytest
import torch

from conftest import BF16_TOL, F32_TOL, rel_err
from oracle import moe as O
from piper_amd import functional as F_
from piper_amd import ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H", [(1, 8), (5, 24), (33, 256), (64, 2048), (3, 4100), (2, 8192)])
def test_rmsnorm_fwd_bwd(dev, dtype, T, H):
    print(f"[case] rmsnorm {dtype} T={T} H={H}", flush=True)
    g = torch.Generator().manual_seed(T * 131 + H)
    x = torch.randn(T, H, generator=g).to(dtype)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    dy = torch.randn(T, H, generator=g).to(dtype)
    add = torch.randn(T, H, generator=g).to(dtype)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    ref = O.rmsnorm(xr, wr, 1e-6)
    ref.backward(dy.double())
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    y, rstd = ops.rmsnorm_fwd(x.to(dev), w.to(dev), 1e-6)
    assert y.dtype == dtype and rel_err(y, ref.detach()) <= tol
    ms = x.double().pow(2).mean(-1)
    assert rel_err(rstd, torch.rsqrt(ms + 1e-6)) <= 1e-5
    dx, dw = ops.rmsnorm_bwd(dy.to(dev), x.to(dev), w.to(dev), rstd)
    assert rel_err(dx, xr.grad) <= tol and rel_err(dw, wr.grad) <= tol
    # addend fused into d_x; accumulate into an existing d_weight; d_weight optional
    dx2, dw2 = ops.rmsnorm_bwd(dy.to(dev), x.to(dev), w.to(dev), rstd, d_x_addend=add.to(dev), d_weight=dw.clone(), accumulate=True)
    assert rel_err(dx2, xr.grad + add.double()) <= tol and rel_err(dw2, 2 * wr.grad) <= tol
    dx3, none = ops.rmsnorm_bwd(dy.to(dev), x.to(dev), w.to(dev), rstd, need_dw=False)
    assert none is None and torch.equal(dx3, dx)


def test_rmsnorm_is_deterministic_and_rejects_bad_arguments(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(700, 512, generator=g).bfloat16().to(dev)
    w = torch.ones(512).bfloat16().to(dev)
    dy = torch.randn(700, 512, generator=g).bfloat16().to(dev)
    y, rstd = ops.rmsnorm_fwd(x, w, 1e-6)
    a = ops.rmsnorm_bwd(dy, x, w, rstd)
    b = ops.rmsnorm_bwd(dy, x, w, rstd)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])      # fixed-order column sums
    with pytest.raises(ValueError):
        ops.rmsnorm_fwd(x, torch.ones(511).bfloat16().to(dev), 1e-6)
    with pytest.raises(ValueError):
        ops.rmsnorm_fwd(x, w.float(), 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_moe_block_matches_oracle(dev, dtype):
    """h + moe(ffn_norm(h)) forward and backward; the residual rides in the combine kernel."""
    print(f"[case] moe_block {dtype}", flush=True)
    T, H, I, E, K = 96, 256, 128, 8, 2
    g = torch.Generator().manual_seed(11)
    h = torch.randn(T, H, generator=g).to(dtype)
    nw = (1.0 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    wg = torch.randn(E, H, generator=g) * 0.02
    w1 = (torch.randn(E, I, H, generator=g) * 0.02).to(dtype)
    w3 = (torch.randn(E, I, H, generator=g) * 0.02).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).to(dtype)
    d_out = torch.randn(T, H, generator=g).to(dtype)
    leaves_cpu = [t.clone().float().requires_grad_(True) for t in (h, nw, wg, w1, w2, w3)]
    ref, aux = O.moe_block(leaves_cpu[0], leaves_cpu[1], leaves_cpu[2], None, leaves_cpu[3], leaves_cpu[4], leaves_cpu[5],
                           K, True, compute_dtype=torch.float32)
    ref.backward(d_out.float())
    leaves = [t.to(dev).requires_grad_(True) for t in (h, nw, wg, w1, w2, w3)]
    out = F_.moe_block(leaves[0], leaves[1], leaves[2], None, leaves[3], leaves[4], leaves[5], top_k=K, route_norm=True)
    out.backward(d_out.to(dev))
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    gtol = 1e-4 if dtype == torch.float32 else 4 * BF16_TOL
    assert out.dtype == dtype and rel_err(out, ref.detach()) <= tol
    for got, want, name in zip(leaves, leaves_cpu, ("h", "norm_weight", "w_gate", "w1", "w2", "w3")):
        assert got.grad is not None and rel_err(got.grad, want.grad) <= gtol, name
    # the fused residual equals a separate add of the region's output
    xn = F_.rmsnorm(leaves[0].detach(), leaves[1].detach())
    region = F_.expert_region(xn, leaves[2].detach(), None, leaves[3].detach(), leaves[4].detach(), leaves[5].detach(),
                              top_k=K, route_norm=True)
    assert torch.equal(out.detach(), leaves[0].detach() + region)


def test_feed_forward_block_module(dev):
    """MoEFeedForwardBlock == x + moe(ffn_norm(x)) built from the separate modules."""
    from piper_amd.moe import MoEArgs, MoEFeedForwardBlock
    args = MoEArgs(num_experts=8, top_k=2, route_norm=True)
    blk = MoEFeedForwardBlock(args, dim=128, hidden_dim=128, dtype=torch.bfloat16).to(dev)
    blk.moe.router.gate.weight.data = blk.moe.router.gate.weight.data.float()
    g = torch.Generator().manual_seed(4)
    blk.moe.init_weights(generator=None)
    x = torch.randn(2, 40, 128, generator=g).bfloat16().to(dev)
    got = blk(x)
    want = x + blk.moe(blk.ffn_norm(x))
    assert got.shape == x.shape and torch.equal(got, want)
    assert sorted(n for n, _ in blk.named_parameters()) == [
        "ffn_norm.weight", "moe.experts.w1", "moe.experts.w2", "moe.experts.w3", "moe.router.gate.weight"]
