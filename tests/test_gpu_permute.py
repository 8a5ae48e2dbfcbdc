"""GPU parity of permute / unpermute+combine (forward and backward) against the CPU oracle."""
import pytest
import torch

from conftest import BF16_TOL, F32_TOL, rel_err
from oracle import moe as O
from piper_amd import ops

pytestmark = pytest.mark.gpu


def _routing(T, E, K, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    scores, idx = O.route_topk(logits, K, True)
    counts, starts, perm, inv = O.sort_by_expert(idx, E)
    return g, scores, idx, counts, starts, perm, inv


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,E,K", [(256, 256, 8, 2), (512, 2048, 128, 8), (33, 250, 8, 3), (5, 7, 4, 2)])
def test_permute_forward_backward(dev, dtype, T, H, E, K):
    print(f"[case] permute {dtype} T={T} H={H} E={E} K={K}", flush=True)
    g, scores, idx, counts, starts, perm, inv = _routing(T, E, K, 1)
    x = torch.randn(T, H, generator=g).to(dtype)
    routed = ops.permute_fwd(x.to(dev), perm.int().to(dev), K)
    assert torch.equal(routed.cpu(), O.permute(x, perm, K)), "permute is a pure copy: bit-exact"
    d_routed = torch.randn(T * K, H, generator=g).to(dtype)
    # oracle backward of x[perm // K]: index_add in fp32
    ref = torch.zeros(T, H).index_add_(0, perm // K, d_routed.float())
    addend = torch.randn(T, H, generator=g)
    got = ops.permute_bwd(d_routed.to(dev), inv.int().to(dev), K)
    got_add = ops.permute_bwd(d_routed.to(dev), inv.int().to(dev), K, addend_f32=addend.to(dev))
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    assert rel_err(got, ref) <= tol
    assert rel_err(got_add, ref + addend) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,E,K", [(256, 256, 8, 2), (512, 2048, 128, 8), (33, 250, 8, 3)])
def test_combine_forward_backward(dev, dtype, T, H, E, K):
    print(f"[case] combine {dtype} T={T} H={H} E={E} K={K}", flush=True)
    g, scores, idx, counts, starts, perm, inv = _routing(T, E, K, 2)
    y = torch.randn(T * K, H, generator=g).to(dtype)
    d_out = torch.randn(T, H, generator=g).to(dtype)
    yr = y.clone().float().requires_grad_(True)
    sr = scores.clone().requires_grad_(True)
    ref = O.unpermute_combine(yr, perm, sr, out_dtype=torch.float32)
    dy_ref, ds_ref = torch.autograd.grad(ref, (yr, sr), d_out.float())
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    out = ops.combine_fwd(y.to(dev), inv.int().to(dev), scores.to(dev))
    assert out.dtype == dtype and rel_err(out, ref) <= tol
    d_y, d_s = ops.combine_bwd(d_out.to(dev), y.to(dev), perm.int().to(dev), scores.to(dev))
    assert rel_err(d_y, dy_ref) <= tol
    assert rel_err(d_s, ds_ref) <= (F32_TOL if dtype == torch.float32 else 1e-4)
