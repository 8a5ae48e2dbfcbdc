"""GPU parity of the ZeRO bucket path: offsets and packing bit-exact, AdamW master weights to 1e-6."""
import math

import pytest
import torch

from conftest import ADAMW_TOL, rel_err
from oracle import bucket as OB
from piper_amd import ops
from piper_amd.bucket import BucketState, ParamStorage, StageStore, flatten_params
from piper_amd.configs import ADAMW, bucket_manifest_cfg2
from piper_amd.optim import FusedAdamW

pytestmark = pytest.mark.gpu


def _tensors(seed, shapes, dtype, scale=1e-3):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(s, generator=g) * scale).to(dtype) for s in shapes]


@pytest.mark.parametrize("src_dtype,flat_dtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                                  (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("align", [256, 1])
def test_pack_accumulate_unpack_bit_exact(dev, src_dtype, flat_dtype, align):
    print(f"[case] pack {src_dtype}->{flat_dtype} align={align}", flush=True)
    shapes = [(3, 5), (8192,), (1,), (777, 13), (2, 8200), (64, 64)]
    grads = _tensors(0, shapes, src_dtype)
    esize = 2 if src_dtype == torch.bfloat16 else 4
    offs, total = ops.bucket_plan([t.numel() for t in grads], esize, align)
    assert (offs, total) == OB.plan_offsets([t.numel() for t in grads], esize, align)
    flat = torch.zeros(total, dtype=flat_dtype, device=dev)
    ref = torch.zeros(total, dtype=flat_dtype)
    dgr = [t.to(dev) for t in grads]
    ops.bucket_pack(dgr, offs, flat, accumulate=True)
    OB.pack(ref, grads, offs)
    assert torch.equal(flat.cpu(), ref)
    # second microbatch with a missing gradient
    dgr2 = [dgr[0], None, dgr[2], dgr[3], None, dgr[5]]
    ops.bucket_pack(dgr2, offs, flat, accumulate=True)
    OB.pack(ref, [grads[0], None, grads[2], grads[3], None, grads[5]], offs)
    assert torch.equal(flat.cpu(), ref), "pack must be bit-exact"
    # overwrite mode + unpack round trip
    ops.bucket_pack(dgr, offs, flat, accumulate=False)
    outs = [torch.empty_like(t) for t in dgr]
    ops.bucket_unpack(flat, outs, offs)
    for o, t in zip(outs, grads):
        assert torch.equal(o.cpu(), t.to(flat_dtype).to(src_dtype))


def test_pack_many_tensors_splits_launches(dev):
    print("[case] pack 300 tensors", flush=True)
    shapes = [(17 + i,) for i in range(300)]
    grads = _tensors(1, shapes, torch.bfloat16)
    offs, total = ops.bucket_plan([t.numel() for t in grads], 2, 256)
    flat = torch.zeros(total, device=dev)
    ops.bucket_pack([t.to(dev) for t in grads], offs, flat, accumulate=True)
    ref = OB.pack(torch.zeros(total), grads, offs)
    assert torch.equal(flat.cpu(), ref)


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 8192 * 3 + 5])
@pytest.mark.parametrize("shadow", [None, torch.bfloat16])
def test_adamw_matches_torch_optim(dev, n, shadow):
    print(f"[case] adamw n={n} shadow={shadow}", flush=True)
    g = torch.Generator().manual_seed(2)
    lr, betas, eps, wd = ADAMW["lr"], ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"]
    p = torch.randn(n, generator=g) * 0.02
    m = torch.zeros(n)
    v = torch.zeros(n)
    P, M, V = p.to(dev), m.to(dev), v.to(dev)
    S = torch.zeros(n, dtype=shadow, device=dev) if shadow else None
    for step in range(1, 5):
        grad = torch.randn(n, generator=g) * 1e-3
        p, m, v = OB.adamw_step_torch(p, grad, m, v, step, lr, betas, eps, wd)
        G = grad.to(dev)
        ops.adamw_fused(P, M, V, G, step=step, lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=wd,
                        shadow=S, zero_grad=(step == 4))
        assert (P.cpu() - p).abs().max().item() <= ADAMW_TOL, f"master weights differ at step {step}"
        assert rel_err(M, m) <= 1e-5 and rel_err(V, v) <= 1e-5
        if S is not None:
            assert torch.equal(S, P.to(shadow))
        if step == 4:
            assert float(G.abs().max()) == 0.0   # zero_grad clears the bucket in the same pass
    assert (P.cpu() - p).abs().max().item() <= 1e-7   # in practice far inside the 1e-6 bar


def test_bucket_zero(dev):
    for n in (1, 5, 4096, 100003):
        t = torch.ones(n, device=dev)
        ops.bucket_zero(t)
        assert float(t.abs().max()) == 0.0


def test_flatten_views_pack_step_unflatten(dev):
    """The reference flow: flatten -> (backward fills p.grad) -> pack -> optimizer step -> params
    (views) see the update.  bf16 params, fp32 grad bucket, fp32 master."""
    print("[case] ParamStorage flow", flush=True)
    shapes = [(64, 32), (32,), (5, 7, 3), (1000,)]
    params0 = _tensors(3, shapes, torch.bfloat16, scale=0.02)
    params = [torch.nn.Parameter(t.clone().to(dev)) for t in params0]
    store = StageStore()
    store.buckets["b0"] = BucketState()
    store.zero_managed_ubids.add("b0")
    lr, betas, eps, wd = ADAMW["lr"], ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"]
    flatten_params(store.buckets["b0"], params, optim_class=lambda ps: FusedAdamW(ps, lr=lr, betas=betas, eps=eps, weight_decay=wd))
    b = store.buckets["b0"]
    offs_ref, total_ref = OB.plan_offsets([math.prod(s) for s in shapes], 2, 256)
    assert [spec[1] for spec in b.param_view_specs] == offs_ref and b.flat_params.numel() == total_ref
    for p, p0, off in zip(params, params0, offs_ref):
        assert torch.equal(p.detach().cpu(), p0)                                   # values kept
        assert p.data_ptr() == b.flat_params.data_ptr() + 2 * off                   # and they are views
        assert (p.data_ptr() % 256) == 0                                            # 256-byte aligned
    storage = ParamStorage(store)
    storage.zero_grad_buffers(None)
    master = OB.flatten(params0, offs_ref, total_ref, torch.float32)
    m = torch.zeros(total_ref)
    v = torch.zeros(total_ref)
    g = torch.Generator().manual_seed(4)
    for step in (1, 2):
        flat_g = torch.zeros(total_ref)
        for mb in range(3):   # three microbatches accumulate into the bucket
            grads = [(torch.randn(s, generator=g) * 1e-3).bfloat16() for s in shapes]
            for p, gr in zip(params, grads):
                p.grad = gr.to(dev)
            storage.accumulate_zero_param_grads_to_flat("b0", None)
            assert all(p.grad is None for p in params)
            OB.pack(flat_g, grads, offs_ref)
        assert torch.equal(b.flat_grads.cpu(), flat_g), "bucket contents must be bit-exact"
        storage.step_zero_shard_optimizers(None, {})
        master, m, v = OB.adamw_step_torch(master, flat_g, m, v, step, lr, betas, eps, wd)
        got_master = b.shard_optimizer.state[b.shard_param]["master"].cpu()
        assert (got_master - master).abs().max().item() <= ADAMW_TOL
        for p, off, s in zip(params, offs_ref, shapes):                              # unflatten = views
            n = math.prod(s)
            assert torch.equal(p.detach().cpu().reshape(-1), master[off:off + n].bfloat16())
        storage.zero_grad_buffers(None)
        assert float(b.flat_grads.abs().max()) == 0.0


def test_cfg2_full_size_properties(dev):
    """Config 2 at full size (96 tensors, ~170 M elements): offsets bit-exact, flatten -> unflatten is
    the identity, packing twice doubles, AdamW step 1 equals its closed form."""
    print("[case] cfg2 full size", flush=True)
    manifest = bucket_manifest_cfg2()
    shapes = [s for _, s in manifest]
    numels = [math.prod(s) for s in shapes]
    offs, total = ops.bucket_plan(numels, 2, 256)
    assert (offs, total) == OB.plan_offsets(numels, 2, 256)
    gen = torch.Generator(device=dev).manual_seed(0)
    grads = [(torch.randn(s, device=dev, generator=gen) * 1e-3).bfloat16() for s in shapes]
    flat_g = torch.zeros(total, device=dev)
    ops.bucket_pack(grads, offs, flat_g, accumulate=True)
    for i in (0, 5, 17, 95):
        assert torch.equal(flat_g[offs[i]:offs[i] + numels[i]], grads[i].float().reshape(-1))
    once = flat_g.clone()
    ops.bucket_pack(grads, offs, flat_g, accumulate=True)
    assert torch.equal(flat_g, once * 2)
    outs = [torch.empty_like(t) for t in grads]
    ops.bucket_unpack(once, outs, offs)
    assert all(torch.equal(a, b) for a, b in zip(outs, grads))
    # AdamW step 1 closed form on the GPU in fp32: p(1-lr wd) - lr g/(|g|+eps)
    lr, betas, eps, wd = ADAMW["lr"], ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"]
    master = torch.randn(total, device=dev, generator=gen) * 0.02
    expect = master.double() * (1 - lr * wd) - lr * once.double() / (once.double().abs() + eps)
    m = torch.zeros_like(master)
    v = torch.zeros_like(master)
    shadow = torch.empty(total, dtype=torch.bfloat16, device=dev)
    ops.adamw_fused(master, m, v, once, step=1, lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=wd, shadow=shadow)
    # padding elements have g == 0 -> update 0/(0+eps) = 0, also covered by the closed form
    assert (master.double() - expect).abs().max().item() <= ADAMW_TOL
    assert torch.equal(shadow, master.bfloat16())


def test_timing_select_brackets_one_kernel_only(dev):
    """pk_timing_select restricts the per-launch event pairs to one kernel id."""
    from piper_amd import _lib
    n = 1 << 16
    g = (torch.randn(n, device=dev) * 1e-3).bfloat16()
    flat = torch.zeros(n, device=dev)
    p = torch.randn(n, device=dev)
    m, v = torch.zeros_like(p), torch.zeros_like(p)

    def work():
        ops.bucket_pack([g], [0], flat, accumulate=False)
        ops.adamw_fused(p, m, v, flat, step=1, lr=1e-3, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)

    try:
        _lib.timing_enable(True)
        _lib.timing_collect()
        work()
        assert sorted(k for k, _ in _lib.timing_collect()) == ["adamw", "bucket_pack"]
        _lib.timing_select("adamw")
        work()
        work()
        rec = _lib.timing_collect()
        assert [k for k, _ in rec] == ["adamw", "adamw"] and all(ms > 0 for _, ms in rec)
        _lib.timing_select(None)
        work()
        assert len(_lib.timing_collect()) == 2
        with pytest.raises(ValueError):
            _lib.timing_select("no_such_kernel")
    finally:
        _lib.timing_select(None)
        _lib.timing_enable(False)
        _lib.timing_collect()


@pytest.mark.parametrize("grad_dtype,param_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32)])
@pytest.mark.parametrize("earlier_microbatches", [0, 2])
def test_adamw_with_the_last_pack_folded_in_is_bit_identical(dev, grad_dtype, param_dtype, earlier_microbatches):
    """pk_adamw_fused_packed against pk_bucket_pack(accumulate) followed by pk_adamw_fused: master,
    moments and the bf16 parameter bucket bit for bit, over tensors whose sizes are not multiples of
    the vector width, a tensor without a gradient, and three steps."""
    print(f"[case] adamw with folded pack {grad_dtype} earlier={earlier_microbatches}", flush=True)
    shapes = [(3, 5), (8192,), (1,), (777, 13), (2, 8200), (64, 64), (1027,)]
    numels = [math.prod(s) for s in shapes]
    esize = 2 if param_dtype == torch.bfloat16 else 4
    offs, total = ops.bucket_plan(numels, esize, 256)
    gen = torch.Generator().manual_seed(7)
    master0 = torch.zeros(total)
    for o, n in zip(offs, numels):
        master0[o:o + n] = torch.randn(n, generator=gen) * 0.02
    hp = dict(lr=ADAMW["lr"], beta1=ADAMW["betas"][0], beta2=ADAMW["betas"][1], eps=ADAMW["eps"], weight_decay=ADAMW["weight_decay"])

    def state():
        m = master0.clone().to(dev)
        sh = m.to(torch.bfloat16) if param_dtype == torch.bfloat16 else None
        return m, torch.zeros_like(m), torch.zeros_like(m), sh

    two, one = state(), state()
    for step in range(1, 4):
        flat_two = torch.zeros(total, device=dev)
        flat_one = torch.zeros(total, device=dev)
        for mb in range(earlier_microbatches):
            gs = [t.to(dev) for t in _tensors(100 * step + mb, shapes, grad_dtype)]
            ops.bucket_pack(gs, offs, flat_two, accumulate=True)
            ops.bucket_pack(gs, offs, flat_one, accumulate=True)
        last = [t.to(dev) for t in _tensors(100 * step + 50, shapes, grad_dtype)]
        last[2] = None if step == 2 else last[2]              # a tensor without a gradient in the last microbatch
        ops.bucket_pack(last, offs, flat_two, accumulate=True)
        ops.adamw_fused(two[0], two[1], two[2], flat_two, step=step, shadow=two[3], **hp)
        ops.adamw_fused_packed(one[0], one[1], one[2], flat_one if earlier_microbatches else None, last, offs, numels,
                               step=step, shadow=one[3], **hp)
        torch.cuda.synchronize()
        for a, b, name in zip(two, one, ("master", "exp_avg", "exp_avg_sq", "bf16 parameters")):
            if a is not None:
                assert torch.equal(a, b), (step, name)
    assert float(one[1].abs().max()) > 0
    # and one step against the oracle: torch.optim.AdamW on the oracle's packed gradient (1e-6 as everywhere)
    if earlier_microbatches == 0:
        grads = _tensors(150, shapes, grad_dtype)
        z = torch.zeros(total)
        ref_m, _, _ = OB.adamw_step_torch(master0, OB.pack(torch.zeros(total), grads, offs), z, z, 1, ADAMW["lr"],
                                          ADAMW["betas"], ADAMW["eps"], ADAMW["weight_decay"])
        m1, v1, s1, sh1 = state()
        ops.adamw_fused_packed(m1, v1, s1, None, [t.to(dev) for t in grads], offs, numels, step=1, shadow=sh1, **hp)
        assert (m1.cpu() - ref_m).abs().max().item() <= ADAMW_TOL
