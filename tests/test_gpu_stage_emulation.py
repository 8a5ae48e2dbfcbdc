"""One-GPU pipeline-stage emulation (benchmark configuration 5): two Qwen3-MoE decoder layers as
two compute buckets, microbatches in 1F1B order, parameters unflattened from a ZeRO-3-style local
bucket before each forward, gradient packing on a second stream, one fused AdamW step.

The MoE half of each layer (ffn_norm, router, experts, combine + residual) runs on the HIP kernels;
attention (GQA with q/k RMSNorm and RoPE) is outside the accelerated path and uses torch operators
on both sides.  A reduced shape is compared with the CPU oracle running the same layers in fp32;
the full shape (hidden 2048, 32/4 heads of 128, 128 experts top-8, intermediate 768, 4 microbatches
of 2 x 2048 tokens) is checked through size-independent properties."""
import math

import pytest
import torch
import torch.nn.functional as TF

from conftest import ADAMW_TOL, BF16_TOL, rel_err
from oracle import bucket as OB
from oracle import moe as O
from piper_amd import functional as F_
from piper_amd.configs import ADAMW
from piper_amd.executor import StageExecutor
from piper_amd.optim import FusedAdamW
from piper_amd.schedule import device_tasks, one_f_one_b_order, plan_stage_buckets
from piper_amd.stage import StageNode, load_stage

pytestmark = pytest.mark.gpu

LAYER_PARAMS = ("attention_norm", "wq", "wk", "wv", "wo", "q_norm", "k_norm", "ffn_norm", "w1", "w3", "w2", "w_gate")


def _layer_shapes(dim, n_heads, n_kv, hd, E, I):
    return dict(attention_norm=(dim,), wq=(n_heads * hd, dim), wk=(n_kv * hd, dim), wv=(n_kv * hd, dim),
                wo=(dim, n_heads * hd), q_norm=(hd,), k_norm=(hd,), ffn_norm=(dim,),
                w1=(E, I, dim), w3=(E, I, dim), w2=(E, dim, I), w_gate=(E, dim))


def _init_layer(gen, shapes, dtype):
    out = {}
    for k, s in shapes.items():
        if k.endswith("norm"):
            out[k] = (1.0 + 0.05 * torch.randn(s, generator=gen)).to(dtype)
        elif k == "w_gate":
            out[k] = torch.randn(s, generator=gen) * 0.02          # fp32 router
        else:
            out[k] = (torch.randn(s, generator=gen) * 0.02).to(dtype)
    return out


def _rope(x, theta=1e6):
    # x [B, S, heads, hd]; rotate-half formulation
    B, S, Hh, hd = x.shape
    pos = torch.arange(S, device=x.device, dtype=torch.float32)
    inv = theta ** (-torch.arange(0, hd, 2, device=x.device, dtype=torch.float32) / hd)
    ang = pos[:, None] * inv[None, :]
    cos, sin = ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]
    x1, x2 = x.float()[..., : hd // 2], x.float()[..., hd // 2:]
    return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).to(x.dtype)


def _attn_forward(x, p, cfg, hip: bool):
    """Attention half of a decoder layer, x [B,S,dim] -> [B,S,dim] (torch operators on both sides;
    only the RMSNorms run on the HIP kernel when hip=True)."""
    dim, n_heads, n_kv, hd, E, I, K = cfg
    B, S, _ = x.shape
    norm = (lambda t, w: F_.rmsnorm(t, w, 1e-6)) if hip else (lambda t, w: O.rmsnorm(t, w, 1e-6))
    h = norm(x, p["attention_norm"])
    q = (h @ p["wq"].t()).view(B, S, n_heads, hd)
    k = (h @ p["wk"].t()).view(B, S, n_kv, hd)
    v = (h @ p["wv"].t()).view(B, S, n_kv, hd)
    q, k = _rope(norm(q, p["q_norm"])), _rope(norm(k, p["k_norm"]))
    a = TF.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True,
                                        enable_gqa=True)
    return x + a.transpose(1, 2).reshape(B, S, n_heads * hd) @ p["wo"].t()


def _moe_forward(x, p, cfg, hip: bool, top_idx=None):
    """MoE half: x + moe(ffn_norm(x)).  top_idx (oracle side only): route with these expert indices
    instead of the oracle's own selection."""
    dim, K = cfg[0], cfg[6]
    B, S, _ = x.shape
    x2 = x.reshape(-1, dim)
    if hip:
        y = F_.moe_block(x2, p["ffn_norm"], p["w_gate"], None, p["w1"], p["w2"], p["w3"], top_k=K, route_norm=True)
    else:
        y, _ = O.moe_block(x2, p["ffn_norm"], p["w_gate"], None, p["w1"], p["w2"], p["w3"], K, True,
                           compute_dtype=torch.float32, top_idx=top_idx)
    return y.reshape(B, S, dim)


def _layer_forward(x, p, cfg, hip: bool, top_idx=None):
    return _moe_forward(_attn_forward(x, p, cfg, hip), p, cfg, hip, top_idx)


ATTN_PARAMS = ("attention_norm", "wq", "wk", "wv", "wo", "q_norm", "k_norm")
MOE_PARAMS = ("w1", "w3", "w2", "ffn_norm", "w_gate")      # placeholder order of the MoE node


def _schedule(n_microbatches, bucket_size_mb):
    """A one-stage schedule file: place, replicate (with or without bucket_size), split and the
    1F1B order row of a single rank."""
    rep = {"op": "replicate", "filter": {"PP": 0}, "devices": [0], "reduce_stream": "dp_stream", "shard_params": True}
    if bucket_size_mb is not None:
        rep["bucket_size"] = bucket_size_mb
    return ([{"op": "place", "filter": {"PP": 0}, "devices": [0]}, rep,
             {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": n_microbatches}]
            + one_f_one_b_order(1, n_microbatches))


def _build(layers, cfg, dev, dtype, n_microbatches, bucket_size_mb=None):
    """The stage as the schedule cuts it: every decoder layer is two compute nodes (attention, MoE
    block); `replicate.bucket_size` groups the nodes into parameter buckets, each a ZeRO-3 style
    compute bucket (parameters re-pointed at the flat buffer before use, the fp32 router gate in a
    companion buffer).  Returns (store, executor, task list, {(layer, name): (state, offset, numel, shape)})."""
    opt = lambda ps: FusedAdamW(ps, **ADAMW)
    nodes, where = [], {}
    for li, l in enumerate(layers):
        ps = {n: torch.nn.Parameter(l[n].to(dev)) for n in LAYER_PARAMS}
        nodes.append(StageNode(lambda x, p, _c=cfg: _attn_forward(x, p, _c, True), {n: ps[n] for n in ATTN_PARAMS}))
        nodes.append(StageNode(lambda x, p, _c=cfg: _moe_forward(x, p, _c, True), {n: ps[n] for n in MOE_PARAMS}))
        for n in LAYER_PARAMS:
            where[id(ps[n])] = (li, n)
    sched = _schedule(n_microbatches, bucket_size_mb)
    groups, stage_ubids = plan_stage_buckets(sched, [[n.param_bytes() for n in nodes]])
    store = load_stage(nodes, groups[0], ubids=stage_ubids[0], optim_class=opt)
    tasks = device_tasks(sched, stage_ubids=stage_ubids)
    ex = StageExecutor(store, compute_stream=torch.cuda.Stream(), pack_stream=torch.cuda.Stream())
    index = {}
    for b in store.buckets.values():
        for state in b.with_companions():
            for (p, off, n, shape) in state.param_view_specs:
                index[where[id(p)]] = (state, off, n, shape)
    return store, ex, tasks, index, groups[0]


def _packed_grad(index, layer, name):
    state, off, n, shape = index[(layer, name)]
    return state.flat_grads[off:off + n].view(shape)


REDUCED = {
    # dim, heads, kv heads, head_dim, E, I, K  ->  bucket_size (MB) and the buckets the planner must produce
    "one_bucket_per_stage": ((256, 4, 2, 64, 8, 128, 2), None, 1),
    # 1 MiB expert tensors under a 1 MB threshold: attention 0 | MoE 0 + attention 1 | MoE 1
    "three_buckets": ((256, 8, 2, 64, 8, 256, 2), 1, 3),
}


@pytest.mark.parametrize("case", list(REDUCED))
def test_reduced_stage_against_cpu_oracle(dev, case):
    cfg, bucket_mb, want_buckets = REDUCED[case]
    B, S, MB = 2, 64, 3
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(21)
    shapes = _layer_shapes(*cfg[:6])
    layers = [_init_layer(gen, shapes, dtype) for _ in range(2)]
    xs = [torch.randn(B, S, cfg[0], generator=gen).to(dtype) for _ in range(MB)]

    # the device runs first and its routing decisions are recorded, in call order (1F1B on one
    # rank: microbatch by microbatch, layer 0 then layer 1)
    from piper_amd import ops
    chosen = []
    real_topk = ops.route_topk

    def recording_topk(*a, **kw):
        scores, idx = real_topk(*a, **kw)
        chosen.append(idx.cpu())
        return scores, idx

    print(f"[case] reduced stage {case} cfg={cfg} bucket_size={bucket_mb}", flush=True)
    store, ex, tasks, index, groups = _build(layers, cfg, dev, dtype, MB, bucket_mb)
    assert len(groups) == want_buckets, groups
    ops.route_topk = recording_topk
    try:
        out = ex.run(tasks, [x.to(dev) for x in xs])
        torch.cuda.synchronize()
    finally:
        ops.route_topk = real_topk
    assert len(chosen) == 2 * MB

    # The oracle routes every token as the device did.  End to end the bf16 stage feeds its routers
    # activations that differ from the fp32 oracle's by bf16 rounding (attention, previous layer), so
    # a few tokens on a near-tie would otherwise choose another expert and move their contribution
    # between expert gradients, which no tolerance on a gradient can tell from a wrong scale.
    ref = [{k: v.clone().float().requires_grad_(True) for k, v in l.items()} for l in layers]
    ref_losses = []
    flips = 0
    for mb, x in enumerate(xs):
        h = x.float()
        for li, p in enumerate(ref):
            idx = chosen[2 * mb + li]
            with torch.no_grad():      # how many tokens the oracle alone would have routed differently
                own = _layer_forward(h, p, cfg, False)
            h_next = _layer_forward(h, p, cfg, False, top_idx=idx)
            flips += int((own - h_next.detach()).abs().amax(dim=-1).gt(0).sum())
            h = h_next
        loss = h.sum()
        loss.backward()
        ref_losses.append(loss.detach())
    print(f"[info] tokens routed differently by the fp32 oracle on its own: {flips} of {2 * MB * B * S}", flush=True)

    for got, want in zip(out["losses"], ref_losses):
        assert abs(got.item() - want.item()) <= max(4 * BF16_TOL * abs(want.item()), 2.0)
    # two layers deep, gradients accumulated over three microbatches: 4x the single-kernel bound
    for li in (0, 1):
        for name in LAYER_PARAMS:
            assert rel_err(_packed_grad(index, li, name), ref[li][name].grad) <= 4 * BF16_TOL, (li, name)


def test_planner_buckets_pack_the_same_gradients_as_one_bucket(dev):
    """A stage that `replicate.bucket_size` cuts into three parameter buckets (pack of a bucket on
    the second stream while the backward of the bucket before it computes) against the same stage
    as one bucket: every packed gradient and every updated parameter bit for bit.  The cut only
    moves where autograd graphs end and which flat buffer a tensor lives in."""
    cfg, bucket_mb, want_buckets = REDUCED["three_buckets"]
    B, S, MB = 2, 64, 3
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(33)
    shapes = _layer_shapes(*cfg[:6])
    layers = [_init_layer(gen, shapes, dtype) for _ in range(2)]
    xs = [torch.randn(B, S, cfg[0], generator=gen).to(dtype).to(dev) for _ in range(MB)]
    results = {}
    for label, mb_size in (("whole", None), ("cut", bucket_mb)):
        print(f"[case] stage as {label} bucket_size={mb_size}", flush=True)
        store, ex, tasks, index, groups = _build(layers, cfg, dev, dtype, MB, mb_size)
        assert len(groups) == (1 if mb_size is None else want_buckets), groups
        if mb_size is not None:
            # the plan is the reference's: attention 0 alone, MoE 0 with attention 1 (the run that
            # holds MoE 0's last small tensors also takes attention 1's), MoE 1
            assert groups == [[0], [1, 2], [3]]
            from piper_amd.tasks import TaskType
            first_bwd = [t.ubid for t in tasks if t.type is TaskType.BWD and t.mb == 0]
            assert first_bwd == [2, 1, 0]
        # attention through torch's reference implementation: the fused attention backward may add
        # its partial results in an order that changes from run to run
        with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
            out = ex.run(tasks, xs)
            torch.cuda.synchronize()
        grads = {key: _packed_grad(index, *key).clone() for key in index}
        params = {key: index[key][0].flat_params[index[key][1]:index[key][1] + index[key][2]].clone() for key in index}
        results[label] = (torch.stack(out["losses"]), grads, params)
    assert torch.equal(results["whole"][0], results["cut"][0])
    for key in results["whole"][1]:
        assert torch.equal(results["whole"][1][key], results["cut"][1][key]), ("gradient", key)
        assert torch.equal(results["whole"][2][key], results["cut"][2][key]), ("parameter", key)
        assert float(results["cut"][1][key].abs().max()) > 0, key


def test_full_size_stage_properties(dev):
    cfg = (2048, 32, 4, 128, 128, 768, 8)
    B, S, MB = 2, 2048, 4
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(5)
    shapes = _layer_shapes(*cfg[:6])
    layers = [_init_layer(gen, shapes, dtype) for _ in range(2)]
    vocab = 151936
    emb = (torch.randn(4096, cfg[0], generator=gen) * 0.5).to(dtype).to(dev)     # rows of a stand-in embedding table
    ids = [torch.randint(0, vocab, (B, S), generator=gen) for _ in range(MB)]
    xs = [emb[(i % 4096).to(dev)] for i in ids]

    # bucket_size 25 (MB), the reference's default threshold (src/bucket.py:20): the 403 MB expert
    # tensors stand alone, attention 0 is a bucket, MoE 0 shares one with attention 1
    print("[case] full-size stage, bucket_size=25", flush=True)
    store, ex, tasks, index, groups = _build(layers, cfg, dev, dtype, MB, 25)
    assert len(groups) >= 3, groups
    states = [st for b in store.buckets.values() for st in b.with_companions()]
    before = [st.flat_params.clone() for st in states]
    out = ex.run(tasks, xs)
    torch.cuda.synchronize()
    assert len(out["losses"]) == MB and all(torch.isfinite(l) for l in out["losses"])
    for b, old in zip(states, before):
        assert torch.isfinite(b.flat_grads).all() and float(b.flat_grads.abs().max()) > 0
        st = b.shard_optimizer.state[b.shard_param]
        assert st["step"] == 1
        # parameters are views of the bucket the optimizer wrote, and the bucket moved
        for (p, off, n, shape) in b.param_view_specs:
            assert p.data_ptr() == b.flat_params.data_ptr() + off * b.flat_params.element_size() and p.grad is None
        assert not torch.equal(old, b.flat_params)
        # the update equals torch.optim.AdamW on a slice of the bucket, given the bucket's own gradient
        n = min(b.flat_params.numel(), 1 << 20)
        m0 = old[:n].float().cpu()
        z = torch.zeros_like(m0)
        want, _, _ = OB.adamw_step_torch(m0, b.flat_grads[:n].cpu(), z, z, 1, ADAMW["lr"], ADAMW["betas"], ADAMW["eps"],
                                         ADAMW["weight_decay"])
        assert (st["master"][:n].cpu() - want).abs().max().item() <= ADAMW_TOL
    # every token contributed K rows to the experts of both layers: the expert gradients are dense
    for li in (0, 1):
        g = _packed_grad(index, li, "w2")
        assert int((g.abs().amax(dim=(1, 2)) > 0).sum()) == cfg[4]


def test_last_pack_folded_into_the_optimizer_step(dev):
    """StageExecutor(fuse_last_pack=True): the pack after a bucket's last backward is skipped and the
    optimizer kernel reads those gradients directly.  Same updated parameters, bit for bit, as the
    iteration that packs every microbatch."""
    cfg, bucket_mb, _ = REDUCED["three_buckets"]
    B, S, MB = 2, 64, 3
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(44)
    shapes = _layer_shapes(*cfg[:6])
    layers = [_init_layer(gen, shapes, dtype) for _ in range(2)]
    xs = [torch.randn(B, S, cfg[0], generator=gen).to(dtype).to(dev) for _ in range(MB)]
    results = {}
    for fuse in (False, True):
        print(f"[case] stage with fuse_last_pack={fuse}", flush=True)
        store, ex, tasks, index, _ = _build(layers, cfg, dev, dtype, MB, bucket_mb)
        ex.fuse_last_pack = fuse
        with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
            out = ex.run(tasks, xs)
            torch.cuda.synchronize()
        params = {key: index[key][0].flat_params[index[key][1]:index[key][1] + index[key][2]].clone() for key in index}
        masters = {key: index[key][0].shard_optimizer.state[index[key][0].shard_param]["master"][
            index[key][1]:index[key][1] + index[key][2]].clone() for key in index}
        results[fuse] = (torch.stack(out["losses"]), params, masters)
        for b in store.buckets.values():
            for st in b.with_companions():
                assert st.pending_grads is None and all(p.grad is None for p, *_ in st.param_view_specs)
    assert torch.equal(results[False][0], results[True][0])
    for key in results[False][1]:
        assert torch.equal(results[False][1][key], results[True][1][key]), ("parameter", key)
        assert torch.equal(results[False][2][key], results[True][2][key]), ("master", key)
