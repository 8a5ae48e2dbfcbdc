"""The benchmark configurations and their seeded synthetic inputs.

Tensors are drawn on the CPU from one ``torch.Generator`` seeded with 0, in a fixed order
(activations, router gate, [router bias], w1, w3, w2, upstream gradient), so that the GPU run and
a CPU checker consume identical bits.  There are no datasets or checkpoints involved.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class ExpertRegionConfig:
    name: str
    tokens: int            # tokens per microbatch (T)
    hidden: int            # H
    num_experts: int       # E
    top_k: int             # K
    inter: int             # I (SwiGLU expert intermediate size)
    dtype: torch.dtype
    microbatches: int = 1
    route_norm: bool = True
    route_scale: float = 1.0
    zipf_s: float | None = None   # router-bias skew (None = no bias)
    zipf_alpha: float = 0.0

    @property
    def routed_rows(self) -> int:
        return self.tokens * self.top_k

    @property
    def gemm_flops_per_token(self) -> int:
        """fwd+bwd flops of the three expert GEMMs: 3 passes x 3 GEMMs x 2*K*H*I."""
        return 18 * self.top_k * self.hidden * self.inter


# Tiny Qwen3-MoE-style region, fp32: 4 microbatches x 2 sequences x 128 tokens.
CFG1 = ExpertRegionConfig("cfg1-tiny-fp32", tokens=256, hidden=256, num_experts=8, top_k=2, inter=512,
                          dtype=torch.float32, microbatches=4)
# Qwen3-30B-A3B-shaped region (examples/models/qwen3.py:151-177), bf16 with fp32 router.
CFG3 = ExpertRegionConfig("cfg3-qwen3-30b-a3b", tokens=4096, hidden=2048, num_experts=128, top_k=8, inter=768,
                          dtype=torch.bfloat16)
# Same shape, 16384 tokens, Zipf(1.2) expert popularity through a router logit bias.  alpha is
# calibrated (seed 0) so that the 8 most popular experts receive about 40 % of the assignments.
CFG4 = ExpertRegionConfig("cfg4-qwen3-30b-a3b-zipf", tokens=16384, hidden=2048, num_experts=128, top_k=8, inter=768,
                          dtype=torch.bfloat16, zipf_s=1.2, zipf_alpha=0.45)

ADAMW = dict(lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)


def zipf_logit_bias(num_experts: int, s: float, alpha: float) -> torch.Tensor:
    """b_e = alpha * log p_e with p_e proportional to (e+1)^-s: expert 0 is the most popular."""
    ranks = torch.arange(1, num_experts + 1, dtype=torch.float64)
    p = ranks.pow(-s)
    p = p / p.sum()
    return (alpha * p.log()).float()


def make_expert_region_inputs(cfg: ExpertRegionConfig, seed: int = 0, microbatch: int = 0) -> dict:
    """CPU tensors of one microbatch.  Weights are identical for every microbatch of a config;
    activations and the upstream gradient depend on the microbatch index."""
    gen = torch.Generator().manual_seed(seed)
    T, H, E, I = cfg.tokens, cfg.hidden, cfg.num_experts, cfg.inter
    xs = [torch.randn(T, H, generator=gen) for _ in range(cfg.microbatches)]
    w_gate = torch.randn(E, H, generator=gen) * 0.02
    gate_bias = zipf_logit_bias(E, cfg.zipf_s, cfg.zipf_alpha) if cfg.zipf_s is not None else None
    w1 = torch.randn(E, I, H, generator=gen) * 0.02
    w3 = torch.randn(E, I, H, generator=gen) * 0.02
    w2 = torch.randn(E, H, I, generator=gen) * 0.02
    douts = [torch.randn(T, H, generator=gen) for _ in range(cfg.microbatches)]
    dt = cfg.dtype
    return dict(x=xs[microbatch].to(dt), w_gate=w_gate, gate_bias=gate_bias, w1=w1.to(dt), w3=w3.to(dt),
                w2=w2.to(dt), d_out=douts[microbatch].to(dt))


# ------------------------------------------------------------------ bucket manifest (config 2)
def bucket_manifest_cfg2() -> list[tuple[str, tuple[int, ...]]]:
    """96 tensors with the parameter shapes of two Qwen3-30B-A3B decoder layers
    (dim 2048, 32 q heads / 4 kv heads of head_dim 128, expert intermediate 768;
    examples/models/qwen3.py:151-177).  Per layer: attention q/k/v/o, the two RMSNorm vectors and
    14 experts x (gate, up, down) -- 48 tensors; 28 experts in total keeps the count at 96."""
    H, I, HD, NQ, NKV = 2048, 768, 128, 32, 4
    out = []
    for layer in range(2):
        p = f"layers.{layer}."
        out += [
            (p + "attention.wq.weight", (NQ * HD, H)),
            (p + "attention.wk.weight", (NKV * HD, H)),
            (p + "attention.wv.weight", (NKV * HD, H)),
            (p + "attention.wo.weight", (H, NQ * HD)),
            (p + "attention_norm.weight", (H,)),
            (p + "ffn_norm.weight", (H,)),
        ]
        for e in range(14):
            out += [
                (p + f"moe.experts.{e}.w1", (I, H)),
                (p + f"moe.experts.{e}.w3", (I, H)),
                (p + f"moe.experts.{e}.w2", (H, I)),
            ]
    assert len(out) == 96
    return out


def manifest_numel(manifest) -> int:
    return sum(math.prod(s) for _, s in manifest)
