#!/usr/bin/env python3
"""Headline benchmark: expert-region forward+backward tokens/s on the Qwen3-30B-A3B-shaped
configuration (one microbatch of 4096 tokens per step), with the roofline of its dominant kernel,
the ZeRO bucket path (pack + fused AdamW) in GB/s, and the CPU oracle timed on the host cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg4] [--no-cpu-baseline]

Prints ONE JSON line.  Inputs are synthetic (seed 0), generated on the host and resident in HBM
before the timed region starts.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0            # MI355X HBM3E


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", choices=["cfg3", "cfg4"], default="cfg3")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bucket", action="store_true")
    ap.add_argument("--no-cfg4", action="store_true", help="skip the cfg4 sub-object of the default run")
    ap.add_argument("--no-accumulate", action="store_true", help="skip the step that accumulates into existing gradients")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB fp32 device copy (pack_kernel<float,float>) so that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings can be scaled to a known size")
    return ap.parse_args()


def kernel_flops(cfg) -> dict:
    """Algorithmic flops of ONE launch of each GEMM kernel: 2*A*H*I per GEMM."""
    one = 2.0 * cfg.routed_rows * cfg.hidden * cfg.inter
    return {
        "swiglu_gate_up": 2 * one,   # gate and up projections in one launch
        "swiglu_down": one,
        "swiglu_dgrad_dh": one,
        "swiglu_dgrad_dx": 2 * one,  # d_g.w1 + d_u.w3
        "swiglu_wgrad": 3 * one,     # d_w1, d_w2, d_w3 in one launch (shapes without the K-contiguous path)
        "swiglu_wgrad_w2": one,      # d_w2 = d_out^T (score h)
        "swiglu_wgrad_w13": 2 * one,  # d_w1 = d_g^T x and d_w3 = d_u^T x in one launch
    }


def kernel_bytes(cfg) -> dict:
    """Algorithmic HBM bytes of ONE launch of each GEMM kernel: every operand read once, every
    result written once (bf16).  A = routed rows, T = tokens, E experts, H hidden, I intermediate.
    The transposed copies that the scaled SwiGLU backward writes for the weight gradient are an
    implementation choice, not algorithmic work: they count as one write / one read of d_g, d_u
    and score*h like the row-major tensors they stand in for."""
    A, T, E, H, I = cfg.routed_rows, cfg.tokens, cfg.num_experts, cfg.hidden, cfg.inter
    w = 2.0 * E * I * H          # one expert weight tensor
    return {
        "swiglu_gate_up": 2 * w + 2.0 * T * H + 3 * 2.0 * A * I,        # w1,w3 + x (each token once) -> g,u,h
        "swiglu_down": w + 2.0 * A * I + 2.0 * A * H,                   # w2 + h -> y
        # w2 + d_out (each token once) + g,u -> d_g,d_u,score*h (+ the score-gradient partials)
        "swiglu_dgrad_dh": w + 2.0 * T * H + 2 * 2.0 * A * I + 3 * 2.0 * A * I + 4.0 * A * (I / 64),
        "swiglu_dgrad_dx": 2 * w + 2 * 2.0 * A * I + 2.0 * A * H,       # w1,w3 + d_g,d_u -> d_x rows
        "swiglu_wgrad": 2 * 2.0 * T * H + 3 * 2.0 * A * I + 3 * w,      # d_out,x (each token once), score*h,d_g,d_u -> d_w1..3
        "swiglu_wgrad_w2": 2.0 * T * H + 2.0 * A * I + w,               # d_out (each token once), score*h -> d_w2
        "swiglu_wgrad_w13": 2.0 * T * H + 2 * 2.0 * A * I + 2 * w,      # x (each token once), d_g, d_u -> d_w1, d_w3
    }


# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same
# counters read for a plain device copy of known size.  The numbers and the commands that produced
# them are in the file named here, whose table this reads (first cell "<workload>:<kernel key>",
# fifth and sixth cell read MB and written MB); a kernel without a row reports null.
TRAFFIC_SOURCE = "profiles/bench_default_hbm_traffic.md"


def measured_traffic_bytes() -> dict:
    """{workload: {kernel key: (read + written) bytes per launch}} from the committed counter summary."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), TRAFFIC_SOURCE)
    out: dict = {}
    try:
        with open(path) as f:
            rows = [line.split("|") for line in f if line.startswith("| `")]
    except OSError:
        return out
    for cells in rows:
        try:
            workload, key = cells[1].strip().strip("`").split(":")
            read_mb, written_mb = (float(cells[i].replace(",", "")) for i in (5, 6))
        except (ValueError, IndexError):
            continue
        out.setdefault(workload, {})[key] = (read_mb + written_mb) * 1e6
    return out


MEASURED_TRAFFIC_BYTES = measured_traffic_bytes()


def bench_region(cfg, steps: int, warmup: int, accumulate: bool = False):
    """accumulate=False: the gradients are cleared before every step (first microbatch of an
    iteration).  accumulate=True: they are left in place and every step adds to them inside the
    weight-gradient kernels (any later microbatch; src/executors.py:333-343)."""
    import torch

    from piper_amd import _lib, functional as F_
    from piper_amd.configs import make_expert_region_inputs

    dev = torch.device("cuda:0")
    inp = make_expert_region_inputs(cfg)
    x = inp["x"].to(dev).requires_grad_(True)
    w_gate = inp["w_gate"].to(dev).requires_grad_(True)
    bias = inp["gate_bias"].to(dev).requires_grad_(True) if inp["gate_bias"] is not None else None
    w1, w2, w3 = (inp[k].to(dev).requires_grad_(True) for k in ("w1", "w2", "w3"))
    d_out = inp["d_out"].to(dev)
    leaves = [t for t in (x, w_gate, bias, w1, w2, w3) if t is not None]

    def step():
        if accumulate:
            x.grad = None         # the activation gradient is handed on, never accumulated
        else:
            for t in leaves:      # clear_param_grads: first microbatch of an iteration
                t.grad = None
        out = F_.expert_region(x, w_gate, bias, w1, w2, w3, top_k=cfg.top_k, route_norm=cfg.route_norm,
                               route_scale=cfg.route_scale)
        with F_.accumulate_weight_grads():      # a no-op while the parameters hold no gradient
            out.backward(d_out)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()

    def summarize(records, n_steps):
        per_kernel: dict = {}
        for name, ms in records:
            tot, n = per_kernel.get(name, (0.0, 0))
            per_kernel[name] = (tot + ms, n + 1)
        return {k: {"launches_per_step": n / n_steps, "avg_ms": tot / n, "ms_per_step": tot / n_steps}
                for k, (tot, n) in per_kernel.items()}

    # Untimed pass with every launch bracketed by events: the per-kernel table, and which GEMM
    # kernel dominates.  Forty event records a step cost the stream about 5% of the step, so the
    # timed region below brackets only that one kernel.
    profile_steps = max(1, min(steps, 5))
    _lib.timing_enable(True)
    _lib.timing_collect()
    for _ in range(profile_steps):
        step()
    torch.cuda.synchronize()
    summary = summarize(_lib.timing_collect(), profile_steps)
    dominant = max((k for k in summary if k in kernel_flops(cfg)), key=lambda k: summary[k]["ms_per_step"])
    _lib.timing_select(dominant)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    enqueue = time.perf_counter() - t0      # host time to launch everything (the GPU runs behind it)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timed = summarize(_lib.timing_collect(), steps)
    _lib.timing_select(None)
    _lib.timing_enable(False)
    summary[dominant] = timed[dominant]     # the dominant kernel's duration comes from the timed region
    summary["__dominant"] = dominant
    summary["__host_enqueue_s"] = enqueue
    return elapsed, summary


def bench_bucket(steps: int, warmup: int):
    """Config 2: 96 bf16 gradient tensors -> fp32 bucket (one pack launch), fused AdamW over the
    whole bucket writing the fp32 master and the bf16 parameter bucket the views alias."""
    import torch

    from piper_amd import _lib, ops
    from piper_amd.configs import ADAMW, bucket_manifest_cfg2

    dev = torch.device("cuda:0")
    manifest = bucket_manifest_cfg2()
    shapes = [s for _, s in manifest]
    numels = [math.prod(s) for s in shapes]
    offs, total = ops.bucket_plan(numels, 2, 256)
    gen = torch.Generator(device=dev).manual_seed(0)
    grads = [(torch.randn(s, device=dev, generator=gen) * 1e-3).bfloat16() for s in shapes]
    flat_g = torch.zeros(total, device=dev)
    master = torch.randn(total, device=dev, generator=gen) * 0.02
    m = torch.zeros_like(master)
    v = torch.zeros_like(master)
    shadow = master.bfloat16()
    state = {"step": 0}

    def step():
        state["step"] += 1
        ops.bucket_pack(grads, offs, flat_g, accumulate=False)
        ops.adamw_fused(master, m, v, flat_g, step=state["step"], lr=ADAMW["lr"], beta1=ADAMW["betas"][0],
                        beta2=ADAMW["betas"][1], eps=ADAMW["eps"], weight_decay=ADAMW["weight_decay"], shadow=shadow)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # timed region: nothing but the two launches per step on the stream
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # per-kernel durations: a second pass with each launch bracketed by HIP events
    _lib.timing_enable(True)
    _lib.timing_collect()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    records = _lib.timing_collect()
    _lib.timing_enable(False)
    # the same step with the pack folded into the optimizer kernel (the last microbatch of an
    # iteration, or the only one): bf16 gradients read straight from the tensors, no fp32 gradient bucket
    def fused_step():
        state["step"] += 1
        ops.adamw_fused_packed(master, m, v, None, grads, offs, numels, step=state["step"], lr=ADAMW["lr"],
                               beta1=ADAMW["betas"][0], beta2=ADAMW["betas"][1], eps=ADAMW["eps"],
                               weight_decay=ADAMW["weight_decay"], shadow=shadow)

    for _ in range(warmup):
        fused_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fused_step()
    torch.cuda.synchronize()
    fused_elapsed = time.perf_counter() - t0
    n_elems = sum(numels)
    pack_ms = [ms for k, ms in records if k == "bucket_pack"]
    adam_ms = [ms for k, ms in records if k == "adamw"]
    pack_avg, adam_avg = sum(pack_ms) / len(pack_ms), sum(adam_ms) / len(adam_ms)
    pack_bytes = 6.0 * n_elems            # read bf16 grad, write fp32 bucket
    adam_bytes = 30.0 * total             # read g,p,m,v (16) + write p,m,v (12) + bf16 parameter (2)
    agg_gbs = (pack_bytes + adam_bytes) * steps / elapsed / 1e9
    cfg2_traffic = MEASURED_TRAFFIC_BYTES.get("cfg2", {})
    traffic = cfg2_traffic["pack"] + cfg2_traffic["adamw"] if {"pack", "adamw"} <= set(cfg2_traffic) else None
    return {
        "metric": "bucket pack + fused AdamW HBM GB/s",
        "value": agg_gbs, "unit": "GB/s", "ms_per_step": elapsed / steps * 1e3,
        "config": {"workload": "cfg2: 96 tensors of two Qwen3-30B-A3B layers, bf16 grads / fp32 master",
                   "tensors": len(shapes), "elements": n_elems, "bucket_elements": total},
        "bytes_per_element": {"pack": 6, "adamw": 30},
        "per_kernel_source": "second pass with each launch bracketed by HIP events; value and ms_per_step are from the "
                             "timed region without brackets",
        "pack": {"avg_ms": pack_avg, "GB/s": pack_bytes / pack_avg / 1e6, "frac": pack_bytes / pack_avg / 1e6 / HBM_PEAK_GBS},
        "adamw": {"avg_ms": adam_avg, "GB/s": adam_bytes / adam_avg / 1e6, "frac": adam_bytes / adam_avg / 1e6 / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "achieved": agg_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": agg_gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                     "bytes_per_step": pack_bytes + adam_bytes},
        # one launch instead of two: its own algorithmic bytes (read bf16 grad 2 + p,m,v 12; write p,m,v 12 +
        # bf16 parameter 2 = 28 per element), and the time it takes against the two-kernel step
        "fused_last_pack": {"ms_per_step": fused_elapsed / steps * 1e3, "bytes_per_element": 28,
                            "GB/s": 28.0 * n_elems * steps / fused_elapsed / 1e9,
                            "frac": 28.0 * n_elems * steps / fused_elapsed / 1e9 / HBM_PEAK_GBS,
                            "traffic": cfg2_traffic.get("adamw_packed"),
                            "vs_two_kernels": (fused_elapsed / steps) / (elapsed / steps)},
    }


def _median_of_3(fn):
    """One warm-up pass, then the median of three timed passes (seconds)."""
    fn()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[1]


def _host_threads() -> int:
    import torch

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    return cores


def cpu_baseline(cfg):
    """The CPU oracle (un-padded per-expert loop, fp32) on a bounded sample of the same workload: one
    eighth of the experts with one eighth of the tokens, so that an expert receives as many rows as in
    the full microbatch and every GEMM keeps its shape; the full microbatch is eight such samples
    (the time of a pass goes into the per-expert matmuls and into writing the weight gradients,
    both proportional to the number of experts).  The fp32 copies of the inputs are made once,
    outside the timed passes."""
    import torch

    from oracle import moe as O
    from piper_amd.configs import make_expert_region_inputs

    cores = _host_threads()
    frac = 8 if cfg.num_experts % 8 == 0 and cfg.num_experts // 8 >= cfg.top_k and cfg.tokens % 8 == 0 else 1
    n_tok, n_exp = cfg.tokens // frac, cfg.num_experts // frac
    inp = make_expert_region_inputs(cfg)
    names = ("x", "w_gate", "w1", "w2", "w3")
    leaves = {k: (inp[k][:n_tok] if k == "x" else inp[k][:n_exp]).float().requires_grad_(True) for k in names}
    d_out = inp["d_out"][:n_tok].float()
    bias = inp["gate_bias"][:n_exp] if inp["gate_bias"] is not None else None

    def one():
        out, _ = O.moe_forward(leaves["x"], leaves["w_gate"], bias, leaves["w1"], leaves["w2"], leaves["w3"], cfg.top_k,
                               cfg.route_norm, cfg.route_scale, compute_dtype=torch.float32)
        torch.autograd.grad(out, list(leaves.values()), d_out)

    t = _median_of_3(one)
    return {"value": n_tok / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"first {n_tok} of {cfg.tokens} tokens routed over the first {n_exp} of {cfg.num_experts} experts "
                      f"({n_tok * cfg.top_k // n_exp} rows per expert on average, as in the full microbatch), fp32 per-expert loop, "
                      f"fwd+bwd, median of 3 after 1 warm-up ({t:.2f} s per pass)"}


def cpu_baseline_padded_bmm():
    """The reference's own formulation of the expert segment -- every expert padded to the total
    row count and run through dense batched matmuls (qwen3_bmm_experts_patch.py:11-50) -- inside the
    oracle's region, at config 1 (fp32, 256 tokens per microbatch; at config 3 the padded operand
    alone would take 17 GB).  Beside it the un-padded per-expert loop on the same input."""
    import torch

    from oracle import moe as O
    from piper_amd.configs import CFG1, make_expert_region_inputs

    cores = _host_threads()
    cfg = CFG1
    inp = make_expert_region_inputs(cfg)
    names = ("x", "w_gate", "w1", "w2", "w3")
    leaves = {k: inp[k].float().requires_grad_(True) for k in names}
    d_out = inp["d_out"].float()

    def region(experts):
        logits = O.gate_logits(leaves["x"], leaves["w_gate"], None)
        scores, idx = O.route_topk(logits, cfg.top_k, cfg.route_norm, cfg.route_scale)
        counts, _starts, perm, _inv = O.sort_by_expert(idx, cfg.num_experts)
        routed = O.permute(leaves["x"], perm, cfg.top_k)
        y = experts(leaves["w1"], leaves["w2"], leaves["w3"], routed, counts)
        out = O.unpermute_combine(y, perm, scores)
        torch.autograd.grad(out, list(leaves.values()), d_out)

    t_pad = _median_of_3(lambda: region(O.padded_bmm_experts))
    t_loop = _median_of_3(lambda: region(O.grouped_swiglu))
    return {"value": cfg.tokens / t_pad, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"config 1 (fp32, one microbatch of {cfg.tokens} tokens, 8 experts top-2), padded batched matmul as in "
                      f"the reference, fwd+bwd, median of 3 ({t_pad * 1e3:.1f} ms per pass)",
            "per_expert_loop_tokens_per_s": cfg.tokens / t_loop}


def cpu_baseline_bucket():
    """The reference's bucket arithmetic on the host cores, config 2 at full size: per tensor
    flat[o:o+n].add_(grad.to(f32)) (src/runtime.py:275-282), then torch.optim.AdamW(foreach=False) on
    the flat fp32 buffer (the shard optimizer of src/runtime.py:470-473 with the benchmark's
    optimizer).  Same algorithmic bytes per element as the GPU figure (6 + 28; the CPU side keeps no
    separate bf16 parameter copy)."""
    import torch

    from oracle import bucket as OB
    from piper_amd.configs import ADAMW, bucket_manifest_cfg2

    cores = _host_threads()
    shapes = [sh for _, sh in bucket_manifest_cfg2()]
    numels = [math.prod(sh) for sh in shapes]
    offs, total = OB.plan_offsets(numels, 2, 256)
    gen = torch.Generator().manual_seed(0)
    grads = [(torch.randn(sh, generator=gen) * 1e-3).bfloat16() for sh in shapes]
    flat_g = torch.zeros(total)
    master = (torch.randn(total, generator=gen) * 0.02).requires_grad_(True)
    opt = torch.optim.AdamW([master], lr=ADAMW["lr"], betas=ADAMW["betas"], eps=ADAMW["eps"],
                            weight_decay=ADAMW["weight_decay"], foreach=False)

    def one():
        flat_g.zero_()
        OB.pack(flat_g, grads, offs)
        master.grad = flat_g
        opt.step()

    t = _median_of_3(one)
    n = sum(numels)
    nbytes = 6.0 * n + 28.0 * total
    return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"config 2 at full size ({n} elements in 96 tensors): per-tensor add_ pack + torch.optim.AdamW("
                      f"foreach=False) on the flat fp32 buffer, median of 3 after 1 warm-up ({t:.2f} s per pass)"}


def region_result(cfg, steps: int, warmup: int, accumulate: bool = False) -> dict:
    """Tokens/s, fraction of the bf16 MFMA peak and the roofline of the dominant GEMM kernel for one
    expert-region configuration."""
    elapsed, kernels = bench_region(cfg, steps, warmup, accumulate)
    host_enqueue = kernels.pop("__host_enqueue_s")
    dominant = kernels.pop("__dominant")
    ms_per_step = elapsed / steps * 1e3
    tokens_per_s = cfg.tokens * steps / elapsed
    gemm_flops_step = cfg.gemm_flops_per_token * cfg.tokens
    mfma_frac_region = gemm_flops_step / (ms_per_step * 1e-3) / (MFMA_BF16_PEAK_TFLOPS * 1e12)

    flops = kernel_flops(cfg)
    gemm_kernels = {k: v for k, v in kernels.items() if k in flops}
    dom = gemm_kernels[dominant]
    nbytes = kernel_bytes(cfg)
    # the roofline that bounds the kernel: below the ridge point (peak flops / peak bandwidth) of
    # the published peaks, moving its algorithmic bytes takes longer than its algorithmic flops
    intensity = flops[dominant] / nbytes[dominant]
    ridge = MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    # the weight-gradient kernels that add to existing gradients have rows of their own (they read the old values)
    in_place = accumulate and dominant.startswith("swiglu_wgrad")
    traffic = MEASURED_TRAFFIC_BYTES.get(cfg.name.split("-")[0], {}).get(dominant + ("_accumulate" if in_place else ""))
    if intensity < ridge:
        achieved = nbytes[dominant] / (dom["avg_ms"] * 1e-3) / 1e9
        roof = {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": traffic}
    else:
        achieved = flops[dominant] / (dom["avg_ms"] * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic}
    roof.update({"traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                 "flops_per_launch": flops[dominant], "bytes_per_launch": nbytes[dominant],
                 "flops_per_byte": intensity, "avg_launch_ms": dom["avg_ms"],
                 "tflops": flops[dominant] / (dom["avg_ms"] * 1e-3) / 1e12})
    return {
        "metric": "expert-region fwd+bwd tokens/s",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "dtype": "bf16",
        "config": {"workload": f"{cfg.name}: T={cfg.tokens} H={cfg.hidden} E={cfg.num_experts} top{cfg.top_k} "
                               f"I={cfg.inter}, bf16 experts, fp32 router, fwd+bwd incl. router and all expert weight grads",
                   "tokens_per_step": cfg.tokens},
        "host_enqueue_ms_per_step": host_enqueue / steps * 1e3,
        "mfma_frac_of_peak_region": mfma_frac_region,
        "gemm_tflops_region": gemm_flops_step / (ms_per_step * 1e-3) / 1e12,
        "roofline": roof,
        # per-kernel table: from a separate, untimed pass with EVERY launch bracketed by HIP events, which
        # costs the stream about 5 % (so the entries add up to more than ms_per_step); only the dominant
        # kernel's entry and the roofline's launch time come from the timed region itself
        "kernels_ms_per_step": {k: round(v["ms_per_step"], 4) for k, v in sorted(kernels.items(), key=lambda kv: -kv[1]["ms_per_step"])},
        "kernels_ms_per_step_source": "untimed pass with every launch bracketed by HIP events (about 5 % slower than "
                                      "the timed region); the dominant kernel's entry is from the timed region",
        "gemm_kernels_tflops": {k: round(flops[k] / (v["avg_ms"] * 1e-3) / 1e12, 1) for k, v in gemm_kernels.items()},
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no collectives, run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    from piper_amd import _lib
    from piper_amd.configs import CFG3, CFG4

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    _lib.load()
    cfg = CFG3 if args.workload == "cfg3" else CFG4
    if args.copy_calibration:
        from piper_amd import ops
        n = 64 * 1024 * 1024
        src = torch.ones(n, device="cuda:0")
        dst = torch.zeros(n, device="cuda:0")
        for _ in range(3):
            ops.bucket_pack([src], [0], dst, accumulate=False)   # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst
    result = region_result(cfg, args.steps, args.warmup)
    result.update({"n_gpus": 1, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic"})
    if args.workload == "cfg3" and not args.no_cfg4:
        # the compute-bound configuration (16384 tokens, Zipf-skewed routing) in the same run
        c4 = region_result(CFG4, args.steps, args.warmup)
        result["cfg4"] = {k: c4[k] for k in ("value", "unit", "ms_per_step", "config", "mfma_frac_of_peak_region",
                                             "gemm_tflops_region", "roofline", "kernels_ms_per_step", "gemm_kernels_tflops")}
    if not args.no_accumulate:
        # the same step on a later microbatch of an iteration: the parameter gradients exist and the
        # weight-gradient kernels add to them (one more read of 3 x E x I x H gradients per step)
        acc = region_result(cfg, args.steps, args.warmup, accumulate=True)
        result["accumulate"] = {k: acc[k] for k in ("value", "unit", "ms_per_step", "mfma_frac_of_peak_region",
                                                    "gemm_tflops_region", "kernels_ms_per_step")}
        result["accumulate"]["vs_clearing_step"] = acc["ms_per_step"] / result["ms_per_step"]
    if not args.no_bucket:
        result["bucket"] = bench_bucket(max(5, args.steps), max(2, args.warmup))
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg)
        result["cpu_baseline"]["padded_bmm_cfg1"] = cpu_baseline_padded_bmm()
        if not args.no_bucket:
            result["bucket"]["cpu_baseline"] = cpu_baseline_bucket()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
