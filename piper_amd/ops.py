"""Tensor-level wrappers over the C ABI (include/piper_amd.h): shape checks, output allocation
through torch's caching allocator, launch on torch's current stream.  No autograd here
(see piper_amd.functional) and no CPU fallback: every function needs GPU tensors and the built
library.

Index tensors are int32 on the device (the reference carries int64; values are identical).
"""
from __future__ import annotations

import ctypes as C
from typing import Sequence

import torch

from . import _lib
from ._lib import call, current_stream, dtype_code, ptr, require_gpu


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


# ------------------------------------------------------------------------- routing
def gate_logits(x: torch.Tensor, w_gate: torch.Tensor, gate_bias: torch.Tensor | None = None) -> torch.Tensor:
    """logits[T,E] = x[T,H] @ w_gate[E,H]^T (+ bias) in fp32 (router gate, qwen3.py:237-241)."""
    require_gpu(x)
    _check(x.dim() == 2 and w_gate.dim() == 2 and x.shape[1] == w_gate.shape[1], "gate_logits: x [T,H], w_gate [E,H]")
    _check(w_gate.dtype == torch.float32, "gate_logits: the router gate is kept in float32")
    T, H = x.shape
    E = w_gate.shape[0]
    if gate_bias is not None:
        _check(gate_bias.dtype == torch.float32 and gate_bias.shape == (E,), "gate_logits: bias must be float32 [E]")
    x = x.contiguous()
    logits = torch.empty((T, E), dtype=torch.float32, device=x.device)
    ws_bytes = int(_lib.load().pk_gate_workspace_bytes(T, H, E))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes > 0 else None
    call("pk_gate_logits", ptr(x), dtype_code(x.dtype), ptr(w_gate.contiguous()), ptr(gate_bias), ptr(logits),
         T, H, E, ptr(ws), ws_bytes if ws is not None else 0, current_stream(x.device))
    return logits


def gate_logits_bwd(d_logits, x, w_gate, need_dx=True, d_w_gate=None, d_gate_bias=None, accumulate=False):
    """Returns d_x (fp32 [T,H]) or None; writes/accumulates d_w_gate / d_gate_bias in place when given."""
    require_gpu(d_logits)
    T, E = d_logits.shape
    H = x.shape[1]
    d_x = torch.empty((T, H), dtype=torch.float32, device=x.device) if need_dx else None
    ws = None
    if d_w_gate is not None:
        ws_bytes = int(_lib.load().pk_gate_bwd_workspace_bytes(T, H, E))
        if ws_bytes > 0:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    call("pk_gate_logits_bwd", ptr(d_logits.contiguous()), ptr(x.contiguous()), dtype_code(x.dtype), ptr(w_gate.contiguous()),
         ptr(d_x), ptr(d_w_gate), ptr(d_gate_bias), int(bool(accumulate)), T, H, E, ptr(ws),
         0 if ws is None else ws.numel(), current_stream(x.device))
    return d_x


def route_topk(logits: torch.Tensor, top_k: int, route_norm: bool, route_scale: float = 1.0):
    """fp32 softmax + top-k (ties -> lower expert index) + optional renorm.  Returns
    (top_scores f32 [T,K], top_idx i32 [T,K])."""
    require_gpu(logits)
    _check(logits.dim() == 2 and logits.dtype == torch.float32, "route_topk: logits must be float32 [T,E]")
    T, E = logits.shape
    logits = logits.contiguous()
    scores = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    idx = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    call("pk_route_topk", ptr(logits), T, E, top_k, int(bool(route_norm)), float(route_scale), ptr(scores), ptr(idx),
         current_stream(logits.device))
    return scores, idx


def route_topk_bwd(logits, top_idx, d_top_scores, route_norm: bool, route_scale: float = 1.0) -> torch.Tensor:
    require_gpu(logits)
    T, E = logits.shape
    K = top_idx.shape[1]
    d_logits = torch.empty_like(logits)
    call("pk_route_topk_bwd", ptr(logits.contiguous()), ptr(top_idx.contiguous()), ptr(d_top_scores.contiguous().float()),
         T, E, K, int(bool(route_norm)), float(route_scale), ptr(d_logits), current_stream(logits.device))
    return d_logits


def sort_by_expert(top_idx: torch.Tensor, num_experts: int, with_order: bool = False):
    """Stable counting sort of the flat (token, k) slots by expert id.
    Returns (counts [E], starts [E+1], perm [A], inv_perm [A]), all int32; with_order appends
    order [E], the experts by descending row count (a scheduling hint for the weight gradient)."""
    require_gpu(top_idx)
    _check(top_idx.dtype == torch.int32, "sort_by_expert: top_idx must be int32")
    flat = top_idx.contiguous().view(-1)
    A = flat.numel()
    dev = flat.device
    counts = torch.empty(num_experts, dtype=torch.int32, device=dev)
    starts = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(A, dtype=torch.int32, device=dev)
    inv_perm = torch.empty(A, dtype=torch.int32, device=dev)
    ws_bytes = _lib.load().pk_sort_workspace_bytes(A, num_experts)
    if ws_bytes < 0:
        raise RuntimeError(f"pk_sort_workspace_bytes failed: {_lib.status_string(ws_bytes)}")
    ws = torch.empty(max(int(ws_bytes), 4), dtype=torch.uint8, device=dev)
    order = torch.empty(num_experts, dtype=torch.int32, device=dev) if with_order else None
    call("pk_sort_by_expert", ptr(flat), A, num_experts, ptr(counts), ptr(starts), ptr(perm), ptr(inv_perm),
         ptr(order), ptr(ws), ws.numel(), current_stream(dev))
    if with_order:
        return counts, starts, perm, inv_perm, order
    return counts, starts, perm, inv_perm


def counts_to_starts(counts: torch.Tensor) -> torch.Tensor:
    """starts[E+1] (int32) = exclusive cumsum of num_tokens_per_expert (int32 or int64)."""
    require_gpu(counts)
    _check(counts.dtype in (torch.int32, torch.int64), "counts must be int32 or int64")
    E = counts.numel()
    starts = torch.empty(E + 1, dtype=torch.int32, device=counts.device)
    call("pk_counts_to_starts", ptr(counts.contiguous()), int(counts.dtype == torch.int64), E, ptr(starts),
         current_stream(counts.device))
    return starts


# ------------------------------------------------------------------------- permute / combine
def permute_fwd(x: torch.Tensor, perm: torch.Tensor, top_k: int) -> torch.Tensor:
    require_gpu(x)
    T, H = x.shape
    A = perm.numel()
    x = x.contiguous()
    routed = torch.empty((A, H), dtype=x.dtype, device=x.device)
    call("pk_permute_fwd", ptr(x), dtype_code(x.dtype), ptr(perm), ptr(routed), A, H, top_k, current_stream(x.device))
    return routed


def permute_bwd(d_routed: torch.Tensor, inv_perm: torch.Tensor, top_k: int, addend_f32: torch.Tensor | None = None) -> torch.Tensor:
    require_gpu(d_routed)
    A, H = d_routed.shape
    T = A // top_k
    d_routed = d_routed.contiguous()
    d_x = torch.empty((T, H), dtype=d_routed.dtype, device=d_routed.device)
    call("pk_permute_bwd", ptr(d_routed), dtype_code(d_routed.dtype), ptr(inv_perm), ptr(addend_f32), ptr(d_x),
         T, H, top_k, current_stream(d_routed.device))
    return d_x


def combine_fwd(y_sorted: torch.Tensor, inv_perm: torch.Tensor, top_scores: torch.Tensor,
                residual: torch.Tensor | None = None) -> torch.Tensor:
    """Unpermute + weighted combine; `residual` [T,H] (same dtype) is added to the rounded sum."""
    require_gpu(y_sorted)
    A, H = y_sorted.shape
    T, K = top_scores.shape
    _check(A == T * K, "combine_fwd: y_sorted rows must equal T*K")
    y_sorted = y_sorted.contiguous()
    if residual is not None:
        _check(residual.shape == (T, H) and residual.dtype == y_sorted.dtype, "combine_fwd: residual must be [T,H] in the dtype of y")
        residual = residual.contiguous()
    out = torch.empty((T, H), dtype=y_sorted.dtype, device=y_sorted.device)
    call("pk_combine_fwd", ptr(y_sorted), dtype_code(y_sorted.dtype), ptr(inv_perm), ptr(top_scores.contiguous()),
         ptr(residual), ptr(out), T, H, K, current_stream(y_sorted.device))
    return out


def rmsnorm_fwd(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last dimension of x [T,H].  Returns (y, rstd f32 [T])."""
    require_gpu(x)
    _check(x.dim() == 2 and weight.shape == (x.shape[1],) and weight.dtype == x.dtype, "rmsnorm_fwd: x [T,H], weight [H] in the dtype of x")
    T, H = x.shape
    x = x.contiguous()
    y = torch.empty_like(x)
    rstd = torch.empty(T, dtype=torch.float32, device=x.device)
    call("pk_rmsnorm_fwd", ptr(x), dtype_code(x.dtype), ptr(weight.contiguous()), float(eps), ptr(y), ptr(rstd), T, H,
         current_stream(x.device))
    return y, rstd


def rmsnorm_bwd(d_y: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor, *,
                d_x_addend: torch.Tensor | None = None, need_dw: bool = True, d_weight: torch.Tensor | None = None,
                accumulate: bool = False):
    """Returns (d_x, d_weight or None); d_x_addend is added to d_x in the same pass."""
    require_gpu(d_y)
    T, H = x.shape
    d_y, x = d_y.contiguous(), x.contiguous()
    d_x = torch.empty_like(x)
    ws = None
    if need_dw:
        if d_weight is None:
            _check(not accumulate, "rmsnorm_bwd: accumulate needs d_weight")
            d_weight = torch.empty_like(weight)
        ws = torch.empty(int(_lib.load().pk_rmsnorm_bwd_workspace_bytes(T, H)), dtype=torch.uint8, device=x.device)
    else:
        d_weight = None
    call("pk_rmsnorm_bwd", ptr(d_y), ptr(x), dtype_code(x.dtype), ptr(weight.contiguous()), ptr(rstd),
         ptr(None if d_x_addend is None else d_x_addend.contiguous()), ptr(d_x), ptr(d_weight), int(bool(accumulate)),
         T, H, ptr(ws), 0 if ws is None else ws.numel(), current_stream(x.device))
    return d_x, d_weight


def combine_bwd(d_out: torch.Tensor, y_sorted: torch.Tensor, perm: torch.Tensor, top_scores: torch.Tensor):
    require_gpu(d_out)
    A, H = y_sorted.shape
    T, K = top_scores.shape
    d_out = d_out.contiguous()
    d_y = torch.empty_like(y_sorted)
    d_scores = torch.empty((T, K), dtype=torch.float32, device=d_out.device)
    call("pk_combine_bwd", ptr(d_out), ptr(y_sorted.contiguous()), dtype_code(y_sorted.dtype), ptr(perm),
         ptr(top_scores.contiguous()), ptr(d_y), ptr(d_scores), A, H, K, current_stream(d_out.device))
    return d_y, d_scores


def zero_rows_from(buf: torch.Tensor, first_row: torch.Tensor) -> None:
    """buf[r] = 0 for r >= first_row[0]; first_row is a one-element int32 device tensor (no host sync)."""
    require_gpu(buf)
    _check(buf.dim() == 2 and buf.is_contiguous(), "zero_rows_from: contiguous [rows, width] buffer")
    _check(first_row.dtype == torch.int32 and first_row.numel() >= 1, "zero_rows_from: int32 device scalar")
    call("pk_zero_rows_from", ptr(buf), dtype_code(buf.dtype), ptr(first_row), buf.shape[0], buf.shape[1],
         current_stream(buf.device))


# ------------------------------------------------------------------------- grouped SwiGLU experts
def _expert_dims(w1, w2, w3):
    _check(w1.dim() == 3 and w2.dim() == 3 and w3.dim() == 3, "expert weights must be [E,I,H], [E,H,I], [E,I,H]")
    E, I, H = w1.shape
    _check(tuple(w3.shape) == (E, I, H) and tuple(w2.shape) == (E, H, I), "expert weight shapes disagree")
    return E, I, H


def grouped_swiglu_fwd(x_rows, w1, w2, w3, starts, *, row_map=None, row_map_div=1, num_rows=None):
    """Returns (y [A,H], g, u, h [A,I]).  With row_map, operand row p is x_rows[row_map[p] // row_map_div]."""
    require_gpu(x_rows)
    E, I, H = _expert_dims(w1, w2, w3)
    A = int(num_rows if num_rows is not None else (row_map.numel() if row_map is not None else x_rows.shape[0]))
    dt = x_rows.dtype
    _check(w1.dtype == dt and w2.dtype == dt and w3.dtype == dt, "expert weights and activations must share a dtype")
    dev = x_rows.device
    g = torch.empty((A, I), dtype=dt, device=dev)
    u = torch.empty((A, I), dtype=dt, device=dev)
    h = torch.empty((A, I), dtype=dt, device=dev)
    y = torch.empty((A, H), dtype=dt, device=dev)
    call("pk_grouped_swiglu_fwd", ptr(x_rows.contiguous()), ptr(row_map), row_map_div, ptr(w1.contiguous()),
         ptr(w2.contiguous()), ptr(w3.contiguous()), ptr(starts), ptr(g), ptr(u), ptr(h), ptr(y), A, H, I, E,
         dtype_code(dt), current_stream(dev))
    return y, g, u, h


def grouped_swiglu_dgrad(d_y, w1, w2, w3, g, u, starts):
    """Returns (d_x_sorted [A,H], d_g, d_u [A,I])."""
    require_gpu(d_y)
    E, I, H = _expert_dims(w1, w2, w3)
    A = d_y.shape[0]
    d_g = torch.empty_like(g)
    d_u = torch.empty_like(u)
    d_x = torch.empty((A, H), dtype=d_y.dtype, device=d_y.device)
    call("pk_grouped_swiglu_dgrad", ptr(d_y.contiguous()), ptr(w1.contiguous()), ptr(w2.contiguous()), ptr(w3.contiguous()),
         ptr(g), ptr(u), ptr(starts), ptr(d_g), ptr(d_u), ptr(d_x), A, H, I, E, dtype_code(d_y.dtype),
         current_stream(d_y.device))
    return d_x, d_g, d_u


def grouped_swiglu_dgrad_dh(d_y, w2, g, u, starts):
    """First half of the input gradient: (d_g, d_u) [A,I] from d_y."""
    require_gpu(d_y)
    E, H, I = w2.shape
    A = d_y.shape[0]
    d_g = torch.empty_like(g)
    d_u = torch.empty_like(u)
    call("pk_grouped_swiglu_dgrad_dh", ptr(d_y.contiguous()), ptr(w2.contiguous()), ptr(g), ptr(u), ptr(starts),
         ptr(d_g), ptr(d_u), A, H, I, E, dtype_code(d_y.dtype), current_stream(d_y.device))
    return d_g, d_u


def grouped_swiglu_dgrad_dh_scaled(d_out, perm, top_scores, w2, g, u, starts):
    """combine_bwd + grouped_swiglu_dgrad_dh in one GEMM launch, without the per-row d_y:
    returns (d_g, d_u, hs = score * h [A,I], d_scores [T,K] f32).  Sorted row r is flat slot perm[r] of
    top_scores [T,K] and token perm[r] // K of d_out [T,H]."""
    require_gpu(d_out)
    E, H, I = w2.shape
    A = perm.numel()
    T, K = top_scores.shape
    dev = d_out.device
    d_g = torch.empty_like(g)
    d_u = torch.empty_like(u)
    hs = torch.empty_like(g)
    d_scores = torch.empty((T, K), dtype=torch.float32, device=dev)
    ws_bytes = int(_lib.load().pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(A, I))
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device=dev)
    call("pk_grouped_swiglu_dgrad_dh_scaled", ptr(d_out.contiguous()), ptr(perm), K, ptr(top_scores.contiguous()),
         ptr(w2.contiguous()), ptr(g), ptr(u), ptr(starts), ptr(d_g), ptr(d_u), ptr(hs), ptr(d_scores), ptr(ws), ws_bytes,
         A, H, I, E, dtype_code(g.dtype), current_stream(dev))
    return d_g, d_u, hs, d_scores


def transposed_ld(A: int, H: int, I: int, E: int, dtype: torch.dtype) -> int:
    """Padded row count `ldt` of the transposed copies for the K-contiguous weight-gradient kernels
    (a multiple of 64; a copy is [ldt / 32, I, 32]), or 0 when the shape / dtype has no such path."""
    if dtype not in (torch.float32, torch.bfloat16):
        return 0
    return int(_lib.load().pk_grouped_swiglu_transposed_ld(A, H, I, E, dtype_code(dtype)))


def grouped_swiglu_dgrad_dh_scaled_t(d_out, perm, top_scores, w2, g, u, starts, row_major: bool = True):
    """grouped_swiglu_dgrad_dh_scaled with the outputs the weight gradient reads written transposed:
    returns (d_g, d_u [A,I], d_gT, d_uT, hsT [ldt/32, I, 32], d_scores [T,K] f32).  A transposed copy
    holds, for every block of 32 padded rows, the I columns with the block's 32 row values
    contiguous: element (column i, padded row r) sits at [r // 32, i, r % 32].  row_major=False:
    d_g and d_u are not written (None is returned for them); grouped_swiglu_dgrad_dx_t then takes
    the input gradient from the transposed copies."""
    require_gpu(d_out)
    E, H, I = w2.shape
    A = perm.numel()
    T, K = top_scores.shape
    dev = d_out.device
    ldt = transposed_ld(A, H, I, E, g.dtype)
    _check(ldt > 0, "grouped_swiglu_dgrad_dh_scaled_t: shape without a transposed path")
    d_g = torch.empty_like(g) if row_major else None
    d_u = torch.empty_like(u) if row_major else None
    d_gT, d_uT, hsT = (torch.empty((ldt // 32, I, 32), dtype=g.dtype, device=dev) for _ in range(3))
    d_scores = torch.empty((T, K), dtype=torch.float32, device=dev)
    ws_bytes = int(_lib.load().pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(A, I))
    ws = torch.empty(max(ws_bytes, 4) // 4, dtype=torch.float32, device=dev)
    call("pk_grouped_swiglu_dgrad_dh_scaled_t", ptr(d_out.contiguous()), ptr(perm), K, ptr(top_scores.contiguous()),
         ptr(w2.contiguous()), ptr(g), ptr(u), ptr(starts), ptr(d_g), ptr(d_u), ptr(d_gT), ptr(d_uT), ptr(hsT), ldt,
         ptr(d_scores), ptr(ws), ws_bytes, A, H, I, E, dtype_code(g.dtype), current_stream(dev))
    return d_g, d_u, d_gT, d_uT, hsT, d_scores


def grouped_swiglu_wgrad_scaled_t(d_out, hsT, d_gT, d_uT, x, starts, E, *, row_map, row_map_div,
                                  d_w1=None, d_w2=None, d_w3=None, accumulate=False, expert_order=None):
    """Weight gradients from the transposed outputs of grouped_swiglu_dgrad_dh_scaled_t."""
    require_gpu(d_out)
    I, ldt = hsT.shape[1], hsT.shape[0] * 32
    H = d_out.shape[1]
    A = row_map.numel()
    dt, dev = d_out.dtype, d_out.device
    if d_w1 is None:
        d_w1 = torch.empty((E, I, H), dtype=dt, device=dev)
        d_w2 = torch.empty((E, H, I), dtype=dt, device=dev)
        d_w3 = torch.empty((E, I, H), dtype=dt, device=dev)
        accumulate = False
    call("pk_grouped_swiglu_wgrad_scaled_t", ptr(d_out.contiguous()), ptr(hsT), ptr(d_gT), ptr(d_uT), ldt, ptr(x.contiguous()),
         ptr(row_map), row_map_div, ptr(starts), ptr(expert_order), ptr(d_w1), ptr(d_w2), ptr(d_w3), int(bool(accumulate)),
         A, H, I, E, dtype_code(dt), current_stream(dev))
    return d_w1, d_w2, d_w3


def dx_from_transposed_pays(A: int, H: int, I: int, E: int, dtype: torch.dtype) -> bool:
    """Whether the fused backward should leave out the row-major d_g / d_u and take d_x from the
    transposed copies (the library's own tuning hint)."""
    if dtype not in (torch.float32, torch.bfloat16):
        return False
    return bool(_lib.load().pk_grouped_swiglu_dx_from_transposed_pays(A, H, I, E, dtype_code(dtype)))


def grouped_swiglu_dgrad_dx_t(d_gT, d_uT, w1, w3, starts, num_rows: int):
    """d_x_sorted [A,H] = d_g . w1 + d_u . w3 with d_g, d_u given as the transposed copies of
    grouped_swiglu_dgrad_dh_scaled_t ([ldt/32, I, 32]); num_rows = A."""
    require_gpu(d_gT)
    E, I, H = w1.shape
    ldt = d_gT.shape[0] * 32
    _check(d_gT.shape == d_uT.shape and d_gT.shape[1] == I and d_gT.shape[2] == 32, "grouped_swiglu_dgrad_dx_t: [ldt/32, I, 32] copies")
    d_x = torch.empty((num_rows, H), dtype=d_gT.dtype, device=d_gT.device)
    call("pk_grouped_swiglu_dgrad_dx_t", ptr(d_gT), ptr(d_uT), ldt, ptr(w1.contiguous()), ptr(w3.contiguous()), ptr(starts),
         ptr(d_x), num_rows, H, I, E, dtype_code(d_gT.dtype), current_stream(d_gT.device))
    return d_x


def grouped_swiglu_dgrad_dx(d_g, d_u, w1, w3, starts):
    """Second half of the input gradient: d_x_sorted [A,H] = d_g . w1 + d_u . w3."""
    require_gpu(d_g)
    E, I, H = w1.shape
    A = d_g.shape[0]
    d_x = torch.empty((A, H), dtype=d_g.dtype, device=d_g.device)
    call("pk_grouped_swiglu_dgrad_dx", ptr(d_g), ptr(d_u), ptr(w1.contiguous()), ptr(w3.contiguous()), ptr(starts),
         ptr(d_x), A, H, I, E, dtype_code(d_g.dtype), current_stream(d_g.device))
    return d_x


def grouped_swiglu_wgrad(d_y, h, d_g, d_u, x_rows, starts, E, *, row_map=None, row_map_div=1,
                         d_w1=None, d_w2=None, d_w3=None, accumulate=False, expert_order=None, scaled=False):
    """Weight gradients.  Without d_w* buffers, fresh tensors are returned; with buffers and
    accumulate=True the kernel adds into them (gradient accumulation over microbatches).
    scaled=True: d_y is d_out [T,H], addressed through the row map like x_rows, and h is score * h
    (the outputs of grouped_swiglu_dgrad_dh_scaled)."""
    require_gpu(d_y)
    A, I = h.shape
    H = d_y.shape[1]
    _check(not scaled or row_map is not None, "scaled weight gradient needs the row map")
    dt, dev = d_y.dtype, d_y.device
    if d_w1 is None:
        d_w1 = torch.empty((E, I, H), dtype=dt, device=dev)
        d_w2 = torch.empty((E, H, I), dtype=dt, device=dev)
        d_w3 = torch.empty((E, I, H), dtype=dt, device=dev)
        accumulate = False
    call("pk_grouped_swiglu_wgrad_scaled" if scaled else "pk_grouped_swiglu_wgrad", ptr(d_y.contiguous()), ptr(h), ptr(d_g), ptr(d_u), ptr(x_rows.contiguous()),
         ptr(row_map), row_map_div, ptr(starts), ptr(expert_order), ptr(d_w1), ptr(d_w2), ptr(d_w3), int(bool(accumulate)),
         A, H, I, E, dtype_code(dt), current_stream(dev))
    return d_w1, d_w2, d_w3


# ------------------------------------------------------------------------- bucket path
def bucket_plan(numels: Sequence[int], elem_size: int, align_bytes: int = 256):
    """Host-only: element offsets of tensors laid out back to back with aligned starts.
    Returns (offsets list, padded_total)."""
    n = len(numels)
    arr_n = (C.c_int64 * max(n, 1))(*numels)
    arr_o = (C.c_int64 * max(n, 1))()
    total = _lib.load().pk_bucket_plan(arr_n, n, elem_size, align_bytes, arr_o)
    if total < 0:
        raise RuntimeError(f"pk_bucket_plan failed with status {total}: {_lib.status_string(total)}")
    return [int(arr_o[i]) for i in range(n)], int(total)


def _ptr_array(tensors: Sequence[torch.Tensor | None]):
    arr = (C.c_void_p * max(len(tensors), 1))()
    for i, t in enumerate(tensors):
        arr[i] = None if t is None else ptr(t)
    return arr


def bucket_pack(tensors: Sequence[torch.Tensor | None], offsets: Sequence[int], flat: torch.Tensor, accumulate: bool,
                numels: Sequence[int] | None = None) -> None:
    """flat[off_i : off_i+n_i] (+)= cast(tensors[i]) for every non-None tensor, in one launch."""
    require_gpu(flat)
    n = len(tensors)
    live = [t for t in tensors if t is not None]
    if not live:
        return
    src_dtype = live[0].dtype
    _check(all(t.dtype == src_dtype for t in live), "bucket_pack: tensors of one call must share a dtype")
    tensors = [None if t is None else t.contiguous() for t in tensors]
    if numels is None:
        numels = [0 if t is None else t.numel() for t in tensors]
    arr_p = _ptr_array(tensors)
    arr_o = (C.c_int64 * n)(*offsets)
    arr_n = (C.c_int64 * n)(*numels)
    call("pk_bucket_pack", arr_p, arr_o, arr_n, n, dtype_code(src_dtype), ptr(flat), dtype_code(flat.dtype),
         int(bool(accumulate)), current_stream(flat.device))


def bucket_unpack(flat: torch.Tensor, tensors: Sequence[torch.Tensor], offsets: Sequence[int]) -> None:
    """tensors[i][:] = cast(flat[off_i : off_i+n_i]) in one launch (tensors must be contiguous)."""
    require_gpu(flat)
    n = len(tensors)
    if n == 0:
        return
    dst_dtype = tensors[0].dtype
    _check(all(t.dtype == dst_dtype and t.is_contiguous() for t in tensors), "bucket_unpack: contiguous tensors of one dtype")
    arr_p = _ptr_array(tensors)
    arr_o = (C.c_int64 * n)(*offsets)
    arr_n = (C.c_int64 * n)(*[t.numel() for t in tensors])
    call("pk_bucket_unpack", ptr(flat), dtype_code(flat.dtype), arr_p, arr_o, arr_n, n, dtype_code(dst_dtype),
         current_stream(flat.device))


def bucket_zero(flat: torch.Tensor) -> None:
    require_gpu(flat)
    _check(flat.dtype == torch.float32, "bucket_zero: fp32 bucket expected")
    call("pk_bucket_zero", ptr(flat), flat.numel(), current_stream(flat.device))


def adamw_fused(master, exp_avg, exp_avg_sq, grad, *, step: int, lr: float, beta1: float, beta2: float, eps: float,
                weight_decay: float, shadow: torch.Tensor | None = None, grad_scale: float = 1.0,
                zero_grad: bool = False) -> None:
    """One fused AdamW step over the whole fp32 bucket (torch.optim.AdamW operation order)."""
    require_gpu(master)
    n = master.numel()
    for t in (master, exp_avg, exp_avg_sq, grad):
        _check(t.dtype == torch.float32 and t.numel() == n and t.is_contiguous(), "adamw_fused: fp32 contiguous buffers of equal size")
    if shadow is not None:
        _check(shadow.numel() == n and shadow.is_contiguous(), "adamw_fused: shadow must match the bucket")
    call("pk_adamw_fused", ptr(master), ptr(exp_avg), ptr(exp_avg_sq), ptr(grad), ptr(shadow),
         dtype_code(shadow.dtype) if shadow is not None else 0, n, float(lr), float(beta1), float(beta2), float(eps),
         float(weight_decay), int(step), float(grad_scale), int(bool(zero_grad)), current_stream(master.device))


def adamw_fused_packed(master, exp_avg, exp_avg_sq, flat_grad, grads: Sequence[torch.Tensor | None], offsets: Sequence[int],
                       numels: Sequence[int], *, step: int, lr: float, beta1: float, beta2: float, eps: float,
                       weight_decay: float, shadow: torch.Tensor | None = None, grad_scale: float = 1.0,
                       zero_grad: bool = False) -> None:
    """AdamW over the tensors of a bucket with the last gradient pack folded in: the gradient of a
    tensor is its slice of `flat_grad` (fp32, may be None) plus `grads[i]` (may be None), and the
    result equals bucket_pack(accumulate=True) followed by adamw_fused bit for bit."""
    require_gpu(master)
    n = len(grads)
    _check(len(offsets) == n and len(numels) == n, "adamw_fused_packed: one offset and element count per tensor")
    total = master.numel()
    for t in (master, exp_avg, exp_avg_sq):
        _check(t.dtype == torch.float32 and t.numel() == total and t.is_contiguous(), "adamw_fused_packed: fp32 contiguous buffers of equal size")
    if flat_grad is not None:
        _check(flat_grad.dtype == torch.float32 and flat_grad.numel() == total and flat_grad.is_contiguous(), "adamw_fused_packed: flat_grad must match the bucket")
    live = [g for g in grads if g is not None]
    gdtype = live[0].dtype if live else torch.bfloat16
    _check(all(g.dtype == gdtype for g in live), "adamw_fused_packed: gradients of one call must share a dtype")
    for g, off, num in zip(grads, offsets, numels):
        _check(off >= 0 and off + num <= total, "adamw_fused_packed: tensor outside the bucket")
        _check(g is None or g.numel() == num, "adamw_fused_packed: gradient size differs from the tensor's")
    if shadow is not None:
        _check(shadow.dtype == torch.bfloat16 and shadow.numel() == total and shadow.is_contiguous(), "adamw_fused_packed: bf16 shadow of the bucket's size")
    grads = [None if g is None else g.contiguous() for g in grads]
    arr_p = _ptr_array(grads)
    arr_o = (C.c_int64 * max(n, 1))(*offsets)
    arr_n = (C.c_int64 * max(n, 1))(*numels)
    call("pk_adamw_fused_packed", ptr(master), ptr(exp_avg), ptr(exp_avg_sq), ptr(flat_grad), arr_p, arr_o, arr_n, n,
         dtype_code(gdtype), ptr(shadow), dtype_code(shadow.dtype) if shadow is not None else 0, float(lr), float(beta1),
         float(beta2), float(eps), float(weight_decay), int(step), float(grad_scale), int(bool(zero_grad)),
         current_stream(master.device))
