"""Autograd wiring of the expert region and registration of the reference's operator.

Two ways in:

* ``expert_region(...)``: the whole region (gate -> top-k -> sort -> grouped SwiGLU with the permute
  fused into the operand load -> unpermute+combine) as ONE autograd node with a hand-written
  backward.  This is what ``piper_amd.moe.AnnotatedMoE`` runs.
* the piecewise operators the reference model code calls one by one
  (examples/models/qwen3.py:237-283): ``router``, ``reorder``, ``permute``, ``bmm_experts``,
  ``combine``.  ``bmm_experts`` is also registered as ``torch.ops.piper_artifact.bmm_experts`` with
  the reference's schema (examples/models/qwen3_bmm_experts_patch.py:63-72), so reference model
  code that looks the op up by name gets the HIP implementation.
"""
from __future__ import annotations

import torch

from . import ops

# --------------------------------------------------------------------------- piecewise operators


class _RouterFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w_gate, gate_bias, top_k, route_norm, route_scale):
        logits = ops.gate_logits(x, w_gate, gate_bias)
        top_scores, top_idx = ops.route_topk(logits, top_k, route_norm, route_scale)
        ctx.save_for_backward(x, w_gate, logits, top_idx)
        ctx.has_bias = gate_bias is not None
        ctx.cfg = (route_norm, route_scale)
        ctx.mark_non_differentiable(top_idx)
        return top_scores, top_idx

    @staticmethod
    def backward(ctx, d_scores, _d_idx):
        x, w_gate, logits, top_idx = ctx.saved_tensors
        route_norm, route_scale = ctx.cfg
        d_logits = ops.route_topk_bwd(logits, top_idx, d_scores, route_norm, route_scale)
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        d_w = torch.empty_like(w_gate) if need_dw else None
        d_b = torch.empty(w_gate.shape[0], dtype=torch.float32, device=x.device) if ctx.has_bias and ctx.needs_input_grad[2] else None
        d_x32 = ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=need_dx, d_w_gate=d_w, d_gate_bias=d_b)
        d_x = d_x32.to(x.dtype) if need_dx else None
        return d_x, d_w, d_b, None, None, None


def _sorted_tables(top_idx: torch.Tensor, num_experts: int):
    """(counts, starts, perm, inv_perm) of the counting sort of `top_idx`, computed once per routing
    result: the tables ride on the index tensor, and the inverse permutation rides on `perm`, so the
    piecewise operators that follow (reorder, permute backward, combine) launch no second sort."""
    # valid for this tensor object, these contents (autograd's version counter moves with every
    # in-place write) and this expert count; a view or a clone is another object and is sorted again
    key = (top_idx._version, int(num_experts))
    cached = getattr(top_idx, "_pk_sorted", None)
    if cached is None or cached[0] != key:
        tables = ops.sort_by_expert(top_idx, num_experts)
        tables[2]._pk_inverse = (tables[2]._version, tables[3])
        cached = (key, tables)
        top_idx._pk_sorted = cached
    return cached[1]


def _inverse_of(perm: torch.Tensor) -> torch.Tensor:
    """inv_perm for a permutation produced by `reorder` (cached there); any other permutation is
    inverted once and remembered on the tensor."""
    cached = getattr(perm, "_pk_inverse", None)
    if cached is None or cached[0] != perm._version:
        inv = torch.empty_like(perm)
        inv[perm.long()] = torch.arange(perm.numel(), dtype=perm.dtype, device=perm.device)
        cached = (perm._version, inv)
        perm._pk_inverse = cached
    return cached[1]


def router(x, w_gate, gate_bias=None, *, top_k: int, route_norm: bool, route_scale: float = 1.0):
    """(top_scores [T,K] f32, selected_experts_indices [T,K] i32, num_tokens_per_expert [E] i32).
    The call `self.router(x, self.expert_bias)` of qwen3.py:237-241.  The histogram is the one the
    counting sort produces (no host sync, no second pass over the indices)."""
    top_scores, top_idx = _RouterFn.apply(x, w_gate, gate_bias, top_k, route_norm, route_scale)
    counts = _sorted_tables(top_idx, w_gate.shape[0])[0]
    return top_scores, top_idx, counts


def reorder(top_scores: torch.Tensor, top_idx: torch.Tensor, num_experts: int):
    """The reorderer of qwen3.py:243-247.  Returns (top_scores_experts_sorted [A],
    token_indices_experts_sorted [A] i32, num_tokens_per_expert [E] i32)."""
    counts, _starts, perm, _inv = _sorted_tables(top_idx, num_experts)
    scores_sorted = top_scores.reshape(-1)[perm.long()]
    return scores_sorted, perm, counts


class _PermuteFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, perm, top_k):
        ctx.top_k = top_k
        ctx.save_for_backward(_inverse_of(perm))
        return ops.permute_fwd(x, perm, top_k)

    @staticmethod
    def backward(ctx, d_routed):
        (inv_perm,) = ctx.saved_tensors
        return ops.permute_bwd(d_routed, inv_perm, ctx.top_k), None, None


def permute(x: torch.Tensor, token_indices_experts_sorted: torch.Tensor, top_k: int) -> torch.Tensor:
    """routed_input = x[token_indices_experts_sorted // top_k]  (qwen3.py:250)."""
    return _PermuteFn.apply(x, token_indices_experts_sorted, top_k)


class _BmmExpertsFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, w1, w2, w3, x, num_tokens_per_expert):
        starts = ops.counts_to_starts(num_tokens_per_expert)
        y, g, u, h = ops.grouped_swiglu_fwd(x, w1, w2, w3, starts)
        # rows past sum(num_tokens_per_expert) belong to no expert: zeros, as in the reference
        # (qwen3_bmm_experts_patch.py:43); the kernels only write rows below starts[E]
        ops.zero_rows_from(y, starts[-1:])
        ctx.save_for_backward(w1, w2, w3, x, starts, g, u, h)
        ctx.params = (w1, w2, w3)
        return y

    @staticmethod
    def backward(ctx, d_y):
        w1, w2, w3, x, starts, g, u, h = ctx.saved_tensors
        d_x, d_g, d_u = ops.grouped_swiglu_dgrad(d_y, w1, w2, w3, g, u, starts)
        ops.zero_rows_from(d_x, starts[-1:])
        d_w1 = d_w2 = d_w3 = None
        if all(ctx.needs_input_grad[:3]) and _can_defer(*ctx.params):
            _queue_expert_wgrad(ctx.params, d_y, h, d_g, d_u, x, starts, None, 1, None)
        elif (_ACCUMULATE_INTO_GRAD and all(ctx.needs_input_grad[:3])
              and all(_accumulates_in_place(p) for p in ctx.params)):
            p1, p2, p3 = ctx.params
            ops.grouped_swiglu_wgrad(d_y, h, d_g, d_u, x, starts, w1.shape[0], d_w1=p1.grad, d_w2=p2.grad, d_w3=p3.grad,
                                     accumulate=True)
        elif any(ctx.needs_input_grad[:3]):
            d_w1, d_w2, d_w3 = ops.grouped_swiglu_wgrad(d_y, h, d_g, d_u, x, starts, w1.shape[0])
        return d_w1, d_w2, d_w3, d_x, None


def _queue_wgrad(params, wgrad) -> None:
    """Queue `wgrad(**buffers)` -> (d_w1, d_w2, d_w3) for the weight pass; it accumulates into the
    parameters' .grad, inside the kernel's epilogue when all three gradients exist already."""
    p1, p2, p3 = params

    def run():
        bufs = [_grad_target(p) for p in (p1, p2, p3)]
        if all(acc for _, acc in bufs):
            wgrad(d_w1=bufs[0][0], d_w2=bufs[1][0], d_w3=bufs[2][0], accumulate=True)
            return
        for p, g in zip((p1, p2, p3), wgrad()):
            if p.grad is None:
                p.grad = g
            else:
                p.grad += g

    _WGRAD_QUEUE.push(run)


def _queue_expert_wgrad(params, d_y, h, d_g, d_u, x, starts, perm, top_k, order, scaled=False) -> None:
    def wgrad(**kw):
        return ops.grouped_swiglu_wgrad(d_y, h, d_g, d_u, x, starts, params[0].shape[0], row_map=perm, row_map_div=top_k,
                                        expert_order=order, scaled=scaled, **kw)
    _queue_wgrad(params, wgrad)


def _traced_without_data(*tensors) -> bool:
    """True under fake-tensor propagation (Dynamo, make_fx) or on the meta device: the call is only
    asked for the output's shape, dtype and whether it takes part in autograd."""
    from torch._subclasses.fake_tensor import FakeTensor
    return any(t.is_meta or isinstance(t, FakeTensor) for t in tensors)


def _bmm_experts_shape_only(w1, w2, w3, x):
    out = torch.empty_like(x)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (w1, w2, w3, x)):
        out.requires_grad_(True)
    return out


def _bmm_experts_autograd(w1, w2, w3, x, num_tokens_per_expert):
    # The reference binds one traceable Python function to every dispatch key, the Autograd key
    # included (qwen3_bmm_experts_patch.py:67-75), so Dynamo's fake-tensor propagation runs this
    # kernel too: it must not touch device pointers then.
    if _traced_without_data(w1, w2, w3, x, num_tokens_per_expert):
        return _bmm_experts_shape_only(w1, w2, w3, x)
    return _BmmExpertsFn.apply(w1, w2, w3, x, num_tokens_per_expert)


def _bmm_experts_forward_only(w1, w2, w3, x, num_tokens_per_expert):
    if _traced_without_data(w1, w2, w3, x, num_tokens_per_expert):
        return torch.empty_like(x)
    starts = ops.counts_to_starts(num_tokens_per_expert)
    y = ops.grouped_swiglu_fwd(x, w1, w2, w3, starts)[0]
    ops.zero_rows_from(y, starts[-1:])
    return y


def _bmm_experts_meta(w1, w2, w3, x, num_tokens_per_expert):
    return torch.empty_like(x)


_LIBS = []


def register_reference_op() -> bool:
    """Define ``piper_artifact::bmm_experts`` (same schema as qwen3_bmm_experts_patch.py:63-65) on
    the CUDA(=HIP)/Autograd/Meta keys.  If the op already exists (the reference patch was imported
    first) only the CUDA and AutogradCUDA kernels are overridden.  Returns True when this call
    registered something."""
    if _LIBS:
        return False
    exists = hasattr(torch.ops, "piper_artifact") and hasattr(torch.ops.piper_artifact, "bmm_experts")
    if not exists:
        def_lib = torch.library.Library("piper_artifact", "DEF")
        def_lib.define(
            "bmm_experts(Tensor w1, Tensor w2, Tensor w3, Tensor x, Tensor num_tokens_per_expert) -> Tensor"
        )
        _LIBS.append(def_lib)
    impl = torch.library.Library("piper_artifact", "IMPL")
    impl.impl("bmm_experts", _bmm_experts_forward_only, "CUDA")
    impl.impl("bmm_experts", _bmm_experts_autograd, "AutogradCUDA")
    if not exists:
        impl.impl("bmm_experts", _bmm_experts_meta, "Meta")
    _LIBS.append(impl)
    return True


def bmm_experts(w1, w2, w3, x, num_tokens_per_expert):
    """Same call as the reference's ``bmm_experts`` (qwen3_bmm_experts_patch.py:78-87)."""
    register_reference_op()
    return torch.ops.piper_artifact.bmm_experts(w1, w2, w3, x, num_tokens_per_expert)


class _CombineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y_sorted, perm, top_scores):
        ctx.save_for_backward(y_sorted, perm, top_scores)
        return ops.combine_fwd(y_sorted, _inverse_of(perm), top_scores)

    @staticmethod
    def backward(ctx, d_out):
        y_sorted, perm, top_scores = ctx.saved_tensors
        d_y, d_scores = ops.combine_bwd(d_out, y_sorted, perm, top_scores)
        return d_y, None, d_scores


def combine(gathered_output, token_indices_experts_sorted, top_scores):
    """Unpermute scatter + fp32 weighted sum over k (qwen3.py:265-283), fused."""
    return _CombineFn.apply(gathered_output, token_indices_experts_sorted, top_scores)


# --------------------------------------------------------------------------- split backward
class WeightGradQueue:
    """Weight-gradient work postponed by a backward-input pass (Piper's BWD_I / BWD_W split,
    src/executors.py:353-476).  ``run()`` launches the postponed kernels and accumulates their
    results into ``param.grad`` as the reference's weight pass does (src/executors.py:333-343)."""

    def __init__(self):
        self._work = []

    def push(self, fn) -> None:
        self._work.append(fn)

    def __len__(self) -> int:
        return len(self._work)

    def run(self) -> None:
        work, self._work = self._work, []
        for fn in work:
            fn()


_WGRAD_QUEUE: WeightGradQueue | None = None


class defer_weight_grads:
    """Context manager: backward passes run inside it compute input gradients only; the weight
    gradients of leaf parameters are queued on the returned WeightGradQueue."""

    def __enter__(self) -> WeightGradQueue:
        global _WGRAD_QUEUE
        self._prev = _WGRAD_QUEUE
        _WGRAD_QUEUE = WeightGradQueue()
        return _WGRAD_QUEUE

    def __exit__(self, *exc) -> None:
        global _WGRAD_QUEUE
        _WGRAD_QUEUE = self._prev


_ACCUMULATE_INTO_GRAD = False


class accumulate_weight_grads:
    """Context manager for backward passes that accumulate into ``.grad`` (``torch.autograd.backward``
    / ``Tensor.backward``, the way the reference's executor runs a backward task,
    src/executors.py:257-296): inside it the fused expert region adds the gradients of leaf
    parameters whose ``.grad`` already exists to that buffer in the epilogue of the weight-gradient
    kernels and hands autograd no gradient for them, instead of writing fresh tensors that
    AccumulateGrad then adds in a separate pass over 3 x E x I x H elements.  Gradient accumulation
    over microbatches as in src/executors.py:333-343.  Not for ``torch.autograd.grad``, which must
    return the gradients and leave ``.grad`` alone."""

    def __enter__(self):
        global _ACCUMULATE_INTO_GRAD
        self._prev = _ACCUMULATE_INTO_GRAD
        _ACCUMULATE_INTO_GRAD = True
        return self

    def __exit__(self, *exc) -> None:
        global _ACCUMULATE_INTO_GRAD
        _ACCUMULATE_INTO_GRAD = self._prev


def _accumulates_in_place(p) -> bool:
    """A leaf whose existing .grad the kernels can add to directly."""
    if p is None or not (p.is_leaf and p.requires_grad):
        return False
    g = p.grad
    return g is not None and g.dtype == p.dtype and g.shape == p.shape and g.is_contiguous() and g.device == p.device


def _router_weight_grads(p_gate, p_bias, d_logits, x, w_gate) -> None:
    """d_w_gate (and d_gate_bias) added to / stored as the parameters' .grad."""
    # the gate weight and the bias may be at different points of their accumulation
    # (one of them cleared, the other not); the kernel has one flag for both
    have_w = p_gate.grad is not None
    have_b = p_bias is not None and p_bias.grad is not None
    if p_bias is None or have_w == have_b:
        gw = p_gate.grad if have_w else torch.empty_like(p_gate)
        gb = None
        if p_bias is not None:
            gb = p_bias.grad if have_b else torch.empty_like(p_bias, dtype=torch.float32)
        ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=False, d_w_gate=gw, d_gate_bias=gb, accumulate=have_w)
        p_gate.grad = gw
        if p_bias is not None:
            p_bias.grad = gb
        return
    gw = torch.empty_like(p_gate)
    gb = torch.empty_like(p_bias, dtype=torch.float32)
    ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=False, d_w_gate=gw, d_gate_bias=gb, accumulate=False)
    p_gate.grad = p_gate.grad.add_(gw) if have_w else gw
    p_bias.grad = p_bias.grad.add_(gb) if have_b else gb


def _can_defer(*params) -> bool:
    return _WGRAD_QUEUE is not None and all(p is None or (p.is_leaf and p.requires_grad) for p in params)


def _grad_target(p):
    """(buffer to accumulate into, accumulate flag) for a leaf parameter."""
    if p.grad is None:
        return None, False
    return p.grad, True


# --------------------------------------------------------------------------- fused region
# Measured on MI355X: running the weight gradient next to the input gradient gains ~1.5 % (both
# kernels are throughput-bound), so it is opt-in; per-kernel timings are only meaningful with it off.
_OVERLAP_WGRAD = False
_SIDE_STREAMS: dict = {}


def set_overlap_wgrad(on: bool) -> None:
    """Run the weight-gradient kernel on a second stream, concurrently with the input gradient."""
    global _OVERLAP_WGRAD
    _OVERLAP_WGRAD = bool(on)


def _side_stream(device) -> torch.cuda.Stream:
    """One extra default-priority stream per device for the weight-gradient kernel."""
    key = torch.device(device).index or 0
    st = _SIDE_STREAMS.get(key)
    if st is None:
        st = torch.cuda.Stream(device=device)
        _SIDE_STREAMS[key] = st
    return st



class _ExpertRegionFn(torch.autograd.Function):
    """x [T,H] -> out [T,H]; saves the routing tables and the SwiGLU pre-activations."""

    @staticmethod
    def forward(ctx, x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale, residual=None):
        E = w1.shape[0]
        logits = ops.gate_logits(x, w_gate, gate_bias)
        top_scores, top_idx = ops.route_topk(logits, top_k, route_norm, route_scale)
        _counts, starts, perm, inv_perm, order = ops.sort_by_expert(top_idx, E, with_order=True)
        y, g, u, h = ops.grouped_swiglu_fwd(x, w1, w2, w3, starts, row_map=perm, row_map_div=top_k)
        out = ops.combine_fwd(y, inv_perm, top_scores, residual)
        # the backward recomputes h from (g, u) and takes the score gradient from the d_h GEMM, so
        # neither h nor y outlives the forward
        ctx.save_for_backward(x, w_gate, w1, w2, w3, logits, top_scores, top_idx, starts, perm, inv_perm, g, u, order)
        ctx.cfg = (top_k, route_norm, route_scale, gate_bias is not None)
        ctx.params = (w_gate, gate_bias, w1, w2, w3)
        return out

    @staticmethod
    def backward(ctx, d_out):
        (x, w_gate, w1, w2, w3, logits, top_scores, top_idx, starts, perm, inv_perm, g, u, order) = ctx.saved_tensors
        top_k, route_norm, route_scale, has_bias = ctx.cfg
        E = w1.shape[0]
        need = ctx.needs_input_grad
        # combine backward folded into the d_h GEMM: d_out rows are gathered per routed row, the
        # score is applied in the epilogue; d_y below is d_out itself and h is score * h
        d_out = d_out.contiguous()
        d_y = d_out
        # shapes with a K-contiguous weight-gradient path get d_g, d_u and score*h transposed as well
        # (score*h only transposed): wgrad(...) below hides which of the two kernel pairs runs
        if ops.transposed_ld(perm.numel(), x.shape[1], g.shape[1], E, g.dtype) > 0:
            # With long experts d_g and d_u exist only as the transposed copies: the weight gradient
            # wants them that way, and the d_x GEMM reads its A operand from the same blocks.  With
            # short experts the row-major pair for the d_x GEMM is written as well.
            blocks_only = ops.dx_from_transposed_pays(perm.numel(), x.shape[1], g.shape[1], E, g.dtype)
            d_g, d_u, d_gT, d_uT, hsT, d_scores = ops.grouped_swiglu_dgrad_dh_scaled_t(d_out, perm, top_scores, w2, g, u, starts,
                                                                                       row_major=not blocks_only)
            h = None

            def input_grad():
                if blocks_only:
                    return ops.grouped_swiglu_dgrad_dx_t(d_gT, d_uT, w1, w3, starts, perm.numel())
                return ops.grouped_swiglu_dgrad_dx(d_g, d_u, w1, w3, starts)

            def wgrad(**kw):
                return ops.grouped_swiglu_wgrad_scaled_t(d_out, hsT, d_gT, d_uT, x, starts, E, row_map=perm,
                                                         row_map_div=top_k, expert_order=order, **kw)
            wgrad_inputs = (d_out, hsT, d_gT, d_uT)
        else:
            d_g, d_u, h, d_scores = ops.grouped_swiglu_dgrad_dh_scaled(d_out, perm, top_scores, w2, g, u, starts)

            def input_grad():
                return ops.grouped_swiglu_dgrad_dx(d_g, d_u, w1, w3, starts)

            def wgrad(**kw):
                return ops.grouped_swiglu_wgrad(d_y, h, d_g, d_u, x, starts, E, row_map=perm, row_map_div=top_k,
                                                expert_order=order, scaled=True, **kw)
            wgrad_inputs = (d_out, h, d_g, d_u)
        # The weight gradient (Piper's BWD_W) depends only on d_y, h, d_g, d_u and x; it runs on a
        # second stream next to the input gradient (BWD_I) so the two kernels fill each other's tails.
        d_w1 = d_w2 = d_w3 = None
        cur = torch.cuda.current_stream(x.device)
        defer = all(need[3:6]) and need[1] and _can_defer(*ctx.params)
        if defer:
            # backward-input pass: the weight gradients of the experts and of the router gate are
            # queued with the tensors they need and computed by the weight pass
            p_gate, p_bias = ctx.params[0], ctx.params[1]
            _queue_wgrad(ctx.params[2:], wgrad)
            d_xs = input_grad()
            d_logits = ops.route_topk_bwd(logits, top_idx, d_scores, route_norm, route_scale)
            d_x32 = ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=need[0], d_w_gate=None, d_gate_bias=None)
            d_x = ops.permute_bwd(d_xs, inv_perm, top_k, addend_f32=d_x32) if need[0] else None

            def run_router():
                _router_weight_grads(p_gate, p_bias, d_logits, x, w_gate)

            _WGRAD_QUEUE.push(run_router)
            return d_x, None, None, None, None, None, None, None, None, (d_out if need[9] else None)
        # backward into .grad with gradients already there (a later microbatch of an iteration): the
        # weight-gradient kernels add to them in their epilogues and autograd gets nothing to add
        experts_in_place = _ACCUMULATE_INTO_GRAD and all(need[3:6]) and all(_accumulates_in_place(p) for p in ctx.params[2:])
        p_gate, p_bias = ctx.params[0], ctx.params[1]
        gate_in_place = (_ACCUMULATE_INTO_GRAD and need[1] and _accumulates_in_place(p_gate)
                         and (p_bias is None or (need[2] and p_bias.is_leaf and p_bias.requires_grad)))
        side = _side_stream(x.device) if (need[3] or need[4] or need[5]) and _OVERLAP_WGRAD and not experts_in_place else None
        if experts_in_place:
            wgrad(d_w1=ctx.params[2].grad, d_w2=ctx.params[3].grad, d_w3=ctx.params[4].grad, accumulate=True)
        elif need[3] or need[4] or need[5]:
            if side is not None:
                side.wait_stream(cur)
                with torch.cuda.stream(side):
                    d_w1, d_w2, d_w3 = wgrad()
            else:
                d_w1, d_w2, d_w3 = wgrad()
        d_xs = input_grad()
        d_logits = ops.route_topk_bwd(logits, top_idx, d_scores, route_norm, route_scale)
        if gate_in_place:
            d_wg = d_b = None
            d_x32 = ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=need[0], d_w_gate=None, d_gate_bias=None)
            _router_weight_grads(p_gate, p_bias, d_logits, x, w_gate)
        else:
            d_wg = torch.empty_like(w_gate) if need[1] else None
            d_b = torch.empty(E, dtype=torch.float32, device=x.device) if (has_bias and need[2]) else None
            d_x32 = ops.gate_logits_bwd(d_logits, x, w_gate, need_dx=need[0], d_w_gate=d_wg, d_gate_bias=d_b)
        d_x = ops.permute_bwd(d_xs, inv_perm, top_k, addend_f32=d_x32) if need[0] else None
        if side is not None:
            cur.wait_stream(side)
            for t in wgrad_inputs:           # allocated on the current stream, read on the side stream
                t.record_stream(side)
            for t in (d_w1, d_w2, d_w3):     # allocated on the side stream, consumed on the current one
                t.record_stream(cur)
        return d_x, d_wg, d_b, d_w1, d_w2, d_w3, None, None, None, (d_out if need[9] else None)


# The fused region and the RMSNorm are torch.library operators too (namespace piper_amd), for the same
# reason the reference wraps its expert segment in one (qwen3_bmm_experts_patch.py:56-75): the model
# is captured by Dynamo with fullgraph=True (src/compile.py:273), which cannot look inside a
# function that launches kernels through a C ABI.  As graph nodes they are opaque calls whose
# output shape comes from the fake-tensor branch of their kernels.
_REGION_LIBS = []


def _expert_region_autograd(x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale, residual):
    ts = [t for t in (x, w_gate, gate_bias, w1, w2, w3, residual) if t is not None]
    if _traced_without_data(*ts):
        out = torch.empty_like(x)
        if torch.is_grad_enabled() and any(t.requires_grad for t in ts):
            out.requires_grad_(True)
        return out
    return _ExpertRegionFn.apply(x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale, residual)


def _expert_region_forward_only(x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale, residual):
    with torch.no_grad():
        return _expert_region_autograd(x, w_gate, gate_bias, w1, w2, w3, top_k, route_norm, route_scale, residual)


def _rmsnorm_autograd(x, weight, eps):
    if _traced_without_data(x, weight):
        out = torch.empty_like(x)
        if torch.is_grad_enabled() and (x.requires_grad or weight.requires_grad):
            out.requires_grad_(True)
        return out
    return _RMSNormFn.apply(x, weight, eps)


def _rmsnorm_forward_only(x, weight, eps):
    with torch.no_grad():
        return _rmsnorm_autograd(x, weight, eps)


def register_region_ops() -> bool:
    """Define ``piper_amd::expert_region`` and ``piper_amd::rmsnorm`` (done when this module is
    imported: a registration cannot happen inside a function Dynamo is tracing).  Returns True when
    this call registered them."""
    if _REGION_LIBS:
        return False
    lib = torch.library.Library("piper_amd", "DEF")
    lib.define("expert_region(Tensor x, Tensor w_gate, Tensor? gate_bias, Tensor w1, Tensor w2, Tensor w3, "
               "int top_k, bool route_norm, float route_scale, Tensor? residual) -> Tensor")
    lib.define("rmsnorm(Tensor x, Tensor weight, float eps) -> Tensor")
    for name, fwd, auto in (("expert_region", _expert_region_forward_only, _expert_region_autograd),
                            ("rmsnorm", _rmsnorm_forward_only, _rmsnorm_autograd)):
        lib.impl(name, fwd, "CUDA")
        lib.impl(name, auto, "AutogradCUDA")
        lib.impl(name, fwd, "Meta")
        # CPU tensors reach the kernels' own check and are refused there; fake CPU tensors get a shape
        lib.impl(name, fwd, "CPU")
        lib.impl(name, auto, "AutogradCPU")
    _REGION_LIBS.append(lib)
    return True


def expert_region(x, w_gate, gate_bias, w1, w2, w3, *, top_k: int, route_norm: bool, route_scale: float = 1.0,
                  residual=None):
    """The whole MoE expert region of AnnotatedMoE.forward (qwen3.py:233-289) on x [T,H].
    `residual` [T,H] is added to the result in the combine kernel."""
    return torch.ops.piper_amd.expert_region(x, w_gate, gate_bias, w1, w2, w3, int(top_k), bool(route_norm),
                                             float(route_scale), residual)


class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        y, rstd = ops.rmsnorm_fwd(x, weight, eps)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, d_y):
        x, weight, rstd = ctx.saved_tensors
        d_x, d_w = ops.rmsnorm_bwd(d_y, x, weight, rstd, need_dw=ctx.needs_input_grad[1])
        return (d_x if ctx.needs_input_grad[0] else None), d_w, None


def rmsnorm(x, weight, eps: float = 1e-6):
    """RMSNorm over the last dimension (the block's ffn_norm, qwen3.py:313-314)."""
    shape = x.shape
    return torch.ops.piper_amd.rmsnorm(x.reshape(-1, shape[-1]), weight, float(eps)).reshape(shape)


def moe_block(h, norm_weight, w_gate, gate_bias, w1, w2, w3, *, top_k: int, route_norm: bool,
              route_scale: float = 1.0, norm_eps: float = 1e-6):
    """h + moe(ffn_norm(h)) on h [T,H] (qwen3.py:313-314): RMSNorm kernel, expert region, residual
    added in the combine kernel."""
    return expert_region(rmsnorm(h, norm_weight, norm_eps), w_gate, gate_bias, w1, w2, w3, top_k=top_k,
                         route_norm=route_norm, route_scale=route_scale, residual=h)


register_region_ops()
