"""ZeRO bucket path on one device: bucket layout, flatten, gradient packing, optimizer step,
unflatten.  Mirrors the runtime half of the reference -- ``BucketState`` / ``ParamStorage``
(src/runtime.py:64-99,202-495) and the flatten block of ``_load_stage`` (src/actor.py:517-601) --
with the same method names and arguments, so an executor written against the reference drives it
unchanged.  Differences, all from the benchmark definition: every tensor starts on a 256-byte
boundary, the optimizer state is an fp32 master bucket, packing is one kernel launch for all
tensors and the optimizer is one fused AdamW launch.

With one GPU dp_degree is 1: the shard is the whole bucket and reduce-scatter / all-gather are
identities, so ``reduce_scatter_grads`` aliases ``flat_grads``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Sequence

import logging

import torch

from . import ops
from .optim import FusedAdamW

BUCKET_ALIGN_BYTES = 256


@dataclass
class BucketState:
    """Loaded runtime state of one compute bucket (field names of src/runtime.py:64-99)."""

    forward_fn: Any = None
    forward_args: list = field(default_factory=list)
    forward_input_meta: list = field(default_factory=list)
    input_idxs: list = field(default_factory=list)
    param_idxs: list = field(default_factory=list)
    param_names: list = field(default_factory=list)
    optimizer: Any = None
    trainable_param_idxs: list = field(default_factory=list)
    activation_checkpoint_subgraph_count: int = 1

    flat_params: torch.Tensor | None = None          # param dtype; parameters are views of it
    flat_grads: torch.Tensor | None = None           # fp32
    shard_param: torch.Tensor | None = None
    shard_optimizer: Any = None
    reduce_scatter_grads: torch.Tensor | None = None
    param_shard_info: tuple | None = None            # (shard_start, shard_size, orig_numel)
    param_view_specs: list = field(default_factory=list)  # (param, offset, numel, shape)
    full_params_fresh: bool = False
    # Flat buffers for the parameters of this compute bucket that have another dtype than
    # flat_params (the fp32 router gate of a bf16 layer): BucketStates without a forward_fn that
    # ParamStorage zeroes, packs, unflattens and steps together with this one.  The reference has
    # no such field: its flatten concatenates the parameters of a bucket whatever their dtype
    # (src/actor.py:534).
    companions: list = field(default_factory=list)
    # Gradients of the last microbatch that were NOT packed (ParamStorage.hold_param_grads): one
    # entry per param_view_spec, consumed by the optimizer step, which adds them to the bucket's
    # gradient inside the AdamW kernel.
    pending_grads: list | None = None

    def with_companions(self) -> list:
        return [self] + list(self.companions)

    def weights(self) -> list:
        return [self.forward_args[i] for i in self.param_idxs if self.forward_args[i] is not None]

    def trainable_params(self) -> list:
        return [self.forward_args[i] for i in self.trainable_param_idxs if self.forward_args[i] is not None]


def plan_bucket(shapes: Sequence[Sequence[int]], elem_size: int, align_bytes: int = BUCKET_ALIGN_BYTES):
    """Element offsets of the tensors inside one bucket and the padded bucket length."""
    numels = [int(torch.Size(s).numel()) for s in shapes]
    return ops.bucket_plan(numels, elem_size, align_bytes)


def flatten_params(bucket: BucketState, params: Sequence[torch.nn.Parameter], *,
                   optim_class: Callable[..., Any] | None = None, align_bytes: int = BUCKET_ALIGN_BYTES,
                   dp_degree: int = 1, dp_rank: int = 0, grad_dtype: torch.dtype = torch.float32) -> BucketState:
    """The ZeRO flatten of src/actor.py:532-586: copy all parameters into one flat buffer, re-point
    each parameter at its view, allocate the fp32 gradient bucket and build the shard optimizer."""
    if dp_degree != 1 or dp_rank != 0:
        raise NotImplementedError("this build runs one GPU: dp_degree must be 1")
    params = list(params)
    if not params:
        raise ValueError("flatten_params: empty parameter list")
    dtype, device = params[0].dtype, params[0].device
    if any(p.dtype != dtype or p.device != device for p in params):
        raise ValueError("all parameters of a bucket must share dtype and device")
    esize = params[0].element_size()
    # offsets must be valid for the param-dtype bucket AND the fp32 buckets that share them
    offsets, padded = ops.bucket_plan([p.numel() for p in params], esize, align_bytes)
    orig_numel = (offsets[-1] + params[-1].numel()) if params else 0

    flat_params = torch.zeros(padded, dtype=dtype, device=device)
    ops.bucket_pack([p.detach() for p in params], offsets, flat_params, accumulate=False)
    view_specs = []
    for p, off in zip(params, offsets):
        n = p.numel()
        p.data = flat_params[off:off + n].view(p.shape)
        p.requires_grad_(True)  # gradients stay in the parameter dtype; the pack kernel widens them
        view_specs.append((p, off, n, tuple(p.shape)))

    shard_param = flat_params[0:padded]
    shard_param.requires_grad_(True)
    shard_param.grad_dtype = None  # accept the fp32 gradient bucket as .grad

    bucket.flat_params = flat_params
    bucket.flat_grads = torch.zeros(padded, dtype=grad_dtype, device=device)
    bucket.reduce_scatter_grads = bucket.flat_grads  # dp_degree == 1: reduce-scatter is the identity
    bucket.shard_param = shard_param
    bucket.shard_optimizer = (optim_class or FusedAdamW)([shard_param])
    bucket.param_shard_info = (0, padded, orig_numel)
    bucket.param_view_specs = view_specs
    bucket.full_params_fresh = True
    bucket.optimizer = None
    return bucket


@dataclass
class StageStore:
    buckets: dict = field(default_factory=dict)
    zero_managed_ubids: set = field(default_factory=set)
    param_sharded_ubids: set = field(default_factory=set)
    grad_sharded_ubids: set = field(default_factory=set)

    def bucket(self, ubid) -> BucketState:
        if ubid not in self.buckets:
            raise KeyError(f"unknown bucket id {ubid!r}")
        return self.buckets[ubid]

    def get_bucket(self, ubid):
        return self.buckets.get(ubid)


@dataclass
class RuntimeState:
    """The few fields of the reference's per-actor runtime record (src/runtime.py:102-200) that the
    bucket path reads.  One GPU: rank 0 of a data-parallel group of one."""

    device: Any = None
    dp_degree: int = 1
    dp_rank: int = 0
    global_rank: int = 0
    dp_group: Any = None


class _DeferredFree:
    """A release that has to wait for a GPU event (src/runtime.py:284-310).  The reference hands
    `evt.synchronize(); free()` to a one-thread pool and keeps the Future; here the release runs
    when somebody asks for the result, which is what every consumer of the Future does before it
    touches the buffer again (`wait_pending_free`, `drain_pending_frees`).  The host waits for the
    event only when the release returns memory (`frees_memory`): with a data-parallel group of one
    nothing is returned -- the bucket is only marked stale -- and blocking the host there would stop
    it from queueing work ahead of the GPU for no benefit."""

    def __init__(self, evt, release, frees_memory: bool = True):
        self._evt, self._release, self._frees_memory, self._done = evt, release, frees_memory, False

    def done(self) -> bool:
        return self._done or self._evt is None or self._evt.query()

    def result(self) -> None:
        if self._done:
            return
        if self._evt is not None and self._frees_memory:
            self._evt.synchronize()
        self._release()
        self._done = True


class ParamStorage:
    """ZeRO parameter and gradient storage of one device (src/runtime.py:202-495): same constructor
    arguments (runtime, stages, logger), same method names and arguments.  `ParamStorage(stages)` is
    accepted as a shorthand.  Differences that follow from running the one GPU's share with a
    data-parallel group of one: the shard is the whole bucket, so "freeing the full parameters"
    releases nothing and only marks the bucket stale, and gradients are packed although the
    reference skips the pack when dp_degree <= 1 (src/runtime.py:254)."""

    def __init__(self, runtime: Any = None, stages: "StageStore | None" = None, logger: Any = None,
                 grad_buffer_dtype: torch.dtype = torch.float32):
        if isinstance(runtime, StageStore) and stages is None:
            runtime, stages = None, runtime
        if stages is None:
            raise TypeError("ParamStorage needs the StageStore of its buckets")
        self.runtime = runtime if runtime is not None else RuntimeState()
        self.stages = stages
        self.logger = logger if logger is not None else logging.getLogger("piper_amd.bucket")
        self.grad_buffer_dtype = grad_buffer_dtype
        self.pending_param_frees: dict = {}
        self.pending_grad_frees: dict = {}

    # ---- deferred frees (src/runtime.py:231-247,284-310)
    def wait_pending_free(self, pending: dict, ubid) -> None:
        if ubid is None:
            return
        fut = pending.pop(ubid, None)
        if fut is not None:
            fut.result()

    def drain_pending_frees(self) -> None:
        for pending in (self.pending_param_frees, self.pending_grad_frees):
            futures = list(pending.values())
            pending.clear()
            for fut in futures:
                fut.result()

    def defer_free_full_params(self, ubid, evt) -> None:
        """Free the bucket's full parameters once `evt` has happened (the forward/backward that
        reads them was recorded before it)."""
        if ubid is None or ubid not in self.stages.param_sharded_ubids:
            return
        self.wait_pending_free(self.pending_param_frees, ubid)
        self.pending_param_frees[ubid] = _DeferredFree(evt, lambda: self.free_full_params(ubid), frees_memory=False)

    def defer_free_full_grads(self, ubid, evt) -> None:
        if ubid is None or ubid not in self.stages.grad_sharded_ubids:
            return
        self.wait_pending_free(self.pending_grad_frees, ubid)
        # the pack that recorded `evt` has already dropped the per-tensor gradients, and with a
        # data-parallel group of one the flat buffer is also the optimizer's shard gradient: after the
        # event nothing is left to release (a late `free_full_grads` would only wipe newer gradients)
        self.pending_grad_frees[ubid] = _DeferredFree(evt, lambda: None, frees_memory=False)

    def _all_states(self):
        for bucket in self.stages.buckets.values():
            yield from bucket.with_companions()

    def clear_param_grads(self) -> None:
        for bucket in self._all_states():
            for p, *_ in bucket.param_view_specs:
                p.grad = None

    def zero_grad_buffers(self, stream: torch.cuda.Stream | None = None) -> None:
        """src/runtime.py:223-229."""
        with torch.cuda.stream(stream):
            for bucket in self._all_states():
                if bucket.flat_grads is not None:
                    ops.bucket_zero(bucket.flat_grads)
                rs = bucket.reduce_scatter_grads
                if rs is not None and rs is not bucket.flat_grads:
                    ops.bucket_zero(rs)

    def accumulate_zero_param_grads_to_flat(self, ubid, stream: torch.cuda.Stream | None = None) -> None:
        """Gradient pack (src/runtime.py:249-282): flat[o:o+n] += grad.to(f32) for every tensor of
        the bucket in one launch, then drop the per-tensor grads."""
        if ubid is None or ubid not in self.stages.zero_managed_ubids:
            return
        if ubid in self.stages.grad_sharded_ubids:
            self.wait_pending_free(self.pending_grad_frees, ubid)
        for bucket in self.stages.bucket(ubid).with_companions():
            self._pack_one(bucket, stream)

    def _pack_one(self, bucket: BucketState, stream) -> None:
        specs = bucket.param_view_specs
        if not specs:
            return
        with torch.cuda.stream(stream):
            if bucket.flat_grads is None:
                bucket.flat_grads = torch.zeros(bucket.param_shard_info[1], dtype=self.grad_buffer_dtype,
                                                device=bucket.flat_params.device)
                bucket.reduce_scatter_grads = bucket.flat_grads
            by_dtype: dict = {}
            for param, offset, numel, _shape in specs:
                grad = param.grad
                if grad is None:
                    continue
                g = grad.detach()
                if stream is not None:
                    g.record_stream(stream)
                by_dtype.setdefault(g.dtype, ([], []))
                by_dtype[g.dtype][0].append(g.reshape(-1))
                by_dtype[g.dtype][1].append(offset)
            for grads, offs in by_dtype.values():
                ops.bucket_pack(grads, offs, bucket.flat_grads, accumulate=True)
            for param, *_ in specs:
                param.grad = None

    def hold_param_grads(self, ubid, stream: torch.cuda.Stream | None = None) -> None:
        """In place of the LAST accumulate_zero_param_grads_to_flat of an iteration: keep the
        per-tensor gradients of the bucket as they are and drop them from the parameters.  The
        optimizer step then reads them directly (FusedAdamW.step_packed), which saves writing them
        into the fp32 bucket and reading them back.  With an optimizer that has no step_packed the
        step packs them first."""
        if ubid is None or ubid not in self.stages.zero_managed_ubids:
            return
        for bucket in self.stages.bucket(ubid).with_companions():
            held = []
            for param, *_ in bucket.param_view_specs:
                g = param.grad
                if g is not None:
                    g = g.detach()
                    if stream is not None:
                        g.record_stream(stream)
                held.append(g)
                param.grad = None
            bucket.pending_grads = held

    def alloc_full_params(self, ubid) -> None:
        """Unflatten (src/runtime.py:312-352): make every parameter a view of the flat bucket."""
        self.wait_pending_free(self.pending_param_frees, ubid)
        for bucket in self.stages.bucket(ubid).with_companions():
            full = bucket.flat_params
            assert full is not None, f"alloc_full_params: missing flat_params buffer for ubid={ubid}"
            assert bucket.param_view_specs, f"alloc_full_params: missing param_view_specs for ubid={ubid}"
            for param, offset, numel, shape in bucket.param_view_specs:
                if param.data_ptr() != full.data_ptr() + offset * full.element_size():
                    param.data = full[offset:offset + numel].view(shape)
                param.requires_grad_(True)
            bucket.full_params_fresh = True

    def free_full_params(self, ubid) -> None:
        """One device keeps the only copy of the parameters, so there is nothing to release;
        the bucket is only marked stale (src/runtime.py:354-371)."""
        for bucket in self.stages.bucket(ubid).with_companions():
            bucket.full_params_fresh = False

    def alloc_full_grads(self, ubid, stream: torch.cuda.Stream | None = None) -> None:
        bucket = self.stages.bucket(ubid)
        self.wait_pending_free(self.pending_grad_frees, ubid)
        with torch.cuda.stream(stream):
            if bucket.flat_grads is None:
                bucket.flat_grads = torch.zeros(bucket.param_shard_info[1], dtype=self.grad_buffer_dtype,
                                                device=bucket.flat_params.device)
                bucket.reduce_scatter_grads = bucket.flat_grads

    def free_full_grads(self, ubid) -> None:
        for bucket in self.stages.bucket(ubid).with_companions():
            for param, *_ in bucket.param_view_specs:
                param.grad = None

    def all_gather_full_params(self, ubid, stream: torch.cuda.Stream | None = None) -> int:
        """dp_degree == 1: the shard is the whole bucket, so the gather moves no bytes."""
        self.alloc_full_params(ubid)
        return 0

    def has_zero_shard_optimizers(self) -> bool:
        return any(b.shard_optimizer is not None for b in self._all_states())

    def step_zero_shard_optimizers(self, stream: torch.cuda.Stream | None = None,
                                   reduce_scatter_events: dict | None = None) -> None:
        """src/runtime.py:454-484: wait for the gradient events, run each bucket's optimizer on its
        shard with the fp32 gradient bucket as .grad."""
        if stream is not None:
            for evt in (reduce_scatter_events or {}).values():
                stream.wait_event(evt)
        for bucket in self._all_states():
            opt = bucket.shard_optimizer
            if opt is None or bucket.reduce_scatter_grads is None:
                continue
            held, bucket.pending_grads = bucket.pending_grads, None
            with torch.cuda.stream(stream):
                if held is not None and hasattr(opt, "step_packed") and len({g.dtype for g in held if g is not None}) <= 1:
                    specs = bucket.param_view_specs
                    opt.step_packed(bucket.shard_param, held, [s[1] for s in specs], [s[2] for s in specs],
                                    bucket.reduce_scatter_grads)
                else:
                    if held is not None:      # an optimizer without the fused entry: pack first
                        for (param, *_), g in zip(bucket.param_view_specs, held):
                            param.grad = g
                        self._pack_one(bucket, stream)
                    bucket.shard_param.grad = bucket.reduce_scatter_grads
                    opt.step()
            bucket.shard_param.grad = None
            for param, *_ in bucket.param_view_specs:
                param.grad = None
