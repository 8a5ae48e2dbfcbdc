"""Single-process, single-GPU executor with the task API of Piper's per-device runtime.

``ComputeExecutor.forward`` / ``.backward`` keep the signatures and the returned dictionaries of
the reference (src/executors.py:212-296).  ``StageExecutor.run`` is the one-device reduction of
``DagExecutor.run`` (src/executors.py:571-1003): it walks an ordered task list, runs compute tasks
on the compute stream, packs gradients into the ZeRO bucket after every backward task on a second
stream (event hand-off as in src/executors.py:592-596,769-772,866) and finishes with the update
task (src/executors.py:1005-1034).  Communication tasks are accepted and skipped: with one GPU
send/recv, all-to-all, all-reduce, reduce-scatter and all-gather have no peer.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Sequence

import torch

from . import functional as F_
from .bucket import ParamStorage, StageStore
from .planner import plan_zero_lifetimes
from .tasks import COMM_TASKS, TaskType


def _as_list(value) -> list:
    if isinstance(value, (list, tuple)):
        return list(value)
    return [value]


def _wants_grad(t) -> bool:
    return isinstance(t, torch.Tensor) and t.requires_grad


def _cut(t):
    """A leaf that shares t's storage: autograd stops here, and the leaf collects the gradient that
    the consumer's backward produces for t."""
    return t.detach().requires_grad_(True) if _wants_grad(t) else t


@dataclass
class ComputeExecutor:
    """Forward / backward of one bucket with the call contract of the reference's executor
    (src/executors.py:169-296): same arguments, same keys in the returned dictionaries."""

    stages: StageStore

    def forward(self, ubid: Any, input_tensors: Any, compute_stream: torch.cuda.Stream | None = None) -> dict:
        """Run the bucket's forward function on `compute_stream`.

        Each input that takes part in autograd enters as a fresh leaf, and each such output is handed
        on as a fresh leaf as well ("detached_outs"), so every bucket owns a closed autograd graph
        whose ends exchange gradients through `.grad`."""
        bucket = self.stages.bucket(ubid)
        args, slots = bucket.forward_args, list(bucket.input_idxs)
        leaves = []
        for value in _as_list(input_tensors)[:len(slots)]:
            # a producer may hand over its whole output list; the boundary tensor is its head
            leaves.append(_cut(_as_list(value)[0]))
        for slot, leaf in zip(slots, leaves):
            args[slot] = leaf
        fwd_inputs = [args[slot] for slot in slots]
        try:
            with torch.cuda.stream(compute_stream):
                result = bucket.forward_fn(args)
        finally:
            for slot in slots:            # activations must not stay alive inside the argument list
                args[slot] = None
        outs = _as_list(result)
        return {
            "pre_detach_outs": outs,
            "detached_outs": [_cut(t) for t in outs],
            "out_with_grad": [t for t in outs if _wants_grad(t)],
            "send_output": result,
            "inp_with_grad": [t for t in fwd_inputs if _wants_grad(t)],
            "fwd_inputs": fwd_inputs,
        }

    def backward(self, ubid: Any, mb_idx: int, outputs_or_loss: list, upstream_grads: Any,
                 pre_detach_outs: Any, detached_outs: Any, inp_with_grad: Any, out_with_grad: Any,
                 compute_stream: torch.cuda.Stream | None = None) -> dict | None:
        """Backward of one bucket.  Without `pre_detach_outs` the roots are `outputs_or_loss` (a loss,
        or outputs with explicit `upstream_grads`); with them, the roots are the bucket's own outputs
        and their gradients are whatever the consumer left in `.grad` of the detached copies.
        Returns {"send_output": input gradients} when the bucket has inputs that received one."""
        if pre_detach_outs is None:
            roots = list(outputs_or_loss) if upstream_grads is not None else [outputs_or_loss[0]]
            grads = upstream_grads
        else:
            roots, grads = [], []
            for produced, handed_on in zip(pre_detach_outs, detached_outs):
                if _wants_grad(handed_on) and handed_on.grad is not None:
                    roots.append(produced)
                    grads.append(handed_on.grad)
            if not roots:
                raise AssertionError(f"backward of bucket {ubid!r}, microbatch {mb_idx}: no output of the "
                                     "bucket received a gradient from its consumer")
        # the backward accumulates into .grad; the HIP operators add to gradients that exist
        # already (later microbatches of an iteration) inside their kernels
        with torch.cuda.stream(compute_stream), F_.accumulate_weight_grads():
            torch.autograd.backward(roots, grads)
        received = [t.grad for t in (inp_with_grad or ()) if t.grad is not None]
        return {"send_output": received} if received else None


@dataclass
class Task:
    """One entry of a per-device schedule: task type, bucket id, microbatch index."""

    type: TaskType
    ubid: Any = None
    mb: int = 0


def one_f_one_b(num_microbatches: int, ubids: Sequence[Any]) -> list[Task]:
    """The 1F1B order of a single pipeline rank: F0 B0 F1 B1 ... then one update
    (the pp_degree == 1 case of build_1f1b_schedule, examples/build_schedule.py:44-72).
    Forward visits the buckets in order, backward in reverse."""
    tasks: list[Task] = []
    for mb in range(num_microbatches):
        tasks += [Task(TaskType.FWD, u, mb) for u in ubids]
        tasks += [Task(TaskType.BWD, u, mb) for u in reversed(list(ubids))]
    tasks.append(Task(TaskType.UPD))
    return tasks


@dataclass
class StageExecutor:
    stages: StageStore
    params: ParamStorage = None
    compute: ComputeExecutor = None
    compute_stream: torch.cuda.Stream | None = None
    pack_stream: torch.cuda.Stream | None = None
    loss_fn: Any = None
    # the pack that follows a bucket's last backward of the iteration is folded into the optimizer
    # step (ParamStorage.hold_param_grads / FusedAdamW.step_packed)
    fuse_last_pack: bool = False
    _fwd: dict = field(default_factory=dict)
    _inp_grads: dict = field(default_factory=dict)
    _wgrad_queues: dict = field(default_factory=dict)

    def __post_init__(self):
        self.params = self.params or ParamStorage(self.stages)
        self.compute = self.compute or ComputeExecutor(self.stages)

    def run(self, tasks: Sequence[Task], microbatches: Sequence[Any], targets: Sequence[Any] | None = None) -> dict:
        """Run one training iteration.  ``microbatches[mb]`` feeds the first bucket's forward; each
        bucket's detached output feeds the next bucket; the last bucket's output goes to ``loss_fn``
        (or is summed when there is no loss_fn)."""
        caller = torch.cuda.current_stream()
        cs = self.compute_stream or caller
        ps = self.pack_stream or cs
        # the microbatches (and whatever else the caller queued) were produced on the caller's stream
        if cs != caller:
            cs.wait_stream(caller)
        if ps != caller and ps is not cs:
            ps.wait_stream(caller)
        self.params.drain_pending_frees()        # src/executors.py:584
        self._fwd.clear()
        self._inp_grads.clear()
        self._wgrad_queues.clear()
        losses = []
        pack_events: dict = {}
        self.params.clear_param_grads()
        self.params.zero_grad_buffers(ps)
        if ps is not cs:
            cs.wait_stream(ps)
        ubids = list(self.stages.buckets.keys())
        # which task gathers / frees a bucket's parameters and which one packs its gradients
        lifetimes = plan_zero_lifetimes(tasks)
        last_pack = {}          # bucket -> index of the task whose gradients are the last ones packed
        if self.fuse_last_pack:
            for ti, task in enumerate(tasks):
                if ti in lifetimes and lifetimes[ti].reduce_grads_after:
                    last_pack[task.ubid] = ti
        for ti, task in enumerate(tasks):
            tt = task.type
            life = lifetimes.get(ti)
            if tt in COMM_TASKS or tt is TaskType.ORDER_DUMMY:
                continue
            if tt is TaskType.FWD:
                pos = ubids.index(task.ubid)
                if pos == 0:
                    inp = microbatches[task.mb]
                else:
                    inp = self._fwd[(ubids[pos - 1], task.mb)]["detached_outs"]
                if task.ubid in self.stages.param_sharded_ubids and life.gather_params_before:
                    self.params.all_gather_full_params(task.ubid, cs)
                self._fwd[(task.ubid, task.mb)] = self.compute.forward(task.ubid, inp, cs)
                if life.free_params_after:
                    self._free_params_after(task.ubid, cs)
            elif tt in (TaskType.BWD, TaskType.FWD_BWD, TaskType.BWD_I):
                # BWD_I is the same walk with the weight gradients of the HIP operators queued
                # instead of computed (src/executors.py:353-411); BWD_W runs the queue (:413-476)
                split = tt is TaskType.BWD_I
                pos = ubids.index(task.ubid)
                rec = self._fwd.pop((task.ubid, task.mb))
                if task.ubid in self.stages.param_sharded_ubids and life.gather_params_before:
                    self.params.all_gather_full_params(task.ubid, cs)
                ctx = F_.defer_weight_grads() if split else None
                queue = ctx.__enter__() if split else None
                try:
                    if pos == len(ubids) - 1:
                        with torch.cuda.stream(cs):
                            out = rec["pre_detach_outs"][0]
                            if self.loss_fn is not None:
                                loss = self.loss_fn(out, None if targets is None else targets[task.mb])
                            else:
                                loss = out.float().sum()
                        losses.append(loss.detach())
                        self.compute.backward(task.ubid, task.mb, [loss], None, None, None,
                                              rec["inp_with_grad"], rec["out_with_grad"], cs)
                    else:
                        # the downstream bucket's input grads become the grads of this bucket's detached
                        # outputs (src/executors.py:826-842)
                        prev = self._inp_grads.pop((ubids[pos + 1], task.mb))
                        for d, g in zip(rec["detached_outs"], prev):
                            if isinstance(d, torch.Tensor) and d.requires_grad and g is not None:
                                d.grad = g
                        self.compute.backward(task.ubid, task.mb, rec["pre_detach_outs"], None, rec["pre_detach_outs"],
                                              rec["detached_outs"], rec["inp_with_grad"], rec["out_with_grad"], cs)
                finally:
                    if split:
                        ctx.__exit__(None, None, None)
                self._inp_grads[(task.ubid, task.mb)] = [
                    t.grad if (isinstance(t, torch.Tensor) and t.requires_grad) else None for t in rec["fwd_inputs"]]
                if split:
                    self._wgrad_queues[(task.ubid, task.mb)] = queue
                if life.reduce_grads_after:
                    self._pack_after_backward(task.ubid, cs, ps, pack_events, hold=last_pack.get(task.ubid) == ti)
                if life.free_params_after:
                    self._free_params_after(task.ubid, cs)
            elif tt is TaskType.BWD_W:
                queue = self._wgrad_queues.pop((task.ubid, task.mb))
                with torch.cuda.stream(cs):
                    queue.run()
                if life.reduce_grads_after:
                    self._pack_after_backward(task.ubid, cs, ps, pack_events, hold=last_pack.get(task.ubid) == ti)
                if life.free_params_after:
                    self._free_params_after(task.ubid, cs)
            elif tt is TaskType.UPD:
                self._update(cs, pack_events)
            else:
                raise NotImplementedError(f"task {tt} is not a per-device task of this executor")
        return {"losses": losses}

    def _free_params_after(self, ubid, cs) -> None:
        """Release the bucket's full parameters once the compute task just queued on `cs` has run
        (src/executors.py:769-774,876)."""
        if ubid not in self.stages.param_sharded_ubids:
            return
        evt = torch.cuda.Event()
        evt.record(cs)
        self.params.defer_free_full_params(ubid, evt)

    def _pack_after_backward(self, ubid, cs, ps, pack_events: dict, hold: bool = False) -> None:
        """Gradient pack on the second stream, ordered after the backward that produced the grads.
        hold: these are the bucket's last gradients of the iteration and the optimizer step, which
        runs on the compute stream, takes them as they are."""
        if hold:
            self.params.hold_param_grads(ubid, cs)
            return
        if ps is not cs:
            evt = torch.cuda.Event()
            evt.record(cs)
            ps.wait_event(evt)
        self.params.accumulate_zero_param_grads_to_flat(ubid, ps)
        if ps is not cs:
            done = torch.cuda.Event()
            done.record(ps)
            pack_events[ubid] = done
            if ubid in self.stages.grad_sharded_ubids:
                self.params.defer_free_full_grads(ubid, done)     # src/executors.py:719

    def _update(self, stream, pack_events: dict):
        """src/executors.py:1005-1034."""
        self.params.drain_pending_frees()
        if self.params.has_zero_shard_optimizers():
            self.params.step_zero_shard_optimizers(stream, pack_events)
        for bucket in self.stages.buckets.values():
            if bucket.optimizer is not None:
                with torch.cuda.stream(stream):
                    bucket.optimizer.step()
        torch.cuda.synchronize()
