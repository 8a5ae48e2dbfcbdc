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


@dataclass
class ComputeExecutor:
    """Bucket forward/backward execution (src/executors.py:169-296)."""

    stages: StageStore

    def forward(self, ubid: Any, input_tensors: Any, compute_stream: torch.cuda.Stream | None = None) -> dict:
        bucket = self.stages.bucket(ubid)
        fwd_fn, fwd_args, input_idxs = bucket.forward_fn, bucket.forward_args, bucket.input_idxs
        if not isinstance(input_tensors, (list, tuple)):
            input_tensors = [input_tensors]
        for i, tensor in zip(input_idxs, input_tensors):
            if isinstance(tensor, (list, tuple)):
                tensor = tensor[0]
            if tensor.requires_grad:
                tensor = tensor.detach().requires_grad_(True)
            fwd_args[i] = tensor
        fwd_inputs = [fwd_args[i] for i in input_idxs]
        inp_with_grad = [t for t in fwd_inputs if t is not None and t.requires_grad]
        with torch.cuda.stream(compute_stream):
            output = fwd_fn(fwd_args)
        for i in input_idxs:
            fwd_args[i] = None
        out_list = list(output) if isinstance(output, tuple) else [output]
        possibly_detached = [
            t.detach().requires_grad_(True) if isinstance(t, torch.Tensor) and t.requires_grad else t
            for t in out_list
        ]
        out_with_grad = [t for t in out_list if isinstance(t, torch.Tensor) and t.requires_grad]
        return {
            "pre_detach_outs": out_list,
            "detached_outs": possibly_detached,
            "out_with_grad": out_with_grad,
            "send_output": output,
            "inp_with_grad": inp_with_grad,
            "fwd_inputs": fwd_inputs,
        }

    def backward(self, ubid: Any, mb_idx: int, outputs_or_loss: list, upstream_grads: Any,
                 pre_detach_outs: Any, detached_outs: Any, inp_with_grad: Any, out_with_grad: Any,
                 compute_stream: torch.cuda.Stream | None = None) -> dict | None:
        if pre_detach_outs is None:
            with torch.cuda.stream(compute_stream):
                if upstream_grads is not None:
                    torch.autograd.backward(outputs_or_loss, upstream_grads)
                else:
                    outputs_or_loss[0].backward()
        else:
            bwd_pairs = [
                (p, d.grad) for p, d in zip(pre_detach_outs, detached_outs)
                if isinstance(d, torch.Tensor) and d.requires_grad and d.grad is not None
            ]
            assert bwd_pairs, (
                f"BWD ubid={ubid} mb={mb_idx}: detached boundary has no tensors with a materialized grad"
            )
            with torch.cuda.stream(compute_stream):
                torch.autograd.backward([p for p, _ in bwd_pairs], [g for _, g in bwd_pairs])
        if inp_with_grad:
            output_grads = [t.grad for t in inp_with_grad if t.grad is not None]
            if output_grads:
                return {"send_output": output_grads}
        return None


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
        cs = self.compute_stream or torch.cuda.current_stream()
        ps = self.pack_stream or cs
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
                if task.ubid in self.stages.param_sharded_ubids and life.free_params_after:
                    self.params.free_full_params(task.ubid)
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
                    self._pack_after_backward(task.ubid, cs, ps, pack_events)
                if task.ubid in self.stages.param_sharded_ubids and life.free_params_after:
                    self.params.free_full_params(task.ubid)
            elif tt is TaskType.BWD_W:
                queue = self._wgrad_queues.pop((task.ubid, task.mb))
                with torch.cuda.stream(cs):
                    queue.run()
                if life.reduce_grads_after:
                    self._pack_after_backward(task.ubid, cs, ps, pack_events)
                if task.ubid in self.stages.param_sharded_ubids and life.free_params_after:
                    self.params.free_full_params(task.ubid)
            elif tt is TaskType.UPD:
                self._update(cs, pack_events)
            else:
                raise NotImplementedError(f"task {tt} is not a per-device task of this executor")
        return {"losses": losses}

    def _pack_after_backward(self, ubid, cs, ps, pack_events: dict) -> None:
        """Gradient pack on the second stream, ordered after the backward that produced the grads."""
        if ps is not cs:
            evt = torch.cuda.Event()
            evt.record(cs)
            ps.wait_event(evt)
        self.params.accumulate_zero_param_grads_to_flat(ubid, ps if ps is not cs else None)
        if ps is not cs:
            done = torch.cuda.Event()
            done.record(ps)
            pack_events[ubid] = done

    def _update(self, stream, pack_events: dict):
        """src/executors.py:1005-1034."""
        if self.params.has_zero_shard_optimizers():
            self.params.step_zero_shard_optimizers(stream, pack_events)
        for bucket in self.stages.buckets.values():
            if bucket.optimizer is not None:
                with torch.cuda.stream(stream):
                    bucket.optimizer.step()
        torch.cuda.synchronize()
