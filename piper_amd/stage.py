"""From a schedule's ``bucket_size`` to the compute buckets of a stage.

In the reference a ``replicate`` directive may carry ``bucket_size`` (MB, src/directives.py:155-169);
the forward nodes it matches are then cut into parameter buckets by ``bucket_stage``
(src/directives.py:560-762, src/bucket.py:15-360), each bucket becoming a compute node of its own
with its own flat parameter / gradient buffers, so that the gradient pack (and, with several GPUs,
the reduce-scatter) of one bucket runs while the backward of the next one is still computing.

Here a stage is a sequence of compute nodes (``StageNode``: a callable and the parameters it
reads), the assignment is ``planner.bucket_layers`` -- the reference's greedy / promote / merge
rules with node i reading its parameters at compute index i -- and ``load_stage`` builds one
``BucketState`` per group with the ZeRO flatten of ``bucket.flatten_params``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Sequence

import torch

from .bucket import BucketState, StageStore, flatten_params
from .planner import DEFAULT_BUCKET_BYTES, bucket_layers


@dataclass
class StageNode:
    """One compute node of a sequential stage: ``fn(x, params) -> x`` with ``params`` the dict
    below (parameters in the order the node's graph would list them as placeholders)."""

    fn: Callable[[Any, dict], Any]
    params: dict = field(default_factory=dict)

    def param_bytes(self) -> list[int]:
        return [int(p.numel() * p.element_size()) for p in self.params.values()]


def plan_stage(nodes: Sequence[StageNode], bucket_size_bytes: int | None) -> list[list[int]]:
    """Node indices per bucket, in execution order.  ``None`` keeps the stage in one bucket (a
    ``replicate`` directive without ``bucket_size``, src/directives.py:1598-1606)."""
    if bucket_size_bytes is None:
        return [list(range(len(nodes)))]
    return bucket_layers([n.param_bytes() for n in nodes], bucket_size_bytes)


def load_stage(nodes: Sequence[StageNode], groups: Sequence[Sequence[int]], *, ubids: Sequence[Any] | None = None,
               optim_class: Callable[..., Any] | None = None, store: StageStore | None = None) -> StageStore:
    """One compute bucket per group: its forward runs the group's nodes back to back, its parameters
    are flattened into one ZeRO bucket per dtype (the dtype of the group's first parameter is the
    bucket's own, the others become companions) and re-pointed at their views.  Buckets are
    registered as ZeRO-managed and parameter-sharded, i.e. unflattened before use and packed
    after every backward, as a stage under ``replicate`` with ``shard_params`` is
    (src/actor.py:517-601)."""
    store = store if store is not None else StageStore()
    ubids = list(ubids) if ubids is not None else list(range(len(store.buckets), len(store.buckets) + len(groups)))
    if len(ubids) != len(groups):
        raise ValueError("load_stage: one bucket id per group")
    for ubid, group in zip(ubids, groups):
        members = [nodes[i] for i in group]
        names, plist, cuts = [], [], [0]
        for k, node in zip(group, members):
            for name, p in node.params.items():
                names.append(f"n{k}.{name}")
                plist.append(p)
            cuts.append(len(plist))
        b = BucketState()
        b.forward_args = [None] + plist
        b.input_idxs = [0]
        b.param_idxs = list(range(1, 1 + len(plist)))
        b.trainable_param_idxs = list(b.param_idxs)
        b.param_names = names

        def forward_fn(args, _members=members, _cuts=cuts):
            x = args[0]
            for node, lo, hi in zip(_members, _cuts, _cuts[1:]):
                x = node.fn(x, dict(zip(node.params.keys(), args[1 + lo:1 + hi])))
            return x

        b.forward_fn = forward_fn
        by_dtype: dict = {}
        for p in plist:
            by_dtype.setdefault(p.dtype, []).append(p)
        if by_dtype:
            main_dtype = plist[0].dtype
            flatten_params(b, by_dtype.pop(main_dtype), optim_class=optim_class)
            for ps in by_dtype.values():
                b.companions.append(flatten_params(BucketState(), ps, optim_class=optim_class))
        store.buckets[ubid] = b
        store.zero_managed_ubids.add(ubid)
        store.param_sharded_ubids.add(ubid)
    return store


__all__ = ["StageNode", "plan_stage", "load_stage", "DEFAULT_BUCKET_BYTES"]
