"""Host-side planning of the ZeRO bucket path: which parameters share a bucket, and which task of a
per-device schedule opens and closes a bucket's parameter / gradient lifetime.  Integer logic only.

``plan_param_buckets`` follows the assignment stages of ``bucket_stage`` (src/bucket.py:66-128 and
the boundary merge of :250-269) on plain lists instead of an FX graph; the reference goes on to cut
the stage graph into one sub-module per bucket (:275-360), which here is the caller's business (a
stage is a list of callables, see ``bucket_layers``).  ``plan_zero_lifetimes`` is the one-device
reduction of ``_prune_zero_lifetime_metadata`` (src/zero.py:16-291): with a single GPU the
all-gather and the reduce-scatter move no bytes, what remains is which task unflattens / frees the
parameters and which one allocates / packs the gradients of a bucket.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Sequence

from .tasks import TaskType

DEFAULT_BUCKET_BYTES = 25 * 1024 * 1024      # src/bucket.py:20


@dataclass
class PlannedBucket:
    first_use: int            # index of the first compute node that reads a member
    last_use: int             # index of the last one
    members: list[int]        # parameter indices, in the order the buckets were merged

    @classmethod
    def of(cls, members: Sequence[int], use_ranges: Sequence[tuple[int, int]]) -> "PlannedBucket":
        return cls(min(use_ranges[i][0] for i in members), max(use_ranges[i][1] for i in members), list(members))

    def absorb(self, other: "PlannedBucket") -> None:
        """Join a bucket that starts no earlier than this one."""
        self.last_use = max(self.last_use, other.last_use)
        self.members += other.members


def _fill_by_bytes(sizes: Sequence[int], limit: int) -> list[list[int]]:
    """Cut the parameter sequence into runs: a run is closed in front of the parameter that would
    take it over `limit` bytes, unless the run holds no bytes yet (src/bucket.py:76-86)."""
    runs: list[list[int]] = [[]]
    used = 0
    for i, nbytes in enumerate(sizes):
        if used > 0 and used + nbytes > limit:
            runs.append([])
            used = 0
        runs[-1].append(i)
        used += nbytes
    return runs


def plan_param_buckets(sizes: Sequence[int], use_ranges: Sequence[tuple[int, int]] | None = None,
                       bucket_size_bytes: int = DEFAULT_BUCKET_BYTES,
                       cut_forbidden: Callable[[int, int], bool] | None = None) -> list[PlannedBucket]:
    """Assign parameters (given in placeholder order) to buckets.

    sizes[i]       bytes of parameter i
    use_ranges[i]  (first, last) index of the compute nodes that read parameter i; default (i, i)
    cut_forbidden  optional predicate (last_use of the earlier bucket, first_use of the later one) ->
                   True when the stage may not be cut there (the reference forbids cuts that an alias
                   of a parameter or a bfloat16_* cast crosses, src/bucket.py:250-269)

    The result equals the reference's assignment (src/bucket.py:76-128,250-269):
      * runs of consecutive parameters filled up to the byte threshold;
      * a parameter that is first read inside one run's span of compute nodes and last read inside
        another's leaves its run and stands alone;
      * what remains is ordered by first use, and neighbours whose spans overlap are joined;
      * neighbours are joined as well wherever the cut between them is forbidden.
    """
    n = len(sizes)
    if use_ranges is None:
        use_ranges = [(i, i) for i in range(n)]
    if len(use_ranges) != n:
        raise ValueError("plan_param_buckets: one use range per parameter")
    if bucket_size_bytes <= 0:
        raise ValueError("plan_param_buckets: bucket_size_bytes must be positive")
    if any(first > last for first, last in use_ranges):
        raise ValueError("plan_param_buckets: use range with first > last")
    if n == 0:
        return []

    runs = _fill_by_bytes(sizes, bucket_size_bytes)
    spans = [PlannedBucket.of(run, use_ranges) for run in runs]

    def home_run(node: int) -> int:
        """The first run whose span covers compute node `node` (run 0 when none does)."""
        return next((r for r, sp in enumerate(spans) if sp.first_use <= node <= sp.last_use), 0)

    straddlers = [i for i, (first, last) in enumerate(use_ranges) if home_run(first) != home_run(last)]
    loners = set(straddlers)
    groups = [[i for i in run if i not in loners] for run in runs] + [[i] for i in straddlers]
    pending = sorted((PlannedBucket.of(g, use_ranges) for g in groups if g), key=lambda b: b.first_use)

    joined: list[PlannedBucket] = []
    for bucket in pending:      # sorted() is stable: runs keep their order, loners follow them
        if joined and bucket.first_use <= joined[-1].last_use:
            joined[-1].absorb(bucket)
        else:
            joined.append(bucket)
    if cut_forbidden is None:
        return joined

    # A join never changes the first use of the left neighbour and takes over the last use of the
    # right one, so one sweep from the left sees every cut exactly as a repeated search would.
    final: list[PlannedBucket] = []
    for bucket in joined:
        if final and cut_forbidden(final[-1].last_use, bucket.first_use):
            final[-1].absorb(bucket)
        else:
            final.append(bucket)
    return final


def bucket_layers(layer_param_bytes: Sequence[Sequence[int]],
                  bucket_size_bytes: int = DEFAULT_BUCKET_BYTES) -> list[list[int]]:
    """Group the layers of a sequential stage into buckets: layer l reads its parameters at compute
    index l, so parameters of one layer always end up together.  Returns layer indices per bucket,
    in execution order."""
    sizes, ranges, owner = [], [], []
    for l, ps in enumerate(layer_param_bytes):
        for sz in ps:
            sizes.append(int(sz))
            ranges.append((l, l))
            owner.append(l)
    plan = plan_param_buckets(sizes, ranges, bucket_size_bytes)
    out: list[list[int]] = []
    covered: set[int] = set()
    for b in plan:
        layers = sorted({owner[i] for i in b.members})
        out.append(layers)
        covered.update(layers)
    # layers without parameters ride with the bucket before them (or the first one)
    for l in range(len(layer_param_bytes)):
        if l not in covered:
            if not out:
                out.append([])
            target = next((g for g in reversed(out) if g and g[0] < l), out[0])
            target.append(l)
            target.sort()
    return out


# ------------------------------------------------------------------------------------------------
@dataclass
class Lifetime:
    """What a compute task of a schedule has to do around its kernel launches."""
    gather_params_before: bool = False     # unflatten / all-gather the bucket's parameters
    free_params_after: bool = False
    alloc_grads_before: bool = False       # allocate / zero the full gradient buffer
    reduce_grads_after: bool = False       # pack (+ reduce-scatter) the gradients into the bucket
    chain: tuple = field(default_factory=tuple)   # indices of the tasks sharing the lifetime


_BACKWARD = (TaskType.BWD, TaskType.BWD_I, TaskType.BWD_W, TaskType.FWD_BWD)
_COMPUTE = (TaskType.FWD,) + _BACKWARD


def _chains(idxs: list[int], bucket_of: dict[int, Any], linked: Callable[[int, int], bool]) -> list[list[int]]:
    """Connected components, per bucket, of the direct-dependency relation restricted to `idxs`;
    each component in schedule order (src/zero.py:57-92)."""
    out: list[list[int]] = []
    by_bucket: dict[Any, list[int]] = {}
    for i in idxs:
        by_bucket.setdefault(bucket_of[i], []).append(i)
    for _, members in sorted(by_bucket.items(), key=lambda kv: str(kv[0])):
        seen: set[int] = set()
        for i in members:
            if i in seen:
                continue
            comp, stack = [], [i]
            seen.add(i)
            while stack:
                c = stack.pop()
                comp.append(c)
                for j in members:
                    if j not in seen and (linked(c, j) or linked(j, c)):
                        seen.add(j)
                        stack.append(j)
            out.append(sorted(comp))
    return out


def plan_zero_lifetimes(tasks: Sequence[Any], direct_deps: set[tuple[int, int]] | None = None) -> dict[int, Lifetime]:
    """For every compute task (by index into `tasks`) of a per-device schedule: the lifetime duties
    left after pruning.  Tasks need `.type`, `.ubid`, `.mb`.

    `direct_deps` holds (i, j) when task j directly depends on task i (data or temporal edge between
    two compute tasks).  When it is not given, the edges of a serial schedule are used: task j
    depends on the compute task right before it in the list, and on the forward / backward-input
    task of the same bucket and microbatch.

    Rule (src/zero.py:156-291): compute tasks of one bucket that are directly linked form a chain;
    gradient chains are built from the backward tasks, parameter chains from all compute tasks.  The
    head of a gradient chain allocates the gradients and its tail reduces them; the head of a
    parameter chain gathers the parameters and its tail frees them.
    """
    comp = [i for i, t in enumerate(tasks) if t.type in _COMPUTE]
    bucket_of = {i: tasks[i].ubid for i in comp}
    if direct_deps is None:
        direct_deps = set()
        for a, b in zip(comp, comp[1:]):
            direct_deps.add((a, b))
        producer: dict[tuple, int] = {}
        for i in comp:
            t = tasks[i]
            key = (t.ubid, t.mb)
            if t.type in (TaskType.FWD, TaskType.BWD_I, TaskType.FWD_BWD):
                if t.type is not TaskType.FWD and key in producer:
                    direct_deps.add((producer[key], i))
                producer[key] = i
            elif key in producer:
                direct_deps.add((producer[key], i))
    linked = lambda a, b: (a, b) in direct_deps

    out = {i: Lifetime() for i in comp}
    for chain in _chains([i for i in comp if tasks[i].type in _BACKWARD], bucket_of, linked):
        out[chain[0]].alloc_grads_before = True
        out[chain[-1]].reduce_grads_after = True
    for chain in _chains(comp, bucket_of, linked):
        out[chain[0]].gather_params_before = True
        out[chain[-1]].free_params_after = True
        for i in chain:
            out[i].chain = tuple(chain)
    return out
