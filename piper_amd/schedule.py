"""Schedule directives -> the task list of one device.

A Piper schedule is a JSON list of directives (src/schedule.py:6-99, src/directives.py):

    {"op": "place" | "replicate" | "shard", "filter": {"PP": 0, ...}, "devices": [...], ...}
    {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": 4}
    {"op": "order", "filters": [[{"PP": 0, "MB": 0, "PASS": "F"}], [{"PP": 0, "MB": 0, "PASS": "B"}], ...]}

The reference lowers them onto a multi-device training DAG.  This module keeps the file format and
its validation and reduces the meaning to what one GPU can act on: `place` tells how many pipeline
stages there are, `split` how many microbatches, `order` the sequence of forward / backward passes;
device lists, streams and `shard` describe other GPUs and are checked for shape only; of
`replicate` the one field that also matters on a single device is `bucket_size` (MB,
src/directives.py:155-169,1620-1621): it cuts the matched stage into parameter buckets
(`stage_bucket_bytes`, `plan_stage_buckets`).  `device_tasks` turns the result into the `Task`
list that `StageExecutor.run` takes, with every stage of the file running on the one device.

PASS values (src/directives.py:23-33): "F" forward, "B" fused backward, "BI" backward-input,
"BW" backward-weight.  A (stage, microbatch) whose backward an order row names as BI / BW runs
split; it then needs exactly one BI and one BW, in the same row, BI first
(src/directives.py:345-402).
"""
from __future__ import annotations

import json
import os
import sys
from typing import Any, Sequence

from .tasks import TaskType

PASS_TO_TASK = {"F": TaskType.FWD, "B": TaskType.BWD, "BI": TaskType.BWD_I, "BW": TaskType.BWD_W}
_FILTER_OPS = ("place", "replicate", "shard", "split")
_ORDER_KEYS = ("PP", "MB", "PASS")
ANY = "*"


# ------------------------------------------------------------------------------- file format
def _check_directive(pos: int, d: Any) -> None:
    if not isinstance(d, dict):
        raise ValueError(f"schedule directive[{pos}] must be an object, got {type(d).__name__}")
    op = d.get("op")
    if op in _FILTER_OPS:
        if not isinstance(d.get("filter"), dict):
            raise ValueError(f"{op} directive[{pos}] needs an object field 'filter': {d}")
        if "filters" in d:
            raise ValueError(f"{op} directive[{pos}] takes 'filter', not 'filters': {d}")
        if op == "replicate" and d.get("bucket_size") is not None:
            try:
                mb = int(d["bucket_size"])
            except (TypeError, ValueError):
                raise ValueError(f"replicate directive[{pos}]: bucket_size must be a number of MB: {d}") from None
            if mb <= 0:
                raise ValueError(f"bucket_size must be > 0 MB, got {mb}")       # src/directives.py:565-566
        if op == "split" and d.get("num_microbatches") == "__MBS__":
            raise ValueError("split.num_microbatches must be a number in the schedule file; the '__MBS__' "
                             "placeholder is not supported")
    elif op == "order":
        groups = d.get("filters")
        if not isinstance(groups, list) or not groups:
            raise ValueError(f"order directive[{pos}] needs a non-empty list field 'filters': {d}")
        for g, group in enumerate(groups):
            if not isinstance(group, list) or not group:
                raise ValueError(f"order directive[{pos}] group[{g}] must be a non-empty list: {d}")
            for f, flt in enumerate(group):
                if not isinstance(flt, dict):
                    raise ValueError(f"order directive[{pos}] group[{g}][{f}] must be a filter object: {d}")
    else:
        raise ValueError(f"schedule directive[{pos}] has unsupported op {op!r}: {d}")


def validate_schedule_directives(directives: Any) -> list[dict]:
    if not isinstance(directives, list):
        raise ValueError(f"a schedule must be a list of directives, got {type(directives).__name__}")
    for pos, d in enumerate(directives):
        _check_directive(pos, d)
    return directives


def load_schedule_directives(path: str) -> list[dict]:
    """Read and shape-check a schedule file (src/schedule.py:6-22)."""
    with open(path, "r", encoding="utf-8") as fh:
        return validate_schedule_directives(json.load(fh))


def derive_schedule_info(directives: Sequence[dict], schedule_path: str = "") -> dict[str, Any]:
    """Stage count, pipeline / data-parallel degree and microbatch count of a schedule
    (src/schedule.py:29-76): every PP index 0..n-1 placed exactly on a device list of the same
    length, all split directives agreeing on the microbatch count."""
    placed: dict[int, tuple[int, ...]] = {}
    microbatches: int | None = None
    for d in directives:
        if not isinstance(d, dict):
            continue
        if d.get("op") == "place":
            flt = d.get("filter")
            stage = flt.get("PP") if isinstance(flt, dict) else None
            devices = d.get("devices", d.get("device"))
            if stage is None or not isinstance(devices, list) or not devices:
                raise ValueError(f"a place directive needs a PP filter and a non-empty device list: {d}")
            placed[int(stage)] = tuple(int(x) for x in devices)
        elif d.get("op") == "split":
            n = int(d.get("num_microbatches", 0))
            if n <= 0:
                raise ValueError(f"a split directive needs num_microbatches > 0: {d}")
            if microbatches not in (None, n):
                raise ValueError(f"split directives disagree on num_microbatches: {microbatches} and {n}")
            microbatches = n
    if not placed:
        raise ValueError("a schedule needs place directives with PP filters")
    if sorted(placed) != list(range(len(placed))):
        raise ValueError(f"PP indices must be 0..n-1 without gaps, got {sorted(placed)}")
    widths = {len(devs) for devs in placed.values()}
    if len(widths) != 1:
        raise ValueError(f"every PP stage must be placed on the same number of devices, got {placed}")
    if microbatches is None:
        raise ValueError("a schedule needs a split directive with num_microbatches")
    return {
        "name": os.path.splitext(os.path.basename(schedule_path))[0],
        "path": schedule_path,
        "num_stages": len(placed),
        "pp_degree": len(set(placed.values())),
        "dp_degree": widths.pop(),
        "num_microbatches": microbatches,
    }


def load_schedule_info(path: str) -> dict[str, Any]:
    return derive_schedule_info(load_schedule_directives(path), path)


# ------------------------------------------------------------------------------- bucket sizes
def _filter_matches_stage(flt: dict, stage: int) -> bool:
    """The tag match of src/directives.py:46-56 against the tag {PP: stage} of a whole stage: a
    filter that names another tag than PP selects part of a stage (an EP segment) and does not
    match the stage as such."""
    for key, want in flt.items():
        if key != "PP":
            return False
        if want != ANY and int(want) != stage:
            return False
    return True


def stage_bucket_bytes(directives: Sequence[dict], num_stages: int | None = None) -> list[int | None]:
    """Per pipeline stage: the parameter-bucket size in bytes that its `replicate` directive asks
    for (`bucket_size` MB x 1024 x 1024, src/directives.py:567), or None when no replicate
    directive with a bucket_size matches the stage (the stage then stays one bucket).  The last
    matching directive wins, as directives are applied in file order (src/directives.py:1607-1621)."""
    directives = validate_schedule_directives(list(directives))
    if num_stages is None:      # the stages that the place directives name
        placed = [int(d["filter"]["PP"]) for d in directives
                  if d.get("op") == "place" and d["filter"].get("PP", ANY) != ANY]
        num_stages = 1 + max(placed, default=0)
    out: list[int | None] = [None] * num_stages
    for d in directives:
        if d.get("op") != "replicate" or d.get("bucket_size") is None:
            continue
        for stage in range(num_stages):
            if _filter_matches_stage(d["filter"], stage):
                out[stage] = int(d["bucket_size"]) * 1024 * 1024
    return out


def plan_stage_buckets(directives: Sequence[dict], stage_node_param_bytes: Sequence[Sequence[Sequence[int]]]):
    """The compute buckets of every stage of a schedule.

    stage_node_param_bytes[p][i] lists the parameter sizes in bytes of compute node i of stage p (in
    placeholder order).  Returns (groups, stage_ubids): groups[p] holds the node indices of each
    bucket of stage p in execution order -- one bucket for a stage without `bucket_size`, the
    assignment of `planner.bucket_layers` otherwise -- and stage_ubids[p] the running bucket ids,
    ready for `device_tasks(..., stage_ubids=...)`."""
    from .planner import bucket_layers

    sizes = stage_bucket_bytes(directives, len(stage_node_param_bytes))
    groups, stage_ubids, next_id = [], [], 0
    for nodes, limit in zip(stage_node_param_bytes, sizes):
        g = [list(range(len(nodes)))] if limit is None else bucket_layers(nodes, limit)
        groups.append(g)
        stage_ubids.append(list(range(next_id, next_id + len(g))))
        next_id += len(g)
    return groups, stage_ubids


# ------------------------------------------------------------------------------- order rows
def _order_rows(directives: Sequence[dict]) -> list[list[list[dict]]]:
    """The order directives as rows of groups of filters over PP / MB / PASS."""
    rows = []
    for d in directives:
        if d.get("op") != "order":
            continue
        groups = d["filters"]
        if len(groups) < 2:
            raise ValueError(f"an order directive needs at least 2 groups: {d}")      # src/directives.py:308
        row = []
        for group in groups:
            clean = []
            for flt in group:
                extra = sorted(set(flt) - set(_ORDER_KEYS))
                if extra:
                    raise ValueError(f"order filter {flt} uses tags {extra}: one device schedules whole stage "
                                     "passes, so only PP, MB and PASS can be ordered")
                if "PASS" in flt and flt["PASS"] not in PASS_TO_TASK:
                    raise ValueError(f"order filter {flt}: PASS must be one of {sorted(PASS_TO_TASK)}")
                clean.append({k: (ANY if v == ANY else (v if k == "PASS" else int(v))) for k, v in flt.items()})
            row.append(clean)
        rows.append(row)
    return rows


def _split_backward_cells(rows) -> set[tuple[int, int]]:
    """(stage, microbatch) cells whose backward the rows split into BI and BW."""
    seen: dict[tuple, dict[str, tuple[int, int, int]]] = {}
    for r, row in enumerate(rows):
        for g, group in enumerate(row):
            for f, flt in enumerate(group):
                if flt.get("PASS") not in ("BI", "BW"):
                    continue
                if flt.get("PP", ANY) == ANY or flt.get("MB", ANY) == ANY:
                    raise ValueError(f"a split backward entry must name its PP and MB: {flt}")
                cell = seen.setdefault((flt["PP"], flt["MB"]), {})
                if flt["PASS"] in cell:
                    raise ValueError(f"duplicate {flt['PASS']} entry for PP={flt['PP']} MB={flt['MB']}")
                cell[flt["PASS"]] = (r, g, f)
    for (pp, mb), cell in seen.items():
        if set(cell) != {"BI", "BW"}:
            raise ValueError(f"PP={pp} MB={mb}: a split backward needs exactly one BI and one BW entry")
        if cell["BI"][0] != cell["BW"][0]:
            raise ValueError(f"PP={pp} MB={mb}: BI and BW must stand in the same order directive")
        if cell["BI"][1:] > cell["BW"][1:]:
            raise ValueError(f"PP={pp} MB={mb}: BI must come before BW")
    return set(seen)


def _matches(op: tuple[int, int, str], flt: dict) -> bool:
    return all(flt.get(key, ANY) in (ANY, val) for key, val in zip(_ORDER_KEYS, op))


def stage_passes(directives: Sequence[dict], num_microbatches: int | None = None) -> list[tuple[int, int, str]]:
    """All (stage, microbatch, PASS) passes of one iteration in the order one device runs them.

    Constraints: the data dependencies of a pipeline (a stage's forward after the previous stage's,
    its backward after its own forward and after the next stage's backward, BW after BI) and, for
    every order row, each group before the next.  Passes are then sorted by their depth in that
    graph -- the earliest time step a pipeline could run them, which is how the reference
    serialises a device's work (src/ordering.py:21-52) -- with ties going to the earlier row, the
    lower microbatch, forward before backward, the lower stage.  Without order directives this
    yields all forwards of a microbatch wave by wave; with the 1F1B row of a single stage it
    yields F0 B0 F1 B1 ... exactly as written."""
    directives = validate_schedule_directives(list(directives))
    rows = _order_rows(directives)
    declared = {int(d.get("num_microbatches", 0)) for d in directives if d.get("op") == "split"}
    if any(d.get("op") == "place" for d in directives):
        with_split = directives if declared else directives + [
            {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": num_microbatches or 0}]
        info = derive_schedule_info(with_split)
        stages, mbs = info["num_stages"], info["num_microbatches"]
    else:
        # order rows alone (what the schedule builders emit): stages are the PP values they name
        named = [flt["PP"] for row in rows for group in row for flt in group if flt.get("PP", ANY) != ANY]
        stages = 1 + max(named, default=0)
        if len(declared) > 1:
            raise ValueError(f"split directives disagree on num_microbatches: {sorted(declared)}")
        mbs = declared.pop() if declared else (num_microbatches or 0)
        if mbs <= 0:
            raise ValueError("the number of microbatches comes from a split directive or from the caller")
    if num_microbatches is not None and num_microbatches != mbs:
        raise ValueError(f"the schedule splits into {mbs} microbatches, the caller asked for {num_microbatches}")
    split_cells = _split_backward_cells(rows)

    ops: list[tuple[int, int, str]] = []
    for mb in range(mbs):
        for pp in range(stages):
            ops.append((pp, mb, "F"))
            ops += [(pp, mb, "BI"), (pp, mb, "BW")] if (pp, mb) in split_cells else [(pp, mb, "B")]
    index = {op: i for i, op in enumerate(ops)}
    preds: list[set[int]] = [set() for _ in ops]

    def bwd_in(pp, mb):
        return (pp, mb, "BI") if (pp, mb) in split_cells else (pp, mb, "B")

    for pp, mb, ps in ops:
        me = index[(pp, mb, ps)]
        if ps == "F" and pp > 0:
            preds[me].add(index[(pp - 1, mb, "F")])
        elif ps in ("B", "BI"):
            preds[me].add(index[(pp, mb, "F")])
            if pp + 1 < stages:
                preds[me].add(index[bwd_in(pp + 1, mb)])
        elif ps == "BW":
            preds[me].add(index[(pp, mb, "BI")])

    row_rank = {}                                     # op -> (row, position in the row)
    for r, row in enumerate(rows):
        earlier: list[int] = []
        pos = 0
        for group in row:
            here: list[int] = []
            for flt in group:
                hit = [index[op] for op in ops if _matches(op, flt)]
                if not hit:
                    raise ValueError(f"order filter {flt} matches no pass of this schedule "
                                     f"({stages} stages, {mbs} microbatches)")
                here += hit
            for i in here:
                preds[i].update(j for j in earlier if j != i)
                row_rank.setdefault(i, (r, pos))
                pos += 1
            earlier = here
    # longest-path depth; a cycle means the order rows contradict the data flow or each other
    depth = [-1] * len(ops)
    state = [0] * len(ops)

    def visit(i: int) -> int:
        if state[i] == 1:
            pp, mb, ps = ops[i]
            raise ValueError(f"the order directives are contradictory around PP={pp} MB={mb} PASS={ps}")
        if state[i] == 2:
            return depth[i]
        state[i] = 1
        depth[i] = 1 + max((visit(j) for j in preds[i]), default=-1)
        state[i] = 2
        return depth[i]

    limit = sys.getrecursionlimit()
    sys.setrecursionlimit(max(limit, 4 * len(ops) + 100))
    try:
        for i in range(len(ops)):
            visit(i)
    finally:
        sys.setrecursionlimit(limit)
    pass_rank = {"F": 0, "B": 1, "BI": 1, "BW": 2}
    far = (len(rows), 0)
    order = sorted(range(len(ops)), key=lambda i: (depth[i], row_rank.get(i, far), ops[i][1], pass_rank[ops[i][2]], ops[i][0]))
    return [ops[i] for i in order]


def device_tasks(directives: Sequence[dict], stage_ubids: Sequence[Sequence[Any]] | None = None,
                 num_microbatches: int | None = None) -> list:
    """The `Task` list for `StageExecutor.run`: every pass of `stage_passes` expanded to the buckets
    of its stage (forward in bucket order, backward in reverse), then one update.
    `stage_ubids[p]` lists the bucket ids of pipeline stage p; by default stage p is bucket p."""
    from .executor import Task

    passes = stage_passes(directives, num_microbatches)
    n_stages = 1 + max(pp for pp, _, _ in passes)
    if stage_ubids is None:
        stage_ubids = [[p] for p in range(n_stages)]
    if len(stage_ubids) != n_stages:
        raise ValueError(f"the schedule has {n_stages} stages, stage_ubids names {len(stage_ubids)}")
    tasks = []
    for pp, mb, ps in passes:
        buckets = list(stage_ubids[pp])
        if ps != "F":
            buckets.reverse()
        tasks += [Task(PASS_TO_TASK[ps], u, mb) for u in buckets]
    tasks.append(Task(TaskType.UPD))
    return tasks


# ------------------------------------------------------------------------------- generators
def _row_directive(pp: int, cells: Sequence[tuple[str, int]]) -> dict:
    return {"op": "order", "filters": [[{"PP": pp, "MB": mb, "PASS": ps}] for ps, mb in cells]}


def one_f_one_b_order(n_ranks: int, n_microbatches: int) -> list[dict]:
    """One order directive per pipeline rank for the 1F1B schedule (the schedule that
    examples/build_schedule.py:44-72 emits): rank r runs n_ranks-1-r forwards ahead, then every
    backward is preceded by the next forward while one is left."""
    return _steady_state_rows(n_ranks, n_microbatches, split=False)


def zero_bubble_order(n_ranks: int, n_microbatches: int) -> list[dict]:
    """The ZB-1 schedule (examples/build_schedule.py:75-125): as 1F1B with the backward split into
    BI and BW, rank r holding its BW passes back by r backward-input passes."""
    return _steady_state_rows(n_ranks, n_microbatches, split=True)


def _steady_state_rows(n_ranks: int, n_mbs: int, split: bool) -> list[dict]:
    if n_ranks <= 0 or n_mbs <= 0:
        raise ValueError("n_ranks and n_microbatches must be positive")
    rows = []
    for rank in range(n_ranks):
        lead = min(n_ranks - 1 - rank, n_mbs)              # forwards in flight before the first backward
        cells: list[tuple[str, int]] = [("F", mb) for mb in range(lead)]
        for mb in range(n_mbs):
            if lead + mb < n_mbs:
                cells.append(("F", lead + mb))
            cells.append(("BI" if split else "B", mb))
            if split and mb >= rank:
                cells.append(("BW", mb - rank))
        if split:
            cells += [("BW", mb) for mb in range(max(n_mbs - rank, 0), n_mbs)]
        rows.append(_row_directive(rank, cells))
    return rows
