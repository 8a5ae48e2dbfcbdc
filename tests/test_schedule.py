"""Schedule directives (file format of src/schedule.py:6-99, order semantics of
src/directives.py:302-402 and examples/build_schedule.py:44-125) reduced to one device's task list.
The fixtures under tests/golden/schedule_*.json are schedule files in the reference's format,
written by piper_amd.schedule's own generators plus place / replicate / shard / split lines."""
import json
import os

import pytest

from piper_amd.schedule import (derive_schedule_info, device_tasks, load_schedule_directives, load_schedule_info,
                                one_f_one_b_order, stage_passes, validate_schedule_directives, zero_bubble_order)
from piper_amd.tasks import TaskType

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _short(passes):
    return " ".join(f"{ps}{mb}" + (f"@{pp}" if pp else "") for pp, mb, ps in passes)


def test_1f1b_file_gives_alternating_forward_backward_then_update():
    path = os.path.join(GOLDEN, "schedule_pp1_1f1b_mb4.json")
    info = load_schedule_info(path)
    assert info == {"name": "schedule_pp1_1f1b_mb4", "path": path, "num_stages": 1, "pp_degree": 1, "dp_degree": 1,
                    "num_microbatches": 4}
    d = load_schedule_directives(path)
    assert _short(stage_passes(d)) == "F0 B0 F1 B1 F2 B2 F3 B3"
    tasks = device_tasks(d, [["layer0", "layer1"]])
    names = [(t.type, t.ubid, t.mb) for t in tasks]
    assert names[:4] == [(TaskType.FWD, "layer0", 0), (TaskType.FWD, "layer1", 0),
                         (TaskType.BWD, "layer1", 0), (TaskType.BWD, "layer0", 0)]
    assert names[-1][0] is TaskType.UPD and len(names) == 4 * 4 + 1


def test_zero_bubble_file_splits_the_backward():
    d = load_schedule_directives(os.path.join(GOLDEN, "schedule_pp1_zerobubble_mb4.json"))
    # rank 0 defers nothing: every BI is followed by its BW (examples/build_schedule.py:108-116)
    assert _short(stage_passes(d)) == "F0 BI0 BW0 F1 BI1 BW1 F2 BI2 BW2 F3 BI3 BW3"
    types = [t.type for t in device_tasks(d)]
    assert types.count(TaskType.BWD_I) == 4 and types.count(TaskType.BWD_W) == 4 and TaskType.BWD not in types


def test_two_stage_zero_bubble_respects_rows_and_data_flow():
    d = load_schedule_directives(os.path.join(GOLDEN, "schedule_pp2_zerobubble_mb4.json"))
    passes = stage_passes(d)
    at = {op: i for i, op in enumerate(passes)}
    assert len(passes) == 2 * 4 * 3
    for mb in range(4):
        assert at[(0, mb, "F")] < at[(1, mb, "F")] < at[(1, mb, "BI")] < at[(0, mb, "BI")]
        for pp in range(2):
            assert at[(pp, mb, "BI")] < at[(pp, mb, "BW")]
    # every order row is kept as written
    for row in (x for x in d if x["op"] == "order"):
        seq = [at[(g[0]["PP"], g[0]["MB"], g[0]["PASS"])] for g in row["filters"]]
        assert seq == sorted(seq)
    # rank 1 holds each BW back by one BI (examples/build_schedule.py:84-118)
    row1 = [(g[0]["PASS"], g[0]["MB"]) for g in zero_bubble_order(2, 4)[1]["filters"]]
    assert row1 == [("F", 0), ("BI", 0), ("F", 1), ("BI", 1), ("BW", 0), ("F", 2), ("BI", 2), ("BW", 1),
                    ("F", 3), ("BI", 3), ("BW", 2), ("BW", 3)]


def test_1f1b_rows_of_a_four_rank_pipeline():
    rows = one_f_one_b_order(4, 6)
    for rank, row in enumerate(rows):
        cells = [(g[0]["PASS"], g[0]["MB"]) for g in row["filters"]]
        lead = 3 - rank
        assert cells[:lead] == [("F", m) for m in range(lead)]           # warm-up forwards
        assert [c for c in cells if c[0] == "F"] == [("F", m) for m in range(6)]
        assert [c for c in cells if c[0] == "B"] == [("B", m) for m in range(6)]
        # never more than lead + 1 microbatches in flight
        live = peak = 0
        for ps, _ in cells:
            live += 1 if ps == "F" else -1
            peak = max(peak, live)
        assert peak == lead + 1
    # on one device the four rows merge into a valid order
    passes = stage_passes(rows, 6)
    at = {op: i for i, op in enumerate(passes)}
    assert all(at[(p, m, "F")] < at[(p + 1, m, "F")] and at[(p + 1, m, "B")] < at[(p, m, "B")]
               for p in range(3) for m in range(6))


def test_groups_with_several_filters_and_wildcards():
    d = [{"op": "place", "filter": {"PP": 0}, "devices": [0]},
         {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": 2},
         {"op": "order", "filters": [[{"PP": 0, "PASS": "F"}], [{"PP": 0, "MB": "*", "PASS": "B"}]]}]
    assert _short(stage_passes(d)) == "F0 F1 B0 B1"
    d[2] = {"op": "order", "filters": [[{"PP": 0, "MB": 0, "PASS": "F"}],
                                       [{"PP": 0, "MB": 0, "PASS": "B"}, {"PP": 0, "MB": 1, "PASS": "F"}],
                                       [{"PP": 0, "MB": 1, "PASS": "B"}]]}
    assert _short(stage_passes(d)) == "F0 B0 F1 B1"


@pytest.mark.parametrize("bad, msg", [
    ({"not": "a list"}, "list of directives"),
    ([["x"]], "must be an object"),
    ([{"op": "teleport"}], "unsupported op"),
    ([{"op": "place", "devices": [0]}], "'filter'"),
    ([{"op": "place", "filter": {"PP": 0}, "filters": []}], "not 'filters'"),
    ([{"op": "order", "filters": []}], "non-empty list"),
    ([{"op": "order", "filters": [[]]}], "non-empty list"),
    ([{"op": "order", "filters": [["F"]]}], "filter object"),
    ([{"op": "split", "filter": {}, "num_microbatches": "__MBS__"}], "__MBS__"),
])
def test_file_format_errors(bad, msg):
    with pytest.raises(ValueError, match=msg):
        validate_schedule_directives(bad)


def test_schedule_info_errors():
    place0 = {"op": "place", "filter": {"PP": 0}, "devices": [0, 2]}
    split = {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": 2}
    assert derive_schedule_info([place0, {"op": "place", "filter": {"PP": 1}, "devices": [1, 3]}, split], "a/b/x.json") == \
        {"name": "x", "path": "a/b/x.json", "num_stages": 2, "pp_degree": 2, "dp_degree": 2, "num_microbatches": 2}
    with pytest.raises(ValueError, match="place directives"):
        derive_schedule_info([split])
    with pytest.raises(ValueError, match="split directive"):
        derive_schedule_info([place0])
    with pytest.raises(ValueError, match="without gaps"):
        derive_schedule_info([{"op": "place", "filter": {"PP": 1}, "devices": [0]}, split])
    with pytest.raises(ValueError, match="same number of devices"):
        derive_schedule_info([place0, {"op": "place", "filter": {"PP": 1}, "devices": [1]}, split])
    with pytest.raises(ValueError, match="disagree"):
        derive_schedule_info([place0, split, dict(split, num_microbatches=3)])
    with pytest.raises(ValueError, match="non-empty device list"):
        derive_schedule_info([{"op": "place", "filter": {"PP": 0}, "devices": []}, split])


def test_order_errors():
    def sched(*rows):
        return [{"op": "place", "filter": {"PP": 0}, "devices": [0]},
                {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": 2}] + \
               [{"op": "order", "filters": [[f] for f in row]} for row in rows]
    F0, B0 = {"PP": 0, "MB": 0, "PASS": "F"}, {"PP": 0, "MB": 0, "PASS": "B"}
    with pytest.raises(ValueError, match="contradictory"):
        stage_passes(sched([B0, F0]))                                    # backward before its forward
    with pytest.raises(ValueError, match="PASS must be"):
        stage_passes(sched([F0, {"PP": 0, "MB": 0, "PASS": "X"}]))
    with pytest.raises(ValueError, match="matches no pass"):
        stage_passes(sched([F0, {"PP": 0, "MB": 7, "PASS": "B"}]))
    with pytest.raises(ValueError, match="only PP, MB and PASS"):
        stage_passes(sched([F0, {"PP": 0, "EP": 0, "PASS": "B"}]))
    with pytest.raises(ValueError, match="at least 2 groups"):
        stage_passes(sched([F0]))
    BI0, BW0 = {"PP": 0, "MB": 0, "PASS": "BI"}, {"PP": 0, "MB": 0, "PASS": "BW"}
    with pytest.raises(ValueError, match="exactly one BI and one BW"):
        stage_passes(sched([F0, BI0]))
    with pytest.raises(ValueError, match="BI must come before BW"):
        stage_passes(sched([F0, BW0, BI0]))
    with pytest.raises(ValueError, match="same order directive"):
        stage_passes(sched([F0, BI0], [F0, BW0]))
    with pytest.raises(ValueError, match="duplicate BI"):
        stage_passes(sched([F0, BI0, BI0, BW0]))
    # a fused B entry for a cell that another row splits matches nothing
    with pytest.raises(ValueError, match="matches no pass"):
        stage_passes(sched([F0, BI0, BW0], [F0, B0]))
    with pytest.raises(ValueError, match="asked for 3"):
        stage_passes(sched([F0, B0]), 3)
    with pytest.raises(ValueError, match="stage_ubids"):
        device_tasks(sched([F0, B0]), [["a"], ["b"]])


def test_fixture_files_are_valid_json_schedules():
    for name in sorted(os.listdir(GOLDEN)):
        if name.startswith("schedule_") and name.endswith(".json"):
            with open(os.path.join(GOLDEN, name)) as fh:
                validate_schedule_directives(json.load(fh))
