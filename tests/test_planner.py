"""Bucket assignment (src/bucket.py:66-128,250-269) and ZeRO lifetime duties (src/zero.py:156-291)
as host logic.  The greedy rule is pinned by the two properties that define it (no bucket can take
the next parameter; no bucket exceeds the threshold unless it is a single parameter), the later
stages by hand-worked cases and by invariants on random inputs."""
import random

import pytest

from piper_amd.executor import Task
from piper_amd.planner import bucket_layers, plan_param_buckets, plan_zero_lifetimes
from piper_amd.tasks import TaskType


def _members(plan):
    return [b.members for b in plan]


def test_greedy_hand_cases():
    assert _members(plan_param_buckets([10, 10, 10, 10], None, 25)) == [[0, 1], [2, 3]]
    # an oversized parameter sits alone; the next one opens a new bucket (src/bucket.py:80-84)
    assert _members(plan_param_buckets([30, 5, 5], None, 25)) == [[0], [1, 2]]
    # exactly the threshold still fits (the test is "> threshold")
    assert _members(plan_param_buckets([10, 15, 1], None, 25)) == [[0, 1], [2]]
    assert plan_param_buckets([], None, 25) == []
    # default threshold is 25 MiB
    mib = 1024 * 1024
    assert _members(plan_param_buckets([10 * mib, 10 * mib, 10 * mib])) == [[0, 1], [2]]


def test_greedy_is_pinned_by_its_two_properties():
    rng = random.Random(0)
    for _ in range(300):
        n = rng.randint(1, 40)
        sizes = [rng.randint(0, 60) for _ in range(n)]
        limit = rng.randint(1, 100)
        plan = plan_param_buckets(sizes, None, limit)
        flat = [i for b in plan for i in b.members]
        assert flat == list(range(n))                       # a partition, in order
        for k, b in enumerate(plan):
            total = sum(sizes[i] for i in b.members)
            # a parameter joins a bucket only if it fits, or if the bucket holds no bytes yet
            before = 0
            for i in b.members:
                assert before + sizes[i] <= limit or before == 0
                before += sizes[i]
            if k + 1 < len(plan):                            # maximal: the next parameter did not fit
                assert total + sizes[plan[k + 1].members[0]] > limit and total > 0


def test_overlapping_use_ranges_merge():
    # two buckets by size, but the first parameter is read again inside the second bucket's range
    plan = plan_param_buckets([20, 20], [(0, 2), (1, 3)], 25)
    assert _members(plan) == [[0, 1]] and (plan[0].first_use, plan[0].last_use) == (0, 3)
    # no overlap: stays split, sorted by first use even when the placeholder order is reversed
    plan = plan_param_buckets([20, 20], [(5, 6), (0, 1)], 25)
    assert _members(plan) == [[1], [0]]


def test_singleton_promotion_hand_case():
    # initial buckets {0,1} (uses 0..3) and {2,3} (uses 2..6); parameter 2 starts inside the first
    # bucket's range and ends in the second: it is promoted (src/bucket.py:103-108) and, spanning
    # both, pulls everything into one bucket at the merge
    plan = plan_param_buckets([10, 10, 10, 10], [(0, 0), (1, 3), (2, 6), (5, 5)], 20)
    assert _members(plan) == [[0, 1, 2, 3]]
    # promoted parameter that only bridges its neighbours' ranges partially
    plan = plan_param_buckets([10, 10, 10, 10, 10, 10], [(0, 0), (1, 1), (2, 2), (3, 3), (8, 8), (9, 9)], 20)
    assert _members(plan) == [[0, 1], [2, 3], [4, 5]]


def test_forbidden_cuts_merge_neighbours():
    sizes = [10] * 6
    plan = plan_param_buckets(sizes, None, 20)
    assert _members(plan) == [[0, 1], [2, 3], [4, 5]]
    # the cut after compute node 1 is crossed by an alias of a parameter: buckets 0 and 1 fuse
    plan = plan_param_buckets(sizes, None, 20, cut_forbidden=lambda last, first: last == 1)
    assert _members(plan) == [[0, 1, 2, 3], [4, 5]]
    plan = plan_param_buckets(sizes, None, 20, cut_forbidden=lambda last, first: True)
    assert _members(plan) == [[0, 1, 2, 3, 4, 5]]


def test_invariants_on_random_ranges():
    rng = random.Random(1)
    for _ in range(300):
        n = rng.randint(1, 30)
        sizes = [rng.randint(1, 50) for _ in range(n)]
        ranges = []
        for _ in range(n):
            lo = rng.randint(0, 40)
            ranges.append((lo, lo + rng.randint(0, 6)))
        plan = plan_param_buckets(sizes, ranges, rng.randint(10, 120))
        assert sorted(i for b in plan for i in b.members) == list(range(n))
        for b in plan:
            assert b.first_use == min(ranges[i][0] for i in b.members)
            assert b.last_use == max(ranges[i][1] for i in b.members)
        for a, b in zip(plan, plan[1:]):                     # execution order, disjoint ranges
            assert a.last_use < b.first_use


def test_bucket_layers():
    mib = 1024 * 1024
    # 4 layers of 3 x 6 MiB: two layers per 25 MiB bucket would be 36 MiB -> greedy cuts inside
    # layer 1, and the shared use index merges the pieces back: layers are never split
    groups = bucket_layers([[6 * mib] * 3] * 4)
    assert sorted(l for g in groups for l in g) == [0, 1, 2, 3]
    assert all(g == sorted(g) for g in groups) and all(a[-1] < b[0] for a, b in zip(groups, groups[1:]))
    assert bucket_layers([[1], [], [1]], 1) == [[0, 1], [2]]


def _t(kind, ubid, mb=0):
    return Task(getattr(TaskType, kind), ubid, mb)


def test_lifetimes_1f1b_single_bucket():
    tasks = [_t("FWD", 0, 0), _t("BWD", 0, 0), _t("FWD", 0, 1), _t("BWD", 0, 1), Task(TaskType.UPD)]
    lt = plan_zero_lifetimes(tasks)
    assert set(lt) == {0, 1, 2, 3}
    # one parameter chain over the four adjacent tasks of the bucket
    assert [lt[i].gather_params_before for i in range(4)] == [True, False, False, False]
    assert [lt[i].free_params_after for i in range(4)] == [False, False, False, True]
    # the backward tasks are not directly linked: each allocates and reduces its own gradients
    assert lt[1].alloc_grads_before and lt[1].reduce_grads_after
    assert lt[3].alloc_grads_before and lt[3].reduce_grads_after
    assert not lt[0].alloc_grads_before and not lt[0].reduce_grads_after


def test_lifetimes_two_buckets_and_split_backward():
    tasks = [_t("FWD", "a"), _t("FWD", "b"), _t("BWD_I", "b"), _t("BWD_I", "a"), _t("BWD_W", "b"), _t("BWD_W", "a")]
    lt = plan_zero_lifetimes(tasks)
    # bucket b: FWD(1) - BWD_I(2) adjacent, BWD_W(4) linked to BWD_I by its data edge
    assert lt[1].chain == (1, 2, 4) and lt[1].gather_params_before and lt[4].free_params_after
    # bucket a: FWD(0) - BWD_I(3) through the saved activations, BWD_W(5) through BWD_I
    assert lt[0].chain == (0, 3, 5) and lt[0].gather_params_before and lt[5].free_params_after
    # gradients: allocated before the input pass, packed after the weight pass
    assert lt[2].alloc_grads_before and not lt[2].reduce_grads_after
    assert lt[4].reduce_grads_after and not lt[4].alloc_grads_before
    assert lt[3].alloc_grads_before and lt[5].reduce_grads_after


def test_lifetimes_adjacent_backwards_share_one_reduction():
    tasks = [_t("FWD", 0, 0), _t("FWD", 0, 1), _t("BWD", 0, 1), _t("BWD", 0, 0)]
    lt = plan_zero_lifetimes(tasks)
    assert lt[2].alloc_grads_before and not lt[2].reduce_grads_after
    assert lt[3].reduce_grads_after and not lt[3].alloc_grads_before
    # explicit edges override the serial default: no link between the two backward tasks
    lt = plan_zero_lifetimes(tasks, direct_deps={(0, 1), (1, 2), (0, 3)})
    assert lt[2].reduce_grads_after and lt[3].reduce_grads_after


def test_assignment_equals_the_restated_reference_rule_on_random_inputs():
    """plan_param_buckets against oracle.planner.assign_buckets (a line-by-line restatement of
    src/bucket.py:76-128) on 20,000 random (sizes, use ranges, threshold): the same buckets with the
    same spans in the same execution order.  Inside a bucket that the merge stage joined, the
    member order may differ (the reference uses it for a log line only, src/bucket.py:133-141), so
    members are compared as sets."""
    from oracle.planner import assign_buckets

    rng = random.Random(1234)
    reordered = 0
    for case in range(20000):
        n = rng.randint(1, 14)
        sizes = [rng.choice((0, 1, 3, 7, 10, 25, 40)) if rng.random() < 0.7 else rng.randint(0, 60) for _ in range(n)]
        limit = rng.randint(1, 80)
        nodes = rng.randint(1, 12)
        ranges = []
        for _ in range(n):
            a = rng.randrange(nodes)
            b = a if rng.random() < 0.6 else rng.randrange(a, nodes)
            ranges.append((a, b))
        if rng.random() < 0.3:      # the common case: parameters in the order their nodes use them
            ranges.sort()
        got = plan_param_buckets(sizes, ranges, limit)
        want = assign_buckets(sizes, ranges, limit)
        assert [(b.first_use, b.last_use, sorted(b.members)) for b in got] == [(f, l, sorted(m)) for f, l, m in want], \
            (case, sizes, ranges, limit)
        reordered += any(b.members != m for b, (_, _, m) in zip(got, want))
    assert reordered < 20000 // 4


def test_hand_cases_pin_the_restated_rule_itself():
    """The hand-worked cases above, put to oracle.planner.assign_buckets directly (parameter i used
    by node i alone where the case gives no use ranges), so that the checker does not rest on its
    agreement with the product alone."""
    from oracle.planner import assign_buckets

    def members(sizes, ranges, limit):
        ranges = ranges if ranges is not None else [(i, i) for i in range(len(sizes))]
        return [sorted(m) for _, _, m in assign_buckets(sizes, ranges, limit)]

    assert members([10, 10, 10, 10], None, 25) == [[0, 1], [2, 3]]
    assert members([30, 5, 5], None, 25) == [[0], [1, 2]]
    assert members([10, 15, 1], None, 25) == [[0, 1], [2]]
    assert members([20, 20], [(0, 2), (1, 3)], 25) == [[0, 1]]
    assert members([20, 20], [(5, 6), (0, 1)], 25) == [[1], [0]]
    assert members([10, 10, 10, 10], [(0, 0), (1, 3), (2, 6), (5, 5)], 20) == [[0, 1, 2, 3]]
    assert members([10] * 6, [(0, 0), (1, 1), (2, 2), (3, 3), (8, 8), (9, 9)], 20) == [[0, 1], [2, 3], [4, 5]]
    spans = [(f, l) for f, l, _ in assign_buckets([20, 20], [(0, 2), (1, 3)], 25)]
    assert spans == [(0, 3)]


def test_bucket_size_of_a_schedule_cuts_the_stage():
    """replicate.bucket_size (MB) -> bytes per stage -> node groups -> bucket ids for device_tasks."""
    from piper_amd.schedule import device_tasks, plan_stage_buckets, stage_bucket_bytes

    mib = 1024 * 1024
    sched = [
        {"op": "place", "filter": {"PP": 0}, "devices": [0]},
        {"op": "place", "filter": {"PP": 1}, "devices": [1]},
        {"op": "replicate", "filter": {"PP": 0}, "devices": [0, 2], "reduce_stream": "dp_stream", "bucket_size": 2},
        {"op": "replicate", "filter": {"PP": 1}, "devices": [1, 3]},
        {"op": "shard", "filter": {"PP": 0, "EP": "*"}, "devices": [0, 2]},
        {"op": "split", "filter": {}, "dim_name": "MB", "num_microbatches": 2},
    ]
    assert stage_bucket_bytes(sched) == [2 * mib, None]
    # stage 0: four nodes of 1.5 MiB of parameters each -> one node per bucket; stage 1 stays whole
    node = [mib, mib // 2]
    groups, ubids = plan_stage_buckets(sched, [[node] * 4, [node] * 3])
    assert groups == [[[0], [1], [2], [3]], [[0, 1, 2]]]
    assert ubids == [[0, 1, 2, 3], [4]]
    tasks = device_tasks(sched, stage_ubids=ubids)
    fwd0 = [t.ubid for t in tasks if t.type is TaskType.FWD and t.mb == 0]
    bwd0 = [t.ubid for t in tasks if t.type is TaskType.BWD and t.mb == 0]
    assert fwd0 == [0, 1, 2, 3, 4] and bwd0 == [4, 3, 2, 1, 0]
    # a wildcard stage filter reaches every stage, a later directive overrides an earlier one
    both = sched + [{"op": "replicate", "filter": {"PP": "*"}, "devices": [0, 1], "bucket_size": 100}]
    assert stage_bucket_bytes(both) == [100 * mib, 100 * mib]
    # a filter on part of a stage (an EP segment) does not set the stage's bucket size
    ep = [sched[0], {"op": "replicate", "filter": {"PP": 0, "EP": 0}, "devices": [0], "bucket_size": 7}]
    assert stage_bucket_bytes(ep) == [None]
    for bad in (0, -3, "x"):
        with pytest.raises(ValueError):
            stage_bucket_bytes([sched[0], {"op": "replicate", "filter": {"PP": 0}, "devices": [0], "bucket_size": bad}])
