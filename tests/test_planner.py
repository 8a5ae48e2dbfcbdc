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
