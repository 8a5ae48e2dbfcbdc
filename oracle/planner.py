"""CPU restatement of the parameter -> bucket assignment of the reference's ``bucket_stage``
(TEST INFRASTRUCTURE, see oracle/__init__.py).

Follows src/bucket.py:76-128 step by step on plain lists: a bucket id per parameter from the greedy
fill (:76-86), the span of every initial bucket and the promotion of parameters whose first and
last use fall into different initial buckets (:88-108), the bucket list sorted by first use and the
merge of overlapping neighbours (:110-128).  The FX-graph parts of the function (what a use range
is, the alias-crossing merges of :250-269, the sub-graph construction) are not restated: the
product takes use ranges as input.

Pinning status (tests/test_planner.py): the greedy stage by the two properties that define a
greedy fill, the later stages by hand-worked cases; this restatement is the second, independently
written statement of the same lines that `piper_amd.planner.plan_param_buckets` is compared with
on random inputs.
"""
from __future__ import annotations


def assign_buckets(sizes, use_ranges, bucket_size_bytes):
    """Returns the merged buckets as (first_use, last_use, member indices) in execution order."""
    n = len(sizes)
    # src/bucket.py:76-86
    bucket_id = {}
    cur_b, cur_sz = 0, 0
    for i in range(n):
        if cur_sz + sizes[i] > bucket_size_bytes and cur_sz > 0:
            cur_b += 1
            cur_sz = 0
        bucket_id[i] = cur_b
        cur_sz += sizes[i]
    n_init = cur_b + 1

    # src/bucket.py:88-96
    init_ranges = []
    for b in range(n_init):
        ms = [i for i in range(n) if bucket_id[i] == b]
        if not ms:
            init_ranges.append((0, 0))
        else:
            init_ranges.append((min(use_ranges[i][0] for i in ms), max(use_ranges[i][1] for i in ms)))

    # src/bucket.py:98-108
    def bucket_at(idx):
        for b, (lo, hi) in enumerate(init_ranges):
            if lo <= idx <= hi:
                return b
        return 0

    sn = n_init
    for i in range(n):
        f, l = use_ranges[i]
        if bucket_at(f) != bucket_at(l):
            bucket_id[i] = sn
            sn += 1

    # src/bucket.py:110-128
    bm = {}
    for i in range(n):
        bm.setdefault(bucket_id[i], []).append(i)
    blist = []
    for members in bm.values():
        blist.append((min(use_ranges[i][0] for i in members), max(use_ranges[i][1] for i in members), members))
    blist.sort(key=lambda t: t[0])
    merged = []
    for f, l, ms in blist:
        if merged and f <= merged[-1][1]:
            pf, pl, pm = merged[-1]
            merged[-1] = (pf, max(pl, l), pm + ms)
        else:
            merged.append((f, l, ms))
    return merged
