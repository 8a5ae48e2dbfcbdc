"""The C-ABI library loads on a CPU-only host and exports every symbol the header declares."""
import ctypes
import re
from pathlib import Path

import pytest

from piper_amd import _lib

HEADER = Path(__file__).resolve().parents[1] / "include" / "piper_amd.h"


def declared_symbols():
    text = HEADER.read_text()
    return sorted(set(re.findall(r"^PK_API\s+[\w\s\*]+?\b(pk_\w+)\s*\(", text, flags=re.M)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    assert len(syms) >= 21
    for must in ("pk_route_topk", "pk_sort_by_expert", "pk_permute_fwd", "pk_combine_fwd",
                 "pk_grouped_swiglu_fwd", "pk_grouped_swiglu_dgrad", "pk_grouped_swiglu_wgrad",
                 "pk_bucket_plan", "pk_bucket_pack", "pk_adamw_fused"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    assert _lib.is_built(), "build the library first: python -m piper_amd.build"
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    # and the ctypes signature table covers exactly the declared set
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_host_only_calls():
    lib = _lib.load()
    assert lib.pk_version() >= 100
    assert _lib.status_string(0) == "ok"
    assert "argument" in _lib.status_string(-1)
    assert lib.pk_sort_workspace_bytes(32768, 128) == (32768 // 512) * 128 * 4
    assert lib.pk_sort_workspace_bytes(-1, 128) < 0


def test_counter_sets_are_handed_out_per_stream_and_capture():
    """Launches that can overlap must not share scheduling counters: every (stream, capture
    sequence) pair keeps a set of its own; the same pair always gets the same set."""
    lib = _lib.load()
    dev = 63                      # a device index no GPU test uses: the directory starts empty there
    stream_a, stream_b = 0x7f0000001000, 0x7f0000002000
    a = lib.pk_sched_slot_index(dev, stream_a, 0, 0)
    b = lib.pk_sched_slot_index(dev, stream_b, 0, 0)
    assert a >= 0 and b >= 0 and a != b
    assert lib.pk_sched_slot_index(dev, stream_a, 0, 0) == a          # stable per stream
    # a launch recorded into a graph on stream a: another set than eager work on stream a,
    # and another capture another set again
    g1 = lib.pk_sched_slot_index(dev, stream_a, 1, 0)
    g2 = lib.pk_sched_slot_index(dev, stream_a, 2, 0)
    assert len({a, b, g1, g2}) == 4
    assert lib.pk_sched_slot_index(dev, stream_a, 1, 0) == g1
    # the per-thread default stream is one handle for many streams: the thread is part of the key
    t1 = lib.pk_sched_slot_index(dev, 2, 0, 111)
    t2 = lib.pk_sched_slot_index(dev, 2, 0, 222)
    assert t1 != t2 and len({a, b, g1, g2, t1, t2}) == 6
    # the null stream has a set like any other
    assert lib.pk_sched_slot_index(dev, 0, 0, 0) not in {a, b, g1, g2, t1, t2}
    # more keys than sets: shared round-robin, still a valid index, and old keys keep theirs
    seen = {lib.pk_sched_slot_index(dev, 0x100000 + 64 * i, 0, 0) for i in range(1100)}
    assert all(0 <= s < 1024 for s in seen) and len(seen) == 1024
    assert lib.pk_sched_slot_index(dev, stream_a, 0, 0) == a
    assert lib.pk_sched_slot_index(-1, 0, 0, 0) < 0 and lib.pk_sched_slot_index(64, 0, 0, 0) < 0
