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
