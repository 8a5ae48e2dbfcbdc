"""Build libpiper_amd.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

Usage: ``python -m piper_amd.build`` or ``piper_amd.build.build_library()``.
The library is written next to this file so that it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libpiper_amd.so"
SOURCES = ["bucket.hip", "route.hip", "permute.hip", "grouped_gemm.hip", "timing.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libpiper_amd.so")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32-ops feature; harmless.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build_library(verbose: bool = False) -> Path:
    """Compile every .hip source for gfx950 and link the shared library.  Always rebuilds."""
    hipcc = _hipcc()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    objs = []
    cmds = []
    for src in SOURCES:
        obj = obj_dir / (src.replace(".hip", ".o"))
        objs.append(str(obj))
        cmds.append([hipcc, *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)])
    if verbose:
        for c in cmds:
            print(" ".join(c))
    with ThreadPoolExecutor(max_workers=min(5, len(cmds))) as pool:
        list(pool.map(_run, cmds))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *objs])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
