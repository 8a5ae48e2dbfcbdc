import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    from piper_amd import _lib

    if not _lib.is_built():
        pytest.fail("libpiper_amd.so is not built: run `python -m piper_amd.build` first")
    return torch.device("cuda:0")


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b| in float64: the normalised maximum error used for every tolerance."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.abs().max().item()
    if denom == 0.0:
        return (a - b).abs().max().item()
    return (a - b).abs().max().item() / denom


def rel_err_by_expert(got: torch.Tensor, ref: torch.Tensor, counts, *, rows: bool):
    """(worst relative error, expert) with every expert judged on its OWN scale: max |a-b| over the
    expert's slice divided by max |b| over the same slice.  A whole-tensor maximum hides an expert
    with few rows, whose gradient is a small fraction of the largest one.

    rows=True : got/ref are [A, ...] and expert e owns rows [sum(counts[:e]), +counts[e])
    rows=False: got/ref are [E, ...] (weight gradients); an expert without rows must hold exact zeros
    """
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    worst, where, start = 0.0, -1, 0
    for e, c in enumerate(int(c) for c in counts):
        if rows:
            a, b = got[start:start + c], ref[start:start + c]
            start += c
            if c == 0:
                continue
        else:
            a, b = got[e], ref[e]
            if c == 0:
                if a.abs().max().item() != 0.0:
                    return float("inf"), e
                continue
        denom = b.abs().max().item()
        err = (a - b).abs().max().item()
        err = err if denom == 0.0 else err / denom
        if err > worst:
            worst, where = err, e
    return worst, where


BF16_TOL = 2e-2   # activations / gradients computed in bf16
F32_TOL = 1e-5    # activations / gradients computed in fp32
ADAMW_TOL = 1e-6  # fp32 master weights after AdamW
