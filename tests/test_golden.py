"""Golden fixtures (tests/golden, written by make_golden.py): the oracle still reproduces them
(CPU), and the HIP kernels reproduce them through the C ABI (GPU)."""
import json
import math
import os

import numpy as np
import pytest
import torch

from conftest import ADAMW_TOL, F32_TOL, rel_err
from oracle import bucket as OB
from oracle import moe as O
from piper_amd import ops
from piper_amd.configs import ADAMW, bucket_manifest_cfg2

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _routing():
    return {k: v for k, v in np.load(os.path.join(G, "routing_small.npz")).items()}


def test_oracle_reproduces_routing_fixture():
    r = _routing()
    logits = torch.from_numpy(r["logits"])
    s, idx = O.route_topk(logits, int(r["top_k"]), True)
    counts, starts, perm, inv = O.sort_by_expert(idx, logits.shape[1])
    assert np.array_equal(idx.numpy(), r["top_idx"]) and np.array_equal(perm.numpy(), r["perm"])
    assert np.array_equal(counts.numpy(), r["counts"]) and np.array_equal(starts.numpy(), r["starts"])
    assert np.allclose(s.numpy(), r["top_scores"], rtol=1e-6, atol=1e-7)
    assert r["top_idx"][0].tolist() == [0, 1, 2, 3]   # an all-equal row takes the lowest indices


def test_bucket_offsets_fixture_oracle_and_c_abi():
    fx = json.load(open(os.path.join(G, "bucket_offsets_cfg2.json")))
    manifest = bucket_manifest_cfg2()
    assert fx["names"] == [n for n, _ in manifest] and fx["numels"] == [math.prod(s) for _, s in manifest]
    assert OB.plan_offsets(fx["numels"], fx["elem_size"], fx["align_bytes"]) == (fx["offsets"], fx["total"])
    assert ops.bucket_plan(fx["numels"], fx["elem_size"], fx["align_bytes"]) == (fx["offsets"], fx["total"])


def test_oracle_reproduces_adamw_fixture():
    fx = np.load(os.path.join(G, "adamw_small.npz"))
    p = torch.from_numpy(fx["params"][0])
    m = torch.zeros_like(p)
    v = torch.zeros_like(p)
    for step in range(1, 4):
        p, m, v = OB.adamw_step_torch(p, torch.from_numpy(fx["grads"][step - 1]), m, v, step, ADAMW["lr"], ADAMW["betas"],
                                      ADAMW["eps"], ADAMW["weight_decay"])
        assert np.allclose(p.numpy(), fx["params"][step], rtol=0, atol=1e-8)


@pytest.mark.gpu
def test_kernels_reproduce_routing_fixture(dev):
    r = _routing()
    logits = torch.from_numpy(r["logits"]).to(dev)
    s, idx = ops.route_topk(logits, int(r["top_k"]), True)
    counts, starts, perm, inv = ops.sort_by_expert(idx, logits.shape[1])
    assert np.array_equal(idx.cpu().numpy(), r["top_idx"])
    assert np.array_equal(perm.cpu().numpy(), r["perm"]) and np.array_equal(inv.cpu().numpy(), r["inv_perm"])
    assert np.array_equal(counts.cpu().numpy(), r["counts"]) and np.array_equal(starts.cpu().numpy(), r["starts"])
    assert rel_err(s, torch.from_numpy(r["top_scores"])) <= F32_TOL


@pytest.mark.gpu
def test_kernels_reproduce_adamw_fixture(dev):
    fx = np.load(os.path.join(G, "adamw_small.npz"))
    p = torch.from_numpy(fx["params"][0]).to(dev)
    m = torch.zeros_like(p)
    v = torch.zeros_like(p)
    for step in range(1, 4):
        g = torch.from_numpy(fx["grads"][step - 1]).to(dev)
        ops.adamw_fused(p, m, v, g, step=step, lr=ADAMW["lr"], beta1=ADAMW["betas"][0], beta2=ADAMW["betas"][1],
                        eps=ADAMW["eps"], weight_decay=ADAMW["weight_decay"])
        assert np.abs(p.cpu().numpy() - fx["params"][step]).max() <= ADAMW_TOL
