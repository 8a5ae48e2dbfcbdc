"""Pins the CPU oracle of the expert region against what the mathematics fixes: float64
evaluations, brute force on tiny inputs, invariants, and the reference's literal padded algorithm.
"""
import itertools

import numpy as np
import pytest
import torch

from oracle import moe as O


def test_gate_logits_matches_float64():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(37, 48, generator=g)
    w = torch.randn(6, 48, generator=g) * 0.02
    b = torch.randn(6, generator=g)
    ref = x.double() @ w.double().t() + b.double()
    assert torch.allclose(O.gate_logits(x, w, b).double(), ref, rtol=0, atol=1e-5)
    assert torch.allclose(O.gate_logits(x.bfloat16(), w, None).double(), x.bfloat16().double() @ w.double().t(), atol=1e-5, rtol=0)


def _brute_topk(row, k):
    """Definition: repeatedly take the largest remaining value, the lowest index among equals."""
    taken, out = set(), []
    for _ in range(k):
        best = None
        for e, v in enumerate(row):
            if e in taken:
                continue
            if best is None or v > row[best]:
                best = e
        taken.add(best)
        out.append(best)
    return out


@pytest.mark.parametrize("E,K", [(4, 2), (5, 3), (8, 2), (8, 8)])
def test_topk_selection_bruteforce_with_ties(E, K):
    # every row over a 3-letter alphabet for small E: all tie patterns appear
    vals = [-1.0, 0.0, 0.5]
    rows = list(itertools.product(vals, repeat=E))[:2000]
    logits = torch.tensor(rows, dtype=torch.float32)
    _, idx = O.route_topk(logits, K, route_norm=False)
    for r, row in enumerate(rows):
        assert idx[r].tolist() == _brute_topk(row, K)


def test_topk_all_equal_row_takes_lowest_indices_and_signed_zero():
    logits = torch.zeros(3, 8)
    logits[1, 3] = -0.0  # -0.0 == +0.0: still a tie
    _, idx = O.route_topk(logits, 4, route_norm=True)
    assert idx.tolist() == [[0, 1, 2, 3]] * 3


def test_scores_are_softmax_and_renorm_sums_to_scale():
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(64, 16, generator=g)
    s, idx = O.route_topk(logits, 4, route_norm=False)
    p64 = torch.softmax(logits.double(), -1)
    assert torch.allclose(s.double(), p64.gather(1, idx), atol=1e-7, rtol=1e-6)
    # selected = the 4 largest probabilities
    assert torch.equal(torch.sort(idx, 1).values, torch.sort(torch.topk(p64, 4, dim=1).indices, 1).values)
    s2, idx2 = O.route_topk(logits, 4, route_norm=True, route_scale=2.5)
    assert torch.equal(idx, idx2)
    assert torch.allclose(s2.sum(1), torch.full((64,), 2.5), atol=1e-6)
    assert torch.allclose(s2, 2.5 * s / s.sum(1, keepdim=True), atol=1e-6)


def test_sort_by_expert_invariants_and_numpy_stable_sort():
    g = torch.Generator().manual_seed(3)
    E, T, K = 7, 93, 3
    idx = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    idx[:, :] = torch.where(idx == 5, torch.zeros_like(idx), idx)  # expert 5 empty (duplicates are fine here)
    counts, starts, perm, inv = O.sort_by_expert(idx, E)
    A = T * K
    flat = idx.reshape(-1)
    assert counts.sum().item() == A and counts[5].item() == 0
    assert starts[0].item() == 0 and starts[-1].item() == A
    assert torch.equal(starts[1:] - starts[:-1], counts)
    assert torch.equal(starts[:-1], torch.cumsum(counts, 0) - counts)          # patch.py:27
    assert sorted(perm.tolist()) == list(range(A))                              # bijection
    sorted_e = flat[perm]
    assert bool((sorted_e[1:] >= sorted_e[:-1]).all())                          # expert-major
    for e in range(E):                                                          # ascending slots within an expert
        seg = perm[starts[e]:starts[e + 1]]
        assert bool((seg[1:] > seg[:-1]).all())
    assert np.array_equal(perm.numpy(), np.argsort(flat.numpy(), kind="stable"))
    assert torch.equal(inv[perm], torch.arange(A))


def _random_region(seed, T, H, E, K, I, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=dtype)
    wg = torch.randn(E, H, generator=g) * 0.5
    w1 = torch.randn(E, I, H, generator=g, dtype=dtype) * 0.3
    w3 = torch.randn(E, I, H, generator=g, dtype=dtype) * 0.3
    w2 = torch.randn(E, H, I, generator=g, dtype=dtype) * 0.3
    return x, wg, w1, w2, w3


def test_grouped_swiglu_equals_reference_padded_algorithm_and_float64_rows():
    x, wg, w1, w2, w3 = _random_region(4, T=40, H=16, E=6, K=2, I=12)
    logits = O.gate_logits(x, wg)
    logits[:, 4] = -1e9  # expert 4 never selected: an empty expert
    _, idx = O.route_topk(logits, 2, True)
    counts, starts, perm, _ = O.sort_by_expert(idx, 6)
    assert counts[4].item() == 0
    routed = O.permute(x, perm, 2)
    y = O.grouped_swiglu(w1, w2, w3, routed, counts)
    y_pad = O.padded_bmm_experts(w1, w2, w3, routed, counts)
    assert torch.allclose(y, y_pad, atol=1e-5, rtol=1e-5)
    # row by row in float64 from the definition
    flat_e = idx.reshape(-1)[perm]
    for p in range(0, routed.shape[0], 7):
        e = int(flat_e[p])
        r = routed[p].double()
        gate, up = w1[e].double() @ r, w3[e].double() @ r
        ref = w2[e].double() @ (gate * torch.sigmoid(gate) * up)
        assert torch.allclose(y[p].double(), ref, atol=1e-5, rtol=1e-5)


def test_unpermute_combine_float64():
    x, wg, w1, w2, w3 = _random_region(5, T=21, H=8, E=5, K=3, I=6)
    out, aux = O.moe_forward(x, wg, None, w1, w2, w3, 3, True)
    T, K = aux["top_scores"].shape
    y_tk = aux["y_sorted"][aux["inv_perm"]].reshape(T, K, -1).double()
    ref = (aux["top_scores"].double()[:, :, None] * y_tk).sum(1)
    assert torch.allclose(out.double(), ref, atol=1e-6, rtol=1e-6)
    # the permutation really is x[perm // K]
    assert torch.equal(O.permute(x, aux["perm"], K), x[aux["perm"] // K])


def test_moe_forward_equals_dense_definition():
    """Independent statement: out[t] = sum over selected e of w_te * FFN_e(x_t)."""
    x, wg, w1, w2, w3 = _random_region(6, T=17, H=8, E=4, K=2, I=6)
    out, aux = O.moe_forward(x, wg, None, w1, w2, w3, 2, True)
    ref = torch.zeros(17, 8, dtype=torch.float64)
    for t in range(17):
        for k in range(2):
            e = int(aux["top_idx"][t, k])
            r = x[t].double()
            gate, up = w1[e].double() @ r, w3[e].double() @ r
            ref[t] += aux["top_scores"][t, k].double() * (w2[e].double() @ (gate * torch.sigmoid(gate) * up))
    assert torch.allclose(out.double(), ref, atol=1e-5, rtol=1e-5)


def test_backward_gradcheck_float64_with_empty_expert():
    T, H, E, K, I = 5, 8, 4, 2, 6
    x, wg, w1, w2, w3 = _random_region(7, T, H, E, K, I, dtype=torch.float64)
    wg = wg.double()
    bias = torch.tensor([0.0, 0.0, -50.0, 0.0], dtype=torch.float64)  # expert 2 empty

    def f(x_, wg_, w1_, w2_, w3_):
        # float64 evaluation of the same graph (the oracle casts the gate to fp32, so restate it here)
        logits = x_ @ wg_.t() + bias
        scores = torch.softmax(logits, -1)
        idx = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :K]
        ts = scores.gather(1, idx)
        ts = ts / (ts.sum(-1, keepdim=True) + 1e-20)
        counts, starts, perm, inv = O.sort_by_expert(idx, E)
        y = O.grouped_swiglu(w1_, w2_, w3_, O.permute(x_, perm, K), counts)
        return O.unpermute_combine(y, perm, ts)

    inputs = [t.clone().requires_grad_(True) for t in (x, wg, w1, w2, w3)]
    assert torch.autograd.gradcheck(f, inputs, eps=1e-6, atol=1e-5, rtol=1e-4)
    # the fp32 oracle's autograd agrees with the float64 graph
    out64 = f(*inputs)
    g64 = torch.autograd.grad(out64.sum(), inputs)
    ins32 = [t.detach().float().requires_grad_(True) for t in (x, wg, w1, w2, w3)]
    out32, _ = O.moe_forward(ins32[0], ins32[1], bias.float(), ins32[2], ins32[3], ins32[4], K, True)
    g32 = torch.autograd.grad(out32.sum(), ins32)
    for a, b in zip(g32, g64):
        assert torch.allclose(a.double(), b, atol=1e-4, rtol=1e-3)
    assert float(g64[2][2].abs().max()) == 0.0  # the empty expert gets an exactly zero weight gradient


def test_rmsnorm_matches_library_routine_and_closed_form():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(7, 48, generator=g, dtype=torch.float64)
    w = torch.randn(48, generator=g, dtype=torch.float64)
    for eps in (1e-6, 1e-5, 0.5):
        got = O.rmsnorm(x, w, eps)
        assert torch.allclose(got, torch.nn.functional.rms_norm(x, (48,), w, eps), rtol=1e-12, atol=1e-12)
        # closed form, element by element
        for t in (0, 3, 6):
            ms = sum(float(v) ** 2 for v in x[t]) / 48
            ref = [float(x[t, h]) / (ms + eps) ** 0.5 * float(w[h]) for h in range(48)]
            assert max(abs(float(got[t, h]) - ref[h]) for h in range(48)) < 1e-12
    # scale invariance (up to eps): rmsnorm(c*x) == rmsnorm(x) for eps -> 0
    assert torch.allclose(O.rmsnorm(3.0 * x, w, 0.0), O.rmsnorm(x, w, 0.0), rtol=1e-12, atol=1e-12)
    # a row of ones with unit weight has unit RMS
    one = torch.ones(1, 48, dtype=torch.float64)
    assert torch.allclose(O.rmsnorm(one, torch.ones(48, dtype=torch.float64), 0.0), one)
    xr = x.clone().requires_grad_(True)
    wr = w.clone().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b: O.rmsnorm(a, b, 1e-6), (xr, wr), eps=1e-6, atol=1e-6)
