"""GPU parity of the grouped SwiGLU expert kernels (forward, input gradient, weight gradient)
against the CPU oracle.  bf16 results are judged against the oracle evaluated in fp32 on the
same bf16 inputs (tolerance 2e-2 of the output's maximum), fp32 results to 1e-5."""
import pytest
import torch

from conftest import BF16_TOL, F32_TOL, rel_err, rel_err_by_expert
from oracle import moe as O
from piper_amd import functional as F_
from piper_amd import ops

pytestmark = pytest.mark.gpu


def _make(seed, counts, H, I, dtype):
    g = torch.Generator().manual_seed(seed)
    E = len(counts)
    A = int(sum(counts))
    x = torch.randn(A, H, generator=g).to(dtype)
    w1 = (torch.randn(E, I, H, generator=g) * 0.05).to(dtype)
    w3 = (torch.randn(E, I, H, generator=g) * 0.05).to(dtype)
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).to(dtype)
    dy = torch.randn(A, H, generator=g).to(dtype)
    return x, w1, w2, w3, dy, torch.tensor(counts, dtype=torch.long)


def _oracle(x, w1, w2, w3, dy, counts):
    """fp32 evaluation with autograd; also returns the SwiGLU intermediates' gradients."""
    xr, w1r, w2r, w3r = (t.float().requires_grad_(True) for t in (x, w1, w2, w3))
    y = O.grouped_swiglu(w1r, w2r, w3r, xr, counts)
    dx, dw1, dw2, dw3 = torch.autograd.grad(y, (xr, w1r, w2r, w3r), dy.float())
    return y.detach(), dx, dw1, dw2, dw3


CASES = [
    # (counts, H, I)   -- ragged, empty experts, single rows, more than one 128-row tile
    ([128, 128, 128, 128], 256, 256),
    ([0, 5, 300, 0, 129, 1, 127, 0], 256, 128),
    ([37] * 16, 128, 384),
    ([0, 0, 0, 700], 384, 256),
    # enough 256-row units per workgroup for the 256x256 tiles, with a reduction of only four k-tiles
    ([8192, 8192], 128, 1536),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("counts,H,I", CASES)
def test_grouped_swiglu_fwd_dgrad_wgrad(dev, dtype, counts, H, I):
    print(f"[case] grouped_swiglu {dtype} counts={counts[:8]} H={H} I={I}", flush=True)
    x, w1, w2, w3, dy, cnt = _make(3, counts, H, I, dtype)
    y_ref, dx_ref, dw1_ref, dw2_ref, dw3_ref = _oracle(x, w1, w2, w3, dy, cnt)
    tol = BF16_TOL if dtype == torch.bfloat16 else F32_TOL
    E = len(counts)
    X, W1, W2, W3, DY = (t.to(dev) for t in (x, w1, w2, w3, dy))
    starts = ops.counts_to_starts(cnt.to(dev))
    y, g, u, h = ops.grouped_swiglu_fwd(X, W1, W2, W3, starts)
    assert y.dtype == dtype and rel_err(y, y_ref) <= tol
    # saved pre-activations are what they claim to be
    if sum(counts) > 0:
        e0 = next(e for e, c in enumerate(counts) if c > 0)
        s0 = int(sum(counts[:e0]))
        g_ref = x[s0:s0 + counts[e0]].float() @ w1[e0].float().t()
        assert rel_err(g[s0:s0 + counts[e0]], g_ref) <= tol
    dx, dg, du = ops.grouped_swiglu_dgrad(DY, W1, W2, W3, g, u, starts)
    assert rel_err(dx, dx_ref) <= tol
    dw1, dw2, dw3 = ops.grouped_swiglu_wgrad(DY, h, dg, du, X, starts, E)
    assert rel_err(dw1, dw1_ref) <= tol and rel_err(dw2, dw2_ref) <= tol and rel_err(dw3, dw3_ref) <= tol
    # every expert on its own scale: its rows of y and d_x, its weight gradients
    for name, got, ref, by_rows in (("y", y, y_ref, True), ("d_x", dx, dx_ref, True), ("d_w1", dw1, dw1_ref, False),
                                    ("d_w2", dw2, dw2_ref, False), ("d_w3", dw3, dw3_ref, False)):
        worst, e = rel_err_by_expert(got, ref, counts, rows=by_rows)
        assert worst <= tol, (name, "expert", e, counts[e], worst)
    for e, c in enumerate(counts):
        if c == 0:  # an expert without rows gets exact zeros, not garbage
            assert float(dw1[e].abs().max()) == 0.0 and float(dw2[e].abs().max()) == 0.0 and float(dw3[e].abs().max()) == 0.0
    # accumulate=True adds a second microbatch on top
    ops.grouped_swiglu_wgrad(DY, h, dg, du, X, starts, E, d_w1=dw1, d_w2=dw2, d_w3=dw3, accumulate=True)
    assert rel_err(dw2, 2 * dw2_ref) <= tol and rel_err(dw1, 2 * dw1_ref) <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("counts,H,I", CASES + [([10, 0, 70, 3, 1], 192, 64)])
def test_scaled_backward_matches_combine_bwd_then_dgrad(dev, dtype, counts, H, I):
    """The backward with the weighted combine folded into the d_h GEMM (d_out rows gathered, score
    applied in the epilogue, score gradient from the same accumulator) against the unfused chain
    combine_bwd -> dgrad_dh -> wgrad, and against fp32 autograd through the oracle."""
    print(f"[case] scaled backward {dtype} counts={counts[:8]} H={H} I={I}", flush=True)
    K = 2
    A = int(sum(counts))
    assert A % K == 0
    T, E = A // K, len(counts)
    gen = torch.Generator().manual_seed(11)
    _, w1, w2, w3, _, cnt = _make(5, counts, H, I, dtype)
    perm = torch.randperm(A, generator=gen).to(torch.int32)          # sorted row -> flat (token, k) slot
    tok = perm.long() // K
    x_tok = torch.randn(T, H, generator=gen).to(dtype)
    x_sorted = x_tok[tok]
    scores = torch.rand(T, K, generator=gen) + 0.1
    d_out = torch.randn(T, H, generator=gen).to(dtype)
    tol = BF16_TOL if dtype == torch.bfloat16 else F32_TOL

    XT, XS, W1, W2, W3, PERM, SC, DO = (t.to(dev) for t in (x_tok, x_sorted, w1, w2, w3, perm, scores, d_out))
    starts = ops.counts_to_starts(cnt.to(dev))
    y, g, u, h = ops.grouped_swiglu_fwd(XT, W1, W2, W3, starts, row_map=PERM, row_map_div=K)

    # fp32 reference: out[t] = sum_k s[t,k] * y[row(t,k)]
    xr, w1r, w2r, w3r = (t.float().requires_grad_(True) for t in (x_sorted, w1, w2, w3))
    sr = scores.clone().requires_grad_(True)
    y_ref = O.grouped_swiglu(w1r, w2r, w3r, xr, cnt)
    out_ref = torch.zeros(T, H).index_add(0, tok, y_ref * sr.reshape(-1)[perm.long()].unsqueeze(1))
    dx_ref, dw1_ref, dw2_ref, dw3_ref, ds_ref = torch.autograd.grad(out_ref, (xr, w1r, w2r, w3r, sr), d_out.float())

    d_g, d_u, hs, d_s = ops.grouped_swiglu_dgrad_dh_scaled(DO, PERM, SC, W2, g, u, starts)
    assert d_s.shape == (T, K) and rel_err(d_s, ds_ref) <= tol
    d_xs = ops.grouped_swiglu_dgrad_dx(d_g, d_u, W1, W3, starts)
    assert rel_err(d_xs, dx_ref) <= tol
    dw1, dw2, dw3 = ops.grouped_swiglu_wgrad(DO, hs, d_g, d_u, XT, starts, E, row_map=PERM, row_map_div=K, scaled=True)
    assert rel_err(dw1, dw1_ref) <= tol and rel_err(dw2, dw2_ref) <= tol and rel_err(dw3, dw3_ref) <= tol
    for name, got, ref, by_rows in (("d_x", d_xs, dx_ref, True), ("d_w1", dw1, dw1_ref, False),
                                    ("d_w2", dw2, dw2_ref, False), ("d_w3", dw3, dw3_ref, False)):
        worst, e = rel_err_by_expert(got, ref, counts, rows=by_rows)
        assert worst <= tol, (name, "expert", e, counts[e], worst)

    # the unfused chain on the same inputs
    d_y, d_s2 = ops.combine_bwd(DO, y, PERM, SC)
    d_g2, d_u2 = ops.grouped_swiglu_dgrad_dh(d_y, W2, g, u, starts)
    loose = 2 * tol          # both sides round at different places
    assert rel_err(d_s, d_s2) <= loose and rel_err(d_g, d_g2) <= loose and rel_err(d_u, d_u2) <= loose
    _, dw2_b, _ = ops.grouped_swiglu_wgrad(d_y, h, d_g2, d_u2, XS, starts, E)
    assert rel_err(dw2, dw2_b) <= loose
    for e, c in enumerate(counts):
        if c == 0:
            assert float(dw2[e].abs().max()) == 0.0


def _row_tile_boundary_counts(E):
    """Row counts around the 256- and 128-row block tiles: exact multiples, one above, a few tens
    above, short and empty experts."""
    edge = [256, 257, 287, 288, 289, 255, 1, 0, 544, 545, 320, 33, 32, 31, 512, 513, 543, 800, 300, 270,
            264, 250, 129, 128, 127, 1056, 1057, 16, 272, 260]
    counts = [edge[i % len(edge)] for i in range(E)]
    return counts


def test_row_tiles_at_block_tile_boundaries(dev):
    """Forward and input gradient on a launch with 128 experts whose row counts sit on every side
    of the block tile boundaries, every expert against fp32 matmuls of the same bf16 inputs on the
    device; the rows of an expert's last, partly filled row tile are also compared on their own."""
    E, H, I = 128, 1024, 512
    counts = _row_tile_boundary_counts(E)
    A = sum(counts)
    print(f"[case] row tile boundaries E={E} A={A} H={H} I={I}", flush=True)
    g_ = torch.Generator().manual_seed(21)
    x = torch.randn(A, H, generator=g_).to(torch.bfloat16).to(dev)
    dy = torch.randn(A, H, generator=g_).to(torch.bfloat16).to(dev)
    w1 = (torch.randn(E, I, H, generator=g_) * 0.05).to(torch.bfloat16).to(dev)
    w3 = (torch.randn(E, I, H, generator=g_) * 0.05).to(torch.bfloat16).to(dev)
    w2 = (torch.randn(E, H, I, generator=g_) * 0.05).to(torch.bfloat16).to(dev)
    starts = ops.counts_to_starts(torch.tensor(counts, dtype=torch.long, device=dev))
    y, g, u, h = ops.grouped_swiglu_fwd(x, w1, w2, w3, starts)
    dx, dg, du = ops.grouped_swiglu_dgrad(dy, w1, w2, w3, g, u, starts)
    torch.cuda.synchronize()
    s = 0
    for e, c in enumerate(counts):
        if c == 0:
            continue
        xe = x[s:s + c].float().requires_grad_(True)
        ge = xe @ w1[e].float().t()
        ue = xe @ w3[e].float().t()
        he = torch.nn.functional.silu(ge) * ue
        ye = he @ w2[e].float().t()
        (dxe,) = torch.autograd.grad(ye, xe, dy[s:s + c].float())
        for name, got, ref in (("g", g, ge), ("u", u, ue), ("h", h, he), ("y", y, ye), ("dx", dx, dxe)):
            assert rel_err(got[s:s + c], ref) <= BF16_TOL, (name, e, c, rel_err(got[s:s + c], ref))
            t0 = (c - 1) // 256 * 256      # first row of the expert's last 256-row group
            if t0 > 0:
                assert rel_err(got[s + t0:s + c], ref[t0:]) <= BF16_TOL, (name, "last row tile", e, c)
        s += c


T_CASES = [
    # ragged around the 8-row padding and the 32-row k-tile, empty experts, one long expert
    ([0, 1, 7, 8, 9, 31, 32, 33, 0, 300, 64, 255], 256, 256),
    ([700, 0, 0, 2], 512, 256),
    ([256] * 6, 256, 512),
    ([4096, 3000, 1000, 96], 256, 1536),
    # more weight-gradient tiles than workgroups, so a workgroup walks several units: units handed
    # out from the counters (long experts) with experts of 0, 1 and 33 rows between long ones ...
    ([3000, 0, 1, 2500, 33, 0, 700, 600, 500, 400, 300, 64, 32, 70, 100, 96], 1024, 768),
    # ... and the static hand-out with many short experts (reductions of 0 to 3 k-tiles back to back)
    ([0, 1, 33, 64, 5, 96, 31, 70, 0, 0, 65, 2] * 24, 256, 256),
    # enough 256-row units per workgroup for the 256x256x32 tiles (the d_x GEMM then reads 32-deep
    # k-tiles of the transposed copies), with ragged last row tiles
    ([8192, 8000, 8300, 7777, 8192, 8448, 8193, 8190], 1024, 256),
]


@pytest.mark.parametrize("counts,H,I", T_CASES)
def test_transposed_backward_pair_matches_the_plain_pair(dev, counts, H, I):
    """pk_grouped_swiglu_dgrad_dh_scaled_t / pk_grouped_swiglu_wgrad_scaled_t (one operand of every
    weight-gradient GEMM K-contiguous, persistent workgroups) against
    pk_grouped_swiglu_dgrad_dh_scaled / pk_grouped_swiglu_wgrad_scaled on the same inputs, against
    fp32 autograd through the oracle, and the layout of the transposed copies."""
    print(f"[case] transposed backward counts={counts} H={H} I={I}", flush=True)
    K = 2
    A = int(sum(counts))
    if A % K:
        counts = list(counts); counts[-1] += 1; A += 1
    T, E = A // K, len(counts)
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(21)
    _, w1, w2, w3, _, cnt = _make(6, counts, H, I, dtype)
    perm = torch.randperm(A, generator=gen).to(torch.int32)
    tok = perm.long() // K
    x_tok = torch.randn(T, H, generator=gen).to(dtype)
    scores = torch.rand(T, K, generator=gen) + 0.1
    d_out = torch.randn(T, H, generator=gen).to(dtype)
    XT, W1, W2, W3, PERM, SC, DO = (t.to(dev) for t in (x_tok, w1, w2, w3, perm, scores, d_out))
    starts = ops.counts_to_starts(cnt.to(dev))
    ldt = ops.transposed_ld(A, H, I, E, dtype)
    assert ldt >= ((A + 63) // 64 + E) * 64 and ldt % 256 == 128
    assert ops.transposed_ld(A, H + 128, I, E, dtype) == 0 and ops.transposed_ld(A, H, I, E, torch.float32) == 0
    _, g, u, _ = ops.grouped_swiglu_fwd(XT, W1, W2, W3, starts, row_map=PERM, row_map_div=K)

    d_g, d_u, hs, d_s = ops.grouped_swiglu_dgrad_dh_scaled(DO, PERM, SC, W2, g, u, starts)
    # poison what the transposed call allocates next, so untouched pad columns would show as NaN
    junk = torch.full((3 * I * ldt + 16,), float("nan"), dtype=dtype, device=dev)
    del junk
    d_g2, d_u2, d_gT, d_uT, hsT, d_s2 = ops.grouped_swiglu_dgrad_dh_scaled_t(DO, PERM, SC, W2, g, u, starts)
    assert torch.equal(d_g, d_g2) and torch.equal(d_u, d_u2) and torch.equal(d_s, d_s2)
    st = starts.cpu().tolist()
    for e, c in enumerate(counts):
        p0 = (st[e] // 64) * 64 + 64 * e
        c32 = (c + 31) // 32 * 32      # zeros up to the end of the expert's last block of 32 rows
        for full, tr in ((d_g, d_gT), (d_u, d_uT), (hs, hsT)):
            # [ldt/32, I, 32] -> [I, ldt]: column i, padded row r
            blk = tr.permute(1, 0, 2).reshape(I, ldt)[:, p0:p0 + c32]
            assert torch.equal(blk[:, :c], full[st[e]:st[e] + c].t()), f"expert {e}"
            assert torch.count_nonzero(blk[:, c:]).item() == 0, f"pad columns of expert {e}"

    # without the row-major outputs: the same transposed copies, and the d_x GEMM that reads its A
    # operand from them gives the d_x of the row-major pair bit for bit (same products, same order)
    none_g, none_u, d_gT3, d_uT3, hsT3, d_s3 = ops.grouped_swiglu_dgrad_dh_scaled_t(DO, PERM, SC, W2, g, u, starts, row_major=False)
    assert none_g is None and none_u is None and torch.equal(d_s3, d_s)
    for e, c in enumerate(counts):
        p0 = (st[e] // 64) * 64 + 64 * e
        c32 = (c + 31) // 32 * 32
        for a, b in ((d_gT, d_gT3), (d_uT, d_uT3), (hsT, hsT3)):
            assert torch.equal(a.permute(1, 0, 2).reshape(I, ldt)[:, p0:p0 + c32], b.permute(1, 0, 2).reshape(I, ldt)[:, p0:p0 + c32])
    d_x_rows = ops.grouped_swiglu_dgrad_dx(d_g, d_u, W1, W3, starts)
    d_x_blocks = ops.grouped_swiglu_dgrad_dx_t(d_gT3, d_uT3, W1, W3, starts, A)
    assert torch.equal(d_x_rows, d_x_blocks)

    ref = ops.grouped_swiglu_wgrad(DO, hs, d_g, d_u, XT, starts, E, row_map=PERM, row_map_div=K, scaled=True)
    order = torch.argsort(cnt, descending=True, stable=True).to(torch.int32).to(dev)
    for eo in (None, order):
        got = ops.grouped_swiglu_wgrad_scaled_t(DO, hsT, d_gT, d_uT, XT, starts, E, row_map=PERM, row_map_div=K, expert_order=eo)
        for a, b, name in zip(got, ref, ("d_w1", "d_w2", "d_w3")):
            # same products, same fp32 summation order over the rows: equal up to the last bf16 bit
            assert rel_err(a, b) <= 2.0 ** -7, name
            for e, c in enumerate(counts):
                if c == 0:
                    assert float(a[e].abs().max()) == 0.0
    # fp32 reference through the oracle
    x_sorted = x_tok[tok]
    xr, w1r, w2r, w3r = (t.float().requires_grad_(True) for t in (x_sorted, w1, w2, w3))
    y_ref = O.grouped_swiglu(w1r, w2r, w3r, xr, cnt)
    out_ref = torch.zeros(T, H).index_add(0, tok, y_ref * scores.reshape(-1)[perm.long()].unsqueeze(1))
    dw_ref = torch.autograd.grad(out_ref, (w1r, w2r, w3r), d_out.float())
    for a, b, name in zip(got, (dw_ref[0], dw_ref[1], dw_ref[2]), ("d_w1", "d_w2", "d_w3")):
        assert rel_err(a, b) <= BF16_TOL
        # every expert on its own scale: a one-row expert's gradient is a few per cent of the
        # largest one and would hide behind the whole-tensor maximum
        worst, e = rel_err_by_expert(a, b, counts, rows=False)
        assert worst <= BF16_TOL, (name, "expert", e, counts[e], worst)
    # accumulate: adds to what is there, twice gives 2x (+ one rounding)
    acc = [t.clone() for t in got]
    ops.grouped_swiglu_wgrad_scaled_t(DO, hsT, d_gT, d_uT, XT, starts, E, row_map=PERM, row_map_div=K,
                                      d_w1=acc[0], d_w2=acc[1], d_w3=acc[2], accumulate=True, expert_order=order)
    for a, b in zip(acc, got):
        assert rel_err(a, 2 * b.float()) <= 2.0 ** -7
    # argument checks: a row length below the query's, and a shape without the path
    with pytest.raises(RuntimeError):
        _lib_call_short_ld(DO, hsT, d_gT, d_uT, XT, PERM, starts, E, H, I, A, K, ldt - 64)


def _lib_call_short_ld(DO, hsT, d_gT, d_uT, XT, PERM, starts, E, H, I, A, K, ldt):
    from piper_amd._lib import call, current_stream, dtype_code, ptr
    w = torch.empty((E, I, H), dtype=DO.dtype, device=DO.device)
    call("pk_grouped_swiglu_wgrad_scaled_t", ptr(DO), ptr(hsT), ptr(d_gT), ptr(d_uT), ldt, ptr(XT), ptr(PERM), K, ptr(starts),
         ptr(None), ptr(w), ptr(None), ptr(None), 0, A, H, I, E, dtype_code(DO.dtype), current_stream(DO.device))


def test_mfma_path_agrees_with_fma_path(dev):
    """bf16 shapes outside the MFMA tiling (H or I not a multiple of 128) run on the FMA kernel."""
    print("[case] bf16 fallback shapes", flush=True)
    counts = [10, 0, 70, 3]
    x, w1, w2, w3, dy, cnt = _make(4, counts, 192, 64, torch.bfloat16)
    y_ref, dx_ref, dw1_ref, dw2_ref, dw3_ref = _oracle(x, w1, w2, w3, dy, cnt)
    X, W1, W2, W3, DY = (t.to(dev) for t in (x, w1, w2, w3, dy))
    starts = ops.counts_to_starts(cnt.to(dev))
    y, g, u, h = ops.grouped_swiglu_fwd(X, W1, W2, W3, starts)
    dx, dg, du = ops.grouped_swiglu_dgrad(DY, W1, W2, W3, g, u, starts)
    dw1, dw2, dw3 = ops.grouped_swiglu_wgrad(DY, h, dg, du, X, starts, 4)
    for a, b in ((y, y_ref), (dx, dx_ref), (dw1, dw1_ref), (dw2, dw2_ref), (dw3, dw3_ref)):
        assert rel_err(a, b) <= BF16_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_permute_operand_load(dev, dtype):
    """row_map = perm, div = K: reading x[perm[p] // K] inside the GEMM equals permute then GEMM."""
    print(f"[case] fused permute {dtype}", flush=True)
    T, H, I, E, K = 300, 256, 128, 8, 2
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g)
    logits[:, 3] = -50.0
    _, idx = O.route_topk(logits, K, True)
    counts, starts_ref, perm, inv = O.sort_by_expert(idx, E)
    x = torch.randn(T, H, generator=g).to(dtype)
    _, w1, w2, w3, _, _ = _make(6, [1] * E, H, I, dtype)
    X, W1, W2, W3 = (t.to(dev) for t in (x, w1, w2, w3))
    starts = starts_ref.int().to(dev)
    P = perm.int().to(dev)
    routed = ops.permute_fwd(X, P, K)
    y_a, g_a, u_a, h_a = ops.grouped_swiglu_fwd(routed, W1, W2, W3, starts)
    y_b, g_b, u_b, h_b = ops.grouped_swiglu_fwd(X, W1, W2, W3, starts, row_map=P, row_map_div=K)
    assert torch.equal(y_a, y_b) and torch.equal(g_a, g_b) and torch.equal(h_a, h_b)
    dy = torch.randn(T * K, H, generator=g).to(dtype).to(dev)
    dx, dg, du = ops.grouped_swiglu_dgrad(dy, W1, W2, W3, g_a, u_a, starts)
    wa = ops.grouped_swiglu_wgrad(dy, h_a, dg, du, routed, starts, E)
    wb = ops.grouped_swiglu_wgrad(dy, h_a, dg, du, X, starts, E, row_map=P, row_map_div=K)
    for a, b in zip(wa, wb):
        assert torch.equal(a, b)


@pytest.mark.parametrize("counts_dtype", [torch.int64, torch.int32])
def test_reference_operator_bmm_experts(dev, counts_dtype):
    """torch.ops.piper_artifact.bmm_experts(w1, w2, w3, x, num_tokens_per_expert) with autograd:
    the reference's operator boundary (qwen3_bmm_experts_patch.py:63-87)."""
    print("[case] piper_artifact::bmm_experts", flush=True)
    counts = [60, 0, 200, 4]
    x, w1, w2, w3, dy, cnt = _make(8, counts, 256, 128, torch.bfloat16)
    y_ref, dx_ref, dw1_ref, dw2_ref, dw3_ref = _oracle(x, w1, w2, w3, dy, cnt)
    F_.register_reference_op()
    X, W1, W2, W3 = (t.to(dev).requires_grad_(True) for t in (x, w1, w2, w3))
    y = torch.ops.piper_artifact.bmm_experts(W1, W2, W3, X, cnt.to(counts_dtype).to(dev))
    assert y.shape == x.shape and rel_err(y, y_ref) <= BF16_TOL
    y.backward(dy.to(dev))
    assert rel_err(X.grad, dx_ref) <= BF16_TOL
    assert rel_err(W1.grad, dw1_ref) <= BF16_TOL and rel_err(W2.grad, dw2_ref) <= BF16_TOL and rel_err(W3.grad, dw3_ref) <= BF16_TOL
    with torch.no_grad():
        y2 = torch.ops.piper_artifact.bmm_experts(W1, W2, W3, X, cnt.to(counts_dtype).to(dev))
    assert torch.equal(y2, y.detach())
    meta = torch.ops.piper_artifact.bmm_experts(*(t.detach().to("meta") for t in (W1, W2, W3, X)), cnt.to("meta"))
    assert meta.shape == x.shape and meta.is_meta


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_bmm_experts_rows_past_the_last_expert_are_zero(dev, dtype):
    """x has more rows than sum(num_tokens_per_expert): the reference returns zeros there
    (`out = x.new_zeros`, qwen3_bmm_experts_patch.py:43) and no gradient flows into them.  Checked
    against the oracle's restatement of the padded-bmm algorithm."""
    print(f"[case] bmm_experts with unowned rows {dtype}", flush=True)
    counts = [40, 0, 130, 5]
    extra = 37
    x, w1, w2, w3, dy, cnt = _make(11, counts, 256, 128, dtype)
    g = torch.Generator().manual_seed(12)
    x = torch.cat([x, torch.randn(extra, x.shape[1], generator=g).to(dtype)])
    dy = torch.cat([dy, torch.randn(extra, dy.shape[1], generator=g).to(dtype)])
    leaves = [t.detach().clone().float().requires_grad_(True) for t in (w1, w2, w3, x)]
    y_ref = O.padded_bmm_experts(*leaves, cnt)
    y_ref.backward(dy.float())
    assert torch.count_nonzero(y_ref[sum(counts):]) == 0 and torch.count_nonzero(leaves[3].grad[sum(counts):]) == 0
    F_.register_reference_op()
    W1, W2, W3, X = (t.to(dev).requires_grad_(True) for t in (w1, w2, w3, x))
    # poison the allocator's free blocks so that rows the kernels skip would show
    junk = torch.full((x.shape[0] * 4, x.shape[1]), float("nan"), device=dev, dtype=dtype)
    del junk
    y = torch.ops.piper_artifact.bmm_experts(W1, W2, W3, X, cnt.to(dev))
    tol = BF16_TOL if dtype == torch.bfloat16 else F32_TOL
    assert torch.count_nonzero(y[sum(counts):]).item() == 0
    assert rel_err(y, y_ref) <= tol
    y.backward(dy.to(dev))
    assert torch.count_nonzero(X.grad[sum(counts):]).item() == 0
    assert rel_err(X.grad, leaves[3].grad) <= tol
    for got, ref in zip((W1, W2, W3), leaves[:3]):
        assert rel_err(got.grad, ref.grad) <= tol
    with torch.no_grad():
        assert torch.count_nonzero(torch.ops.piper_artifact.bmm_experts(W1, W2, W3, X, cnt.to(dev))[sum(counts):]).item() == 0


def test_argument_errors(dev):
    z = torch.zeros(4, 8, device=dev, dtype=torch.bfloat16)
    w = torch.zeros(2, 16, 8, device=dev, dtype=torch.bfloat16)
    w2 = torch.zeros(2, 8, 16, device=dev, dtype=torch.bfloat16)
    starts = torch.tensor([0, 2, 4], dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        ops.grouped_swiglu_fwd(z, w, w, w, starts)             # w2 has the wrong shape
    with pytest.raises(ValueError):
        ops.grouped_swiglu_fwd(z.float(), w, w2, w, starts)    # dtype mismatch


def test_reference_operator_under_dynamo_fullgraph(dev):
    """The op traced by Dynamo with fullgraph=True (src/compile.py:273) and run by the eager
    backend gives the same forward and gradients as the direct call."""
    counts = [5, 0, 130, 61]
    x, w1, w2, w3, dy, cnt = _make(9, counts, 256, 128, torch.bfloat16)
    X, W1, W2, W3, DY, CNT = (t.to(dev) for t in (x, w1, w2, w3, dy, cnt))

    def region(w1, w2, w3, x, c):
        return F_.bmm_experts(w1, w2, w3, x, c)

    def run(fn):
        leaves = [t.clone().requires_grad_(True) for t in (W1, W2, W3, X)]
        out = fn(*leaves, CNT)
        grads = torch.autograd.grad(out, leaves, DY)
        return out, grads

    torch._dynamo.reset()
    o1, g1 = run(region)
    o2, g2 = run(torch.compile(region, backend="eager", fullgraph=True))
    assert torch.equal(o1, o2)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)


def test_scaled_backward_argument_errors_and_empty_input(dev):
    """Status codes of the C entry point itself: nothing is launched for a bad call."""
    from piper_amd import _lib
    from piper_amd._lib import PK_BF16, current_stream, ptr
    lib = _lib.load()
    E, H, I, T, K = 2, 256, 128, 16, 2
    A = T * K
    bf = dict(device=dev, dtype=torch.bfloat16)
    d_out, w2 = torch.zeros(T, H, **bf), torch.zeros(E, H, I, **bf)
    g, u, dg, du, hs = (torch.zeros(A, I, **bf) for _ in range(5))
    perm = torch.arange(A, dtype=torch.int32, device=dev)
    sc = torch.ones(T, K, device=dev)
    ds = torch.zeros(T, K, device=dev)
    starts = torch.tensor([0, A // 2, A], dtype=torch.int32, device=dev)
    need = int(lib.pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(A, I))
    assert need == (I // 64) * A * 4
    ws = torch.zeros(need // 4, device=dev)
    s = current_stream(dev)

    def call(ws_ptr, ws_bytes, rows=A, row_map=ptr(perm), div=K):
        return lib.pk_grouped_swiglu_dgrad_dh_scaled(ptr(d_out), row_map, div, ptr(sc), ptr(w2), ptr(g), ptr(u), ptr(starts),
                                                     ptr(dg), ptr(du), ptr(hs), ptr(ds), ws_ptr, ws_bytes, rows, H, I, E,
                                                     PK_BF16, s)
    assert call(ptr(ws), need) == 0
    assert call(ptr(ws), need - 4) == -4          # PK_ERR_WORKSPACE
    assert call(None, 0) == -4
    assert call(ptr(ws), need, row_map=None) == -1     # PK_ERR_ARG: the gather map is not optional here
    assert call(ptr(ws), need, div=0) == -1
    assert call(None, 0, rows=0) == 0                  # no rows: nothing to do, nothing required
    assert lib.pk_grouped_swiglu_dgrad_dh_scaled_workspace_bytes(-1, I) == -1
    torch.cuda.synchronize()


def test_grouped_gemms_replay_in_a_hip_graph(dev):
    """The persistent kernels take their work units from counters that the last workgroup of a
    launch resets: a captured graph must give the eager result on every replay, also with new
    input values and with eager launches in between."""
    counts = [300, 0, 513, 77, 128, 1, 260, 5]
    H, I = 256, 256
    x, w1, w2, w3, dy, cnt = _make(7, counts, H, I, torch.bfloat16)
    X, W1, W2, W3, DY = (t.to(dev) for t in (x, w1, w2, w3, dy))
    starts = ops.counts_to_starts(cnt.to(dev))
    E = len(counts)

    def run(xin, dyin):
        y, g, u, h = ops.grouped_swiglu_fwd(xin, W1, W2, W3, starts)
        dx, dg, du = ops.grouped_swiglu_dgrad(dyin, W1, W2, W3, g, u, starts)
        dw1, dw2, dw3 = ops.grouped_swiglu_wgrad(dyin, h, dg, du, xin, starts, E)
        return y, dx, dw1, dw2, dw3

    xs, dys = X.clone(), DY.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(xs, dys)                       # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(xs, dys)
    for rep in range(4):
        scale = 1.0 + 0.25 * rep
        xs.copy_(X * scale)
        dys.copy_(DY * (2.0 - 0.25 * rep))
        graph.replay()
        torch.cuda.synchronize()
        want = run(xs.clone(), dys.clone())            # eager, between the replays
        torch.cuda.synchronize()
        for got, ref, name in zip(outs, want, ("y", "dx", "dw1", "dw2", "dw3")):
            assert torch.equal(got, ref), f"replay {rep}: {name}"
