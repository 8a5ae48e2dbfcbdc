"""pk_sort_by_expert_static: the counting sort for callers that cannot allocate (its per-chunk
histograms live in a fixed array inside the library).  Called through the C ABI and compared bit
for bit with pk_sort_by_expert, on two calls in a row, the second with a smaller input, so that
whatever the first call left in the shared array is there when the second one runs."""
import ctypes as C

import pytest
import torch

from piper_amd import _lib

pytestmark = pytest.mark.gpu

PK_ERR_WORKSPACE = -4
PK_SORT_STATIC_WORDS = 256 * 1024


def _outputs(A, E, dev):
    mk = lambda n: torch.full((n,), -7, dtype=torch.int32, device=dev)
    return dict(counts=mk(E), starts=mk(E + 1), perm=mk(A), inv_perm=mk(A), order=mk(E))


def _p(t):
    return C.c_void_p(t.data_ptr())


def _run_both(top_idx, E, dev):
    lib = _lib.load()
    A = top_idx.numel()
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    ref = _outputs(A, E, dev)
    ws_bytes = lib.pk_sort_workspace_bytes(A, E)
    ws = torch.empty(max(int(ws_bytes), 4), dtype=torch.uint8, device=dev)
    rc = lib.pk_sort_by_expert(_p(top_idx), A, E, _p(ref["counts"]), _p(ref["starts"]), _p(ref["perm"]),
                               _p(ref["inv_perm"]), _p(ref["order"]), _p(ws), ws.numel(), stream)
    assert rc == 0
    got = _outputs(A, E, dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    rc = lib.pk_sort_by_expert_static(_p(top_idx), A, E, _p(got["counts"]), _p(got["starts"]), _p(got["perm"]),
                                      _p(got["inv_perm"]), _p(got["order"]), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    for name in ref:
        assert torch.equal(ref[name], got[name]), name
    return got


def test_static_sort_matches_workspace_sort_twice_in_a_row(dev):
    g = torch.Generator().manual_seed(0)
    E = 128
    # first call: 16384 tokens x top-8 with a skewed expert distribution and an empty expert
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -1.2
    p[17] = 0.0
    big = torch.multinomial(p, 16384 * 8, replacement=True, generator=g).to(torch.int32).to(dev)
    print("[case] static sort A=131072 E=128", flush=True)
    out = _run_both(big, E, dev)
    assert out["counts"][17].item() == 0 and out["starts"][E].item() == big.numel()
    # second call, smaller and ragged (not a multiple of the 512-slot chunk), fewer experts
    mid = torch.randint(0, 120, (60003,), generator=g, dtype=torch.int32).to(dev)
    print("[case] static sort A=60003 E=120", flush=True)
    out = _run_both(mid, 120, dev)
    assert out["starts"][120].item() == mid.numel()
    import numpy as np
    assert np.array_equal(out["perm"].cpu().numpy(), np.argsort(mid.cpu().numpy(), kind="stable").astype(np.int32))
    # third call: a short input
    small = torch.randint(0, 8, (1000 * 2 + 3,), generator=g, dtype=torch.int32).to(dev)
    print("[case] static sort A=2003 E=8", flush=True)
    out = _run_both(small, 8, dev)
    assert out["starts"][8].item() == small.numel()
    # oracle for the third call: numpy's stable argsort
    ref_perm = np.argsort(small.cpu().numpy(), kind="stable").astype(np.int32)
    assert np.array_equal(out["perm"].cpu().numpy(), ref_perm)


def test_static_sort_rejects_inputs_beyond_its_scratch(dev):
    lib = _lib.load()
    E = 1024
    A = (PK_SORT_STATIC_WORDS // E + 1) * 512            # one chunk too many
    idx = torch.zeros(A, dtype=torch.int32, device=dev)
    o = _outputs(A, E, dev)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    rc = lib.pk_sort_by_expert_static(_p(idx), A, E, _p(o["counts"]), _p(o["starts"]), _p(o["perm"]), _p(o["inv_perm"]),
                                      _p(o["order"]), stream)
    assert rc == PK_ERR_WORKSPACE
    torch.cuda.synchronize()
    assert all((t == -7).all().item() for t in o.values())   # nothing was launched
    # the largest input that fits is accepted
    A_ok = (PK_SORT_STATIC_WORDS // E) * 512
    o = _outputs(A_ok, E, dev)
    rc = lib.pk_sort_by_expert_static(_p(idx[:A_ok]), A_ok, E, _p(o["counts"]), _p(o["starts"]), _p(o["perm"]),
                                      _p(o["inv_perm"]), _p(o["order"]), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert o["counts"][0].item() == A_ok and o["starts"][E].item() == A_ok
    assert torch.equal(o["perm"], torch.arange(A_ok, dtype=torch.int32, device=dev))


def test_static_sort_recorded_into_a_hip_graph(dev):
    """Two static sorts recorded into one HIP graph (after pk_init on the device, as the header
    asks: a symbol look-up is not legal while a stream is capturing) and replayed with new inputs,
    with eager work between the replays; every replay against pk_sort_by_expert on the same inputs."""
    lib = _lib.load()
    _lib.init_device()
    g = torch.Generator().manual_seed(3)
    shapes = [(8192 * 8, 128), (1000 * 2 + 3, 8)]
    inputs = [torch.zeros(A, dtype=torch.int32, device=dev) for A, _ in shapes]
    outs = [_outputs(A, E, dev) for A, E in shapes]

    def fill():
        for buf, (A, E) in zip(inputs, shapes):
            buf.copy_(torch.randint(0, E, (A,), generator=g, dtype=torch.int32))

    def static_sorts():
        stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        for buf, o, (A, E) in zip(inputs, outs, shapes):
            rc = lib.pk_sort_by_expert_static(_p(buf), A, E, _p(o["counts"]), _p(o["starts"]), _p(o["perm"]),
                                              _p(o["inv_perm"]), _p(o["order"]), stream)
            assert rc == 0

    fill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        static_sorts()                     # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    print("[case] static sort under graph capture", flush=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_sorts()
    for rep in range(3):
        fill()
        for o in outs:
            for t in o.values():
                t.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        for buf, o, (A, E) in zip(inputs, outs, shapes):       # eager, between the replays
            ref = _outputs(A, E, dev)
            ws = torch.empty(max(int(lib.pk_sort_workspace_bytes(A, E)), 4), dtype=torch.uint8, device=dev)
            rc = lib.pk_sort_by_expert(_p(buf), A, E, _p(ref["counts"]), _p(ref["starts"]), _p(ref["perm"]),
                                       _p(ref["inv_perm"]), _p(ref["order"]), _p(ws), ws.numel(),
                                       C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
            assert rc == 0
            torch.cuda.synchronize()
            for name in ref:
                assert torch.equal(ref[name], o[name]), f"replay {rep}: {name} (A={A}, E={E})"
