"""The drop-in operator boundary on a machine without a GPU: schema, Meta behaviour, the FX JSON
target form the reference serialises (src/fx.py:73-90) and resolves again (src/fx.py:198-212), and
capture by Dynamo with fullgraph=True (src/compile.py:273) as a single graph node."""
import pytest
import torch

from piper_amd import functional as F_


@pytest.fixture(scope="module")
def op():
    F_.register_reference_op()
    return torch.ops.piper_artifact.bmm_experts


def _meta_args(E=4, H=16, I=8, A=10, dtype=torch.bfloat16, counts_dtype=torch.int64):
    m = dict(device="meta", dtype=dtype)
    return (torch.empty(E, I, H, **m), torch.empty(E, H, I, **m), torch.empty(E, I, H, **m), torch.empty(A, H, **m),
            torch.empty(E, device="meta", dtype=counts_dtype))


def test_schema_is_the_reference_schema(op):
    schema = str(op.default._schema)
    assert schema == ("piper_artifact::bmm_experts(Tensor w1, Tensor w2, Tensor w3, Tensor x, "
                      "Tensor num_tokens_per_expert) -> Tensor")
    assert F_.register_reference_op() is False          # idempotent


@pytest.mark.parametrize("counts_dtype", [torch.int32, torch.int64])
def test_meta_kernel_returns_empty_like_x(op, counts_dtype):
    args = _meta_args(counts_dtype=counts_dtype)
    out = op(*args)
    assert out.device.type == "meta" and out.shape == args[3].shape and out.dtype == args[3].dtype


def test_fx_json_target_round_trip(op):
    # serialisation rule of the reference for op overloads: {"kind": "torch_op", "path": str(target)}
    for target in (op, op.default):
        path = str(target)
        assert path in ("piper_artifact.bmm_experts", "piper_artifact.bmm_experts.default")
        obj = torch.ops
        for part in path.split("."):                    # the reference's resolver
            obj = getattr(obj, part)
        assert obj is target


def test_dynamo_fullgraph_captures_one_node(op):
    graphs = []

    def backend(gm, example_inputs):
        graphs.append(gm)
        # the CPU has no kernel for the op: hand back a stand-in of the right structure instead of running it
        return lambda *a: (torch.empty_like(a[3]),)

    def region(w1, w2, w3, x, counts):
        return F_.bmm_experts(w1, w2, w3, x, counts)

    E, H, I, A = 4, 16, 8, 10
    args = (torch.zeros(E, I, H), torch.zeros(E, H, I), torch.zeros(E, I, H), torch.zeros(A, H),
            torch.tensor([3, 0, 5, 2]))
    torch._dynamo.reset()
    out = torch.compile(region, backend=backend, fullgraph=True)(*args)
    assert out.shape == (A, H)
    assert len(graphs) == 1
    calls = [n for n in graphs[0].graph.nodes if n.op == "call_function"]
    assert len(calls) == 1 and "piper_artifact.bmm_experts" in str(calls[0].target)
    # fake-tensor propagation went through the Meta kernel
    assert tuple(calls[0].meta["example_value"].shape) == (A, H)


def test_fused_region_and_norm_are_single_graph_nodes_under_dynamo():
    """h + moe(ffn_norm(h)) (qwen3.py:313-314) captured with fullgraph=True: two opaque calls."""
    graphs = []

    def backend(gm, example_inputs):
        graphs.append(gm)
        return lambda *a: (torch.empty_like(a[0]),)

    def block(h, nw, wg, w1, w2, w3):
        return F_.moe_block(h, nw, wg, None, w1, w2, w3, top_k=2, route_norm=True)

    T, H, E, I = 6, 16, 4, 8
    args = (torch.zeros(T, H), torch.ones(H), torch.zeros(E, H), torch.zeros(E, I, H), torch.zeros(E, H, I),
            torch.zeros(E, I, H))
    torch._dynamo.reset()
    out = torch.compile(block, backend=backend, fullgraph=True)(*args)
    assert out.shape == (T, H)
    assert len(graphs) == 1
    targets = [str(n.target) for n in graphs[0].graph.nodes if n.op == "call_function"]
    assert sum("piper_amd.rmsnorm" in t for t in targets) == 1
    assert sum("piper_amd.expert_region" in t for t in targets) == 1


def test_region_ops_refuse_real_cpu_tensors():
    T, H, E, I = 6, 16, 4, 8
    with pytest.raises((RuntimeError, ValueError)):
        F_.expert_region(torch.zeros(T, H), torch.zeros(E, H), None, torch.zeros(E, I, H), torch.zeros(E, H, I),
                         torch.zeros(E, I, H), top_k=2, route_norm=True)
