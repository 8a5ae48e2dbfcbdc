"""Host-side logic that needs no GPU: annotate semantics, task names, bucket planning through
the C ABI, schedules, configuration manifests."""
import math

import pytest
import torch

import piper_amd
from oracle import bucket as OB
from piper_amd import ops
from piper_amd.annotate import annotate, current_annotations, current_tag, reset_annotation_state
from piper_amd.configs import CFG1, CFG3, CFG4, bucket_manifest_cfg2, make_expert_region_inputs
from piper_amd.executor import Task, one_f_one_b
from piper_amd.tasks import TaskType


def test_annotate_indices_stack_and_errors():
    # semantics of src/piper.py:51-80: per-name auto index, global uid, nested stack
    reset_annotation_state()
    with annotate("PP") as a0:
        assert a0 == {"name": "PP", "index": 0, "uid": 0}
        with annotate("EP") as e0:
            assert e0 == {"name": "EP", "index": 0, "uid": 1}
            assert current_tag() == {"PP": 0, "EP": 0}
            assert [a["name"] for a in current_annotations()] == ["PP", "EP"]
        assert current_tag() == {"PP": 0}
    with annotate("PP") as a1:
        assert a1["index"] == 1 and a1["uid"] == 2
    assert current_annotations() == ()
    for bad in ("", None, 3):
        with pytest.raises(ValueError):
            with annotate(bad):
                pass
    reset_annotation_state()
    with annotate("PP") as a:
        assert a["index"] == 0


def test_task_type_names_match_reference():
    # src/tasks.py:8-22
    expected = {
        "FWD": "forward", "BWD": "backward", "UPD": "update", "BWD_I": "backward_input",
        "BWD_W": "backward_weight", "FWD_BWD": "forward_backward", "SEND": "send", "RECV": "recv",
        "ALL_REDUCE": "all_reduce", "REDUCE_SCATTER": "reduce_scatter", "ALL_GATHER": "all_gather",
        "FWD_A2A": "forward_a2a", "BWD_A2A": "backward_a2a", "ORDER_DUMMY": "order_dummy",
    }
    assert {t.name: t.value for t in TaskType} == expected
    assert piper_amd.TaskType is TaskType


def test_bucket_plan_c_abi_matches_oracle():
    g = torch.Generator().manual_seed(0)
    for _ in range(20):
        n = int(torch.randint(1, 40, (1,), generator=g))
        numels = [int(v) for v in torch.randint(0, 5000, (n,), generator=g)]
        for esize, align in ((2, 256), (4, 256), (2, 1), (4, 16), (2, 4096)):
            got = ops.bucket_plan(numels, esize, align)
            assert got == OB.plan_offsets(numels, esize, align)
    m = bucket_manifest_cfg2()
    numels = [math.prod(s) for _, s in m]
    offs, total = ops.bucket_plan(numels, 2, 256)
    assert (offs, total) == OB.plan_offsets(numels, 2, 256)
    assert ops.bucket_plan([], 2, 256) == ([], 0)
    with pytest.raises(RuntimeError):
        ops.bucket_plan([1, 2], 2, 3)       # alignment must be a power of two
    with pytest.raises(RuntimeError):
        ops.bucket_plan([1, -2], 2, 256)    # negative size


def test_one_f_one_b_single_rank_order():
    # pp_degree 1, 4 microbatches: F0 B0 F1 B1 F2 B2 F3 B3 U (examples/build_schedule.py:44-72)
    tasks = one_f_one_b(4, ["s0"])
    assert [(t.type, t.mb) for t in tasks[:-1]] == [
        (TaskType.FWD, 0), (TaskType.BWD, 0), (TaskType.FWD, 1), (TaskType.BWD, 1),
        (TaskType.FWD, 2), (TaskType.BWD, 2), (TaskType.FWD, 3), (TaskType.BWD, 3)]
    assert tasks[-1].type is TaskType.UPD
    two = one_f_one_b(1, ["a", "b"])
    assert [(t.type, t.ubid) for t in two] == [
        (TaskType.FWD, "a"), (TaskType.FWD, "b"), (TaskType.BWD, "b"), (TaskType.BWD, "a"), (TaskType.UPD, None)]


def test_config_shapes_and_flops():
    assert CFG3.gemm_flops_per_token == 226_492_416
    assert CFG1.gemm_flops_per_token == 4_718_592
    assert CFG3.routed_rows == 32768 and CFG4.routed_rows == 131072
    inp = make_expert_region_inputs(CFG1, microbatch=3)
    assert inp["x"].shape == (256, 256) and inp["w1"].shape == (8, 512, 256) and inp["w2"].shape == (8, 256, 512)
    assert inp["x"].dtype == torch.float32 and inp["w_gate"].dtype == torch.float32
    again = make_expert_region_inputs(CFG1, microbatch=3)
    assert all(torch.equal(inp[k], again[k]) for k in inp if inp[k] is not None)
    other = make_expert_region_inputs(CFG1, microbatch=0)
    assert torch.equal(inp["w1"], other["w1"]) and not torch.equal(inp["x"], other["x"])


def test_kernels_refuse_cpu_tensors():
    # the product path has no CPU fallback
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.route_topk(torch.zeros(4, 8), 2, True)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.bucket_zero(torch.zeros(16))


def test_annotate_is_traceable_by_dynamo_fullgraph():
    """The model's forward runs under Dynamo with fullgraph=True (src/compile.py:273): the scope
    bookkeeping must not break the graph."""
    import torch

    def fn(x):
        with annotate("PP"):
            with annotate("EP"):
                y = x + 1
        return y * 2

    reset_annotation_state()
    out = torch.compile(fn, fullgraph=True, backend="eager")(torch.ones(3))
    assert torch.equal(out, torch.full((3,), 4.0))
    assert current_annotations() == ()
