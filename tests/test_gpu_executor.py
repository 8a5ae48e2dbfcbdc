"""One-GPU pipeline-stage emulation through the executor: two MoE layers (two buckets) run 4
microbatches in 1F1B order, parameters live in ZeRO buckets, gradient packing runs on a second
stream after every backward, one fused AdamW step closes the iteration.  Compared with the CPU
oracle doing the same thing with torch autograd and torch.optim.AdamW."""
import pytest
import torch

from conftest import ADAMW_TOL, BF16_TOL, F32_TOL, rel_err
from oracle import bucket as OB
from oracle import moe as O
from piper_amd import functional as F_
from piper_amd.bucket import BucketState, ParamStorage, StageStore, flatten_params
from piper_amd.configs import ADAMW
from piper_amd.executor import StageExecutor, Task, one_f_one_b
from piper_amd.optim import FusedAdamW
from piper_amd.tasks import TaskType

pytestmark = pytest.mark.gpu

T, H, I, E, K, MB = 128, 256, 128, 8, 2, 4
NAMES = ("w_gate", "w1", "w3", "w2")


def _init(seed, dtype):
    g = torch.Generator().manual_seed(seed)
    layers = []
    for _ in range(2):
        layers.append(dict(w_gate=torch.randn(E, H, generator=g) * 0.02,
                           w1=(torch.randn(E, I, H, generator=g) * 0.02).to(dtype),
                           w3=(torch.randn(E, I, H, generator=g) * 0.02).to(dtype),
                           w2=(torch.randn(E, H, I, generator=g) * 0.02).to(dtype)))
    xs = [torch.randn(T, H, generator=g).to(dtype) for _ in range(MB)]
    return layers, xs


def _oracle_iteration(layers, xs, dtype):
    params = [{k: v.clone().float().requires_grad_(True) for k, v in l.items()} for l in layers]
    losses = []
    for x in xs:
        h = x.float()
        for p in params:
            y, _ = O.moe_forward(h, p["w_gate"], None, p["w1"], p["w2"], p["w3"], K, True, compute_dtype=torch.float32)
            h = h + y
        loss = h.sum()
        loss.backward()
        losses.append(loss.detach())
    return params, losses


def _make_executor(layers, xs, dev, dtype, two_streams):
    """Two MoE layers as two compute buckets (+ fp32 gate buckets when the experts are bf16)."""
    store = StageStore()
    for ubid, l in enumerate(layers):
        b = BucketState()
        # gate (fp32) and experts (param dtype) live in separate buckets when the dtypes differ
        plist = [torch.nn.Parameter(l[k].to(dev)) for k in NAMES]
        b.forward_args = [None] + plist
        b.input_idxs = [0]
        b.param_idxs = [1, 2, 3, 4]
        b.trainable_param_idxs = [1, 2, 3, 4]
        b.param_names = list(NAMES)

        def fwd(args):
            x, wg, w1, w3, w2 = args
            return x + F_.expert_region(x, wg, None, w1, w2, w3, top_k=K, route_norm=True)

        b.forward_fn = fwd
        store.buckets[ubid] = b
        store.zero_managed_ubids.add(ubid)
    # flatten: one bucket per dtype group of each stage (the reference flattens per bucket, src/actor.py:532)
    opt = lambda ps: FusedAdamW(ps, **ADAMW)
    extra = []
    for ubid, b in list(store.buckets.items()):
        experts = [b.forward_args[i] for i in (2, 3, 4)]
        gate = [b.forward_args[1]]
        if dtype == torch.float32:
            flatten_params(b, gate + experts, optim_class=opt)
        else:
            flatten_params(b, experts, optim_class=opt)
            gb = BucketState()
            flatten_params(gb, gate, optim_class=opt)
            extra.append((f"gate{ubid}", gb))
    for name, gb in extra:
        store.buckets[name] = gb
        store.zero_managed_ubids.add(name)

    compute_ubids = [0, 1]
    # gate buckets have no forward of their own: they are packed right after their stage's backward
    ex = StageExecutor(store, compute_stream=torch.cuda.Stream() if two_streams else None,
                       pack_stream=torch.cuda.Stream() if two_streams is True else None)
    # the executor walks store.buckets in order for FWD chaining: restrict chaining to compute buckets
    ex_ubids = compute_ubids

    # run: reuse StageExecutor.run with a store view that only chains the compute buckets
    class View(StageStore):
        pass
    view = View(buckets={u: store.buckets[u] for u in ex_ubids}, zero_managed_ubids=set(ex_ubids))
    ex.stages = view
    ex.params = ParamStorage(store)          # storage covers every bucket (incl. gate buckets)
    ex.compute.stages = view
    mbs = [x.to(dev).requires_grad_(False) for x in xs]

    # gate-bucket packing hooks: pack after each backward of its stage
    orig_acc = ex.params.accumulate_zero_param_grads_to_flat

    def acc(ubid, stream=None):
        orig_acc(ubid, stream)
        if f"gate{ubid}" in store.buckets:
            orig_acc(f"gate{ubid}", stream)
    ex.params.accumulate_zero_param_grads_to_flat = acc

    return store, ex, mbs, compute_ubids


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("two_streams", [True, False])
def test_two_bucket_1f1b_iteration(dev, dtype, two_streams):
    print(f"[case] executor {dtype} two_streams={two_streams}", flush=True)
    layers, xs = _init(0, dtype)
    ref_params, ref_losses = _oracle_iteration(layers, xs, dtype)

    store, ex, mbs, compute_ubids = _make_executor(layers, xs, dev, dtype, two_streams)
    tasks = one_f_one_b(MB, compute_ubids)
    out = ex.run(tasks, mbs)
    torch.cuda.synchronize()
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    for got, ref in zip(out["losses"], ref_losses):
        assert abs(got.item() - ref.item()) <= max(tol * abs(ref.item()), 0.05 if dtype == torch.bfloat16 else 1e-2)

    # bucket contents = accumulated gradients of 4 microbatches
    for ubid in compute_ubids:
        b = store.buckets[ubid]
        for (p, off, n, shape), name in zip(b.param_view_specs, NAMES if dtype == torch.float32 else NAMES[1:]):
            ref_g = ref_params[ubid][name].grad
            got_g = b.flat_grads[off:off + n].view(shape)
            # after the update the grads are still in the bucket (zeroed at the start of the next iteration)
            assert rel_err(got_g, ref_g) <= (1e-4 if dtype == torch.float32 else 4 * BF16_TOL), name
        # optimizer: given the bucket's own gradient, master == torch.optim.AdamW to 1e-6
        st = b.shard_optimizer.state[b.shard_param]
        assert st["step"] == 1
        names = NAMES if dtype == torch.float32 else NAMES[1:]
        offs = [s[1] for s in b.param_view_specs]
        master0 = OB.flatten([layers[ubid][k] for k in names], offs, b.flat_params.numel(), torch.float32)
        z = torch.zeros_like(master0)
        ref_master, _, _ = OB.adamw_step_torch(master0, b.flat_grads.cpu(), z, z, 1, ADAMW["lr"], ADAMW["betas"],
                                               ADAMW["eps"], ADAMW["weight_decay"])
        assert (st["master"].cpu() - ref_master).abs().max().item() <= ADAMW_TOL
        # parameters are views of the updated bucket
        for (p, off, n, shape) in b.param_view_specs:
            assert p.data_ptr() == b.flat_params.data_ptr() + off * b.flat_params.element_size()
            assert torch.equal(p.detach().reshape(-1).cpu(), ref_master[off:off + n].to(dtype)) or \
                rel_err(p.detach().reshape(-1), ref_master[off:off + n]) <= 1e-2
        assert all(p.grad is None for p, *_ in b.param_view_specs)


def _buckets_after(layers, xs, dev, dtype, streams, tasks_of):
    store, ex, mbs, ubids = _make_executor(layers, xs, dev, dtype, streams)
    out = ex.run(tasks_of(ubids), mbs)
    torch.cuda.synchronize()
    return out["losses"], {u: (store.buckets[u].flat_grads.clone(), store.buckets[u].flat_params.clone()) for u in store.buckets}


def _assert_same_buckets(ref, got):
    (l0, b0), (l1, b1) = ref, got
    assert len(l0) == len(l1) and all(torch.equal(a, b) for a, b in zip(l0, l1))
    for u in b0:
        assert torch.equal(b0[u][0], b1[u][0]), f"gradient bucket {u}"
        assert torch.equal(b0[u][1], b1[u][1]), f"parameter bucket {u}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compute_stream_without_pack_stream(dev, dtype):
    """Only a compute stream: backward and gradient pack share it, and it first waits for the
    caller's stream, which produced the microbatches.  Same buckets, bit for bit, as on one stream."""
    print(f"[case] compute stream only {dtype}", flush=True)
    layers, xs = _init(3, dtype)
    ref = _buckets_after(layers, xs, dev, dtype, False, lambda ubids: one_f_one_b(MB, ubids))
    got = _buckets_after(layers, xs, dev, dtype, "compute only", lambda ubids: one_f_one_b(MB, ubids))
    _assert_same_buckets(ref, got)


@pytest.mark.parametrize("name, stages", [("schedule_pp1_1f1b_mb4.json", 1), ("schedule_pp1_zerobubble_mb4.json", 1),
                                          ("schedule_pp2_zerobubble_mb4.json", 2)])
def test_schedule_file_drives_the_executor(dev, name, stages):
    """A schedule file in the reference's format (src/schedule.py:6-99) becomes the task list of
    the one device and gives the same buckets as the hand-built 1F1B list."""
    import os
    from piper_amd.schedule import device_tasks, load_schedule_directives
    print(f"[case] schedule file {name}", flush=True)
    directives = load_schedule_directives(os.path.join(os.path.dirname(__file__), "golden", name))
    layers, xs = _init(4, torch.float32)
    ref = _buckets_after(layers, xs, dev, torch.float32, False, lambda ubids: one_f_one_b(MB, ubids))

    def tasks_of(ubids):
        stage_ubids = [list(ubids)] if stages == 1 else [[u] for u in ubids]
        tasks = device_tasks(directives, stage_ubids)
        assert tasks[-1].type is TaskType.UPD
        return tasks

    got = _buckets_after(layers, xs, dev, torch.float32, True, tasks_of)
    # the losses come out in the order the last stage's backward passes run; every schedule here
    # runs them by ascending microbatch
    _assert_same_buckets(ref, got)


def test_comm_tasks_are_noops_and_unknown_bucket_raises(dev):
    store = StageStore()
    ex = StageExecutor(store)
    out = ex.run([Task(TaskType.SEND), Task(TaskType.ALL_GATHER), Task(TaskType.ORDER_DUMMY)], [])
    assert out["losses"] == []
    with pytest.raises(KeyError):
        store.bucket("missing")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_split_backward_tasks_match_whole_backward(dev, dtype):
    """BWD_I + BWD_W (src/executors.py:353-476) in a zero-bubble-like order give the same gradient
    buckets and the same update as whole BWD tasks: the weight pass runs the same kernels later."""
    print(f"[case] split backward {dtype}", flush=True)
    layers, xs = _init(1, dtype)
    results = []
    for split in (False, True):
        store, ex, mbs, ubids = _make_executor(layers, xs, dev, dtype, False)
        tasks = []
        for mb in range(MB):
            tasks += [Task(TaskType.FWD, u, mb) for u in ubids]
            if split:   # all input gradients first, then the weight gradients (any order is allowed)
                tasks += [Task(TaskType.BWD_I, u, mb) for u in reversed(ubids)]
                tasks += [Task(TaskType.BWD_W, u, mb) for u in ubids]
            else:
                tasks += [Task(TaskType.BWD, u, mb) for u in reversed(ubids)]
        tasks.append(Task(TaskType.UPD))
        out = ex.run(tasks, mbs)
        torch.cuda.synchronize()
        results.append((out["losses"], {u: (store.buckets[u].flat_grads.clone(), store.buckets[u].flat_params.clone())
                                        for u in store.buckets}))
    (l0, b0), (l1, b1) = results
    for a, b in zip(l0, l1):
        assert torch.equal(a, b)
    for u in b0:
        assert torch.equal(b0[u][0], b1[u][0]), f"gradient bucket {u}"
        assert torch.equal(b0[u][1], b1[u][1]), f"parameter bucket {u}"


def test_weight_grad_queue_accumulates_into_existing_grads(dev):
    """Without packing in between, the weight pass adds to .grad like the reference's weight pass."""
    layers, xs = _init(2, torch.float32)
    l = layers[0]
    ps = {k: torch.nn.Parameter(l[k].to(dev)) for k in NAMES}
    x = xs[0].to(dev)

    def run(deferred):
        for p in ps.values():
            p.grad = None
        for _ in range(2):
            out = F_.expert_region(x, ps["w_gate"], None, ps["w1"], ps["w2"], ps["w3"], top_k=K, route_norm=True)
            if deferred:
                with F_.defer_weight_grads() as q:
                    out.sum().backward()
                assert len(q) == 2 and (ps["w1"].grad is None or _ == 1)
                q.run()
            else:
                out.sum().backward()
        return {k: p.grad.clone() for k, p in ps.items()}

    ref, got = run(False), run(True)
    for k in NAMES:
        assert rel_err(got[k], ref[k]) <= 1e-6, k
