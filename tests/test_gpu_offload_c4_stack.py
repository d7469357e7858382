"""Two layers of the offloaded-expert configuration at its real shape (each: 4096 tokens x 4096, 32 experts of
4096 -> 14336 -> 4096 in bf16 from pinned host memory, top-2, no drop; 30 GB of pinned host memory in all) over
one pool of 48 slots - fewer than the two layers' 64 experts, so slots are recycled through the prefetch stack and
one layer's compute hides fetches for the other.  Checked: the scheduler's profiling window measures the layers and
plans local and cross-layer prefetch from what it measured - the plan equals the planner fed the same numbers by
hand - and the steps that run under that plan, and under a hand-fed plan with cross-layer counts in both
directions, give the output, the input gradient and all 2 x 4 x 32 host gradients of the step without any
prefetch, bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu

S, M, E, K, FD = 4096, 4096, 32, 2, 14336
POOL, EBATCH, LAYERS = 48, 8, 2


@pytest.fixture(scope="module")
def stack():
    from mole_amd.moe.layer import MOLEModule
    from mole_amd.utils import Uparam
    from mole_amd.utils.Uscheduler import UniScheduler
    print("c4 stack: pinning 30 GB of host memory", flush=True)
    MOLEModule.reset_instances()
    UniScheduler.reset()
    keep = Uparam._init_
    Uparam._init_ = lambda *a, **kw: None      # the weights are drawn on the GPU below, not 7.6e9 numbers on the host
    try:
        layers = [MOLEModule(E, 0, M, FD, POOL, K, EBATCH, {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", 1, False,
                             True, dtype=torch.bfloat16) for _ in range(LAYERS)]
    finally:
        Uparam._init_ = keep
    g = torch.Generator(device="cuda").manual_seed(0)
    for m in layers:
        for cp in (m.FC1_W_CPU, m.FC1_B_CPU, m.FC2_W_CPU, m.FC2_B_CPU):
            for e0 in range(0, E, 8):
                cp.all_tensors[e0:e0 + 8].copy_((torch.randn(8, *cp.size, device="cuda", generator=g) * 0.02).bfloat16())
        with torch.no_grad():
            m.gate[0].linear.weight.copy_(torch.randn(E, M, device="cuda", generator=g) * 0.02)
    torch.cuda.synchronize()
    yield layers
    MOLEModule.reset_instances()
    UniScheduler.reset()


def _train_step(layers, x, dy, i=None):
    """One step the way a training loop drives the scheduler; i = None: no scheduler policy, no prefetch."""
    from mole_amd import core
    from mole_amd.utils.Uscheduler import UniScheduler
    time_it = prefetch = False
    if i is not None:
        UniScheduler.set_step(i)
        time_it, prefetch = UniScheduler.time_it(), UniScheduler.prefetch_it()
        UniScheduler.prefetch_fwd()
    xin = x.clone().requires_grad_(True)
    h = xin
    for m in layers:
        h = m(h, capacity_factor=0.0, time_it=time_it, prefetch=prefetch)
    h.backward(dy)
    torch.cuda.synchronize(); core.synchronize_tran()
    um = core.get_UniMem()
    assert um.virtual_offset() == 0 and um.view_pool_size() == POOL
    plan = UniScheduler.profile_prefetch() if i is not None else None
    grads = [t.grad_.cuda() for m in layers for t in m.d_experts_param()]
    for m in layers:
        m.gate[0].linear.weight.grad = None
    return h.detach().clone(), xin.grad.clone(), grads, plan


def _same(got, want, what):
    assert torch.equal(got[0], want[0]), f"{what}: output"
    assert torch.equal(got[1], want[1]), f"{what}: input gradient"
    for j, (a, b) in enumerate(zip(got[2], want[2])):
        assert torch.equal(a, b), f"{what}: host gradient array {j}"


def test_c4_stack_measured_plan_and_cross_layer_prefetch(stack):
    from mole_amd.utils.Uscheduler import UniScheduler, plan_prefetch
    layers = stack
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(S, M, device="cuda", generator=g).bfloat16()
    dy = (torch.randn(S, M, device="cuda", generator=g) * 1e-2).bfloat16()
    print("c4 stack: plain step", flush=True)
    want = _train_step(layers, x, dy)
    assert all(int((m.last_route.kept_rows > 0).sum()) == E for m in layers)
    assert float(want[0].float().abs().max()) > 0 and all(float(gr.float().abs().max()) > 0 for gr in want[2])

    UniScheduler.schedule_policy(profile_step=4, prefetch_on=True, deactivate_first_prefetch=False, prefetch_floor=True,
                                 global_prefetch=True)
    plans = []
    for i in range(4):
        print(f"c4 stack: profiled step {i}", flush=True)
        got = _train_step(layers, x, dy, i)
        plans.append(got[3])
        _same(got, want, f"profiled step {i}")
    assert [p is not None for p in plans] == [False, False, True, True]
    fwd, bwd, ftime = UniScheduler.fwd_stat, UniScheduler.bwd_stat, UniScheduler.ftime
    print(f"c4 stack: measured forward {fwd} s, backward {bwd} s (last layer first), one expert's fetch {ftime} s", flush=True)
    # a forward pass takes at least the time its 7.5 GB of experts need on the bus (the last layer's backward finds
    # most of them still in the pool from its forward); one expert is 235 MB
    assert len(fwd) == len(bwd) == LAYERS and all(t > 0.05 for t in fwd) and all(t > 0 for t in bwd) and 1e-3 < ftime < 0.1
    by_hand = plan_prefetch(POOL, fwd, bwd, ftime, [E] * LAYERS, prefetch_floor=True, deactivate_first_prefetch=False,
                            global_prefetch=True)
    print(f"c4 stack: measured plan {by_hand}", flush=True)
    assert plans[3] == by_hand == UniScheduler.last_plan
    assert [m.local_prefetch_fwd_count for m in layers] == [p["local_fwd"] for p in by_hand]
    assert [m.global_prefetch_fwd_count for m in layers] == [p["global_fwd"] for p in by_hand]
    assert any(p["local_fwd"] for p in by_hand) and any(p["local_bwd"] for p in by_hand)
    for i in (5, 6):
        print(f"c4 stack: step {i} under the measured plan", flush=True)
        assert UniScheduler.prefetch_it() or i == 5
        _same(_train_step(layers, x, dy, i), want, f"step {i} under the measured plan")

    # a plan with cross-layer counts in both directions, whatever the box measured: 40 fetches fit under the first
    # layer's forward (8 more than it has experts: they go to the second layer's), 8 under the second's, and the
    # mirror image on the way back
    plan = UniScheduler.set_prefetch_scheme(fwd_stat=[40.0, 8.0], bwd_stat=[40.0, 8.0], ftime=1.0, prefetch_floor=True,
                                            global_prefetch=True)
    print(f"c4 stack: hand-fed plan {plan}", flush=True)
    assert plan[0]["global_fwd"] == [[1, 8]] and plan[1]["global_bwd"] == [[0, 8]]
    for i in (7, 8):
        print(f"c4 stack: step {i} under the hand-fed cross-layer plan", flush=True)
        _same(_train_step(layers, x, dy, i), want, f"step {i} under the cross-layer plan")
