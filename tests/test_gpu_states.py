"""Checkpoint files and the scheduler's profiling window on the GPU: UniScheduler.save_states / load_states against
the committed fixture in the reference's file layout, and the measured prefetch plan against the planner fed by hand."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import rel_err

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _layer(s_experts, d_experts, adv_adam=False, seed=0):
    from mole_amd.moe.layer import MOLEModule
    torch.manual_seed(seed)
    z = np.load(os.path.join(GOLD, "layer_small.npz"))
    M, F = z["x"].shape[1], z["w1"].shape[1]
    m = MOLEModule(d_experts, s_experts, M, F, d_experts if d_experts else -1, 2, 2,
                   {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", 1, adv_adam, d_experts > 0, dtype=torch.float32)
    return m, z


@pytest.mark.parametrize("s_experts,d_experts", [(4, 0), (2, 2), (0, 4)])
def test_load_states_reads_the_reference_layout_and_save_states_writes_it_back(s_experts, d_experts, tmp_path):
    """The fixture lists its experts GPU-resident first, then offloaded (MOLE/moe/layer.py:403-410): loaded into a
    layer of any split, the layer computes the oracle's output for the fixture's weights, holds the fixture's
    gradients, and a file saved from it equals the fixture entry by entry."""
    from mole_amd import core
    from mole_amd.moe.layer import MOLEModule
    from mole_amd.utils.Uscheduler import UniScheduler
    print(f"states s={s_experts} d={d_experts}", flush=True)
    MOLEModule.reset_instances()
    UniScheduler.reset()
    m, z = _layer(s_experts, d_experts)
    x = torch.from_numpy(z["x"]).cuda()
    y_before = m(x, capacity_factor=1.0).detach().clone()
    want = UniScheduler.load_states(os.path.join(GOLD, "MOLE_states_tiny"), grad=True)
    y = m(x, capacity_factor=1.0).detach()
    assert rel_err(y, torch.from_numpy(z["y"])) < 1e-5 and rel_err(y_before, torch.from_numpy(z["y"])) > 1e-2
    # the loaded gradients are where the optimizer reads them: device buffers for GPU-resident experts, pinned host
    # arrays for offloaded ones, .grad of the gate weight
    E = s_experts + d_experts
    names = ("tanh/g_w1", "tanh/g_b1", "tanh/g_w2", "tanh/g_b2")
    for gp, cp, name in zip((m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU),
                            (m.FC1_W_CPU, m.FC1_B_CPU, m.FC2_W_CPU, m.FC2_B_CPU), names):
        if s_experts:
            assert np.array_equal(gp.grad_tensors.cpu().numpy(), z[name][:s_experts])
        if d_experts:
            assert np.array_equal(cp.all_tensors.grad_.numpy(), z[name][s_experts:])
    assert np.array_equal(m.gate[0].linear.weight.grad.cpu().numpy(), z["tanh/dwg"])
    # a backward pass from the loaded weights reproduces the fixture's gradients (they are the oracle's)
    m.gate[0].linear.weight.grad = None
    xin = x.clone().requires_grad_(True)
    m(xin, capacity_factor=1.0).backward(torch.from_numpy(z["dy"]).cuda())
    torch.cuda.synchronize(); core.synchronize_tran()
    assert rel_err(xin.grad, torch.from_numpy(z["tanh/dx"])) < 1e-5
    # save, then read the file the way the fixture is read: same structure, same order, same values
    UniScheduler.save_states(str(tmp_path / "states"), grad=True)
    got = torch.load(str(tmp_path / "states.pt"), map_location="cpu", weights_only=True)
    assert len(got) == 2 and len(got[0]) == 1 and got[1] == [None, None]
    a, b = got[0][0], want[0][0]
    assert sorted(a) == sorted(b) == ["experts", "gate", "grad"]
    assert torch.equal(a["gate"][0], b["gate"][0]) and a["gate"][1] is None
    assert len(a["experts"]) == E and len(a["grad"]) == E + 2 and a["grad"][E + 1] is None
    for e in range(E):
        for u, v in zip(a["experts"][e], b["experts"][e]):
            assert torch.equal(u, v)
        for u, v, name in zip(a["grad"][e], b["grad"][e], names):
            assert rel_err(u, v) < 1e-5, f"gradient {name} of expert {e} after the backward pass"
    assert rel_err(a["grad"][E], b["grad"][E]) < 1e-5
    MOLEModule.reset_instances()


def test_optimizer_state_of_the_in_pipeline_adam_round_trips_through_a_file(tmp_path):
    """The fp32 moments of the offloaded experts and the step counter, in the reference's [expert_state, gate_state]
    layout (MOLE/optim/mixed_optim.py:245-277), survive save_states / load_states into a freshly built layer, and
    the next in-pipeline update continues from them: parameters after the step equal those of the uninterrupted run."""
    from mole_amd import core
    from mole_amd.moe.layer import MOLEModule
    from mole_amd.utils.Uscheduler import UniScheduler
    print("states adam", flush=True)

    def params(m):
        return [cp.all_tensors for cp in (m.FC1_W_CPU, m.FC1_B_CPU, m.FC2_W_CPU, m.FC2_B_CPU)]

    def step(m, x, t):
        m.MOLECore.set_adam(0.9, 0.999, t, 1e-2, 0.01, 1e-8, True, -1)
        xin = x.clone().requires_grad_(True)
        y = m(xin, capacity_factor=1.0)
        y.backward(y.detach() * 1e-1)
        torch.cuda.synchronize(); core.synchronize_tran()

    MOLEModule.reset_instances(); UniScheduler.reset()
    m, z = _layer(0, 4, adv_adam=True, seed=3)
    x = torch.from_numpy(z["x"]).cuda()
    step(m, x, 0)
    UniScheduler.save_states(str(tmp_path / "adam"), grad=False)
    saved = torch.load(str(tmp_path / "adam.pt"), map_location="cpu", weights_only=True)
    assert sorted(saved[1][0]) == [0, 1, 2, 3] and saved[1][1] is None
    assert saved[1][0][0]["step"] == 1 and saved[1][0][2]["exp_avg"].shape == params(m)[2].shape
    assert float(saved[1][0][0]["exp_avg_sq"].abs().max()) > 0
    step(m, x, 1)
    want = [p.clone() for p in params(m)] + [p.momentum.clone() for p in params(m)]
    MOLEModule.reset_instances()
    m2, _ = _layer(0, 4, adv_adam=True, seed=99)
    m2.MOLECore.set_adam(0.9, 0.999, 0, 1e-2, 0.01, 1e-8, True, -1)
    UniScheduler.load_states(str(tmp_path / "adam"), grad=False)
    assert m2.MOLECore.adam[2] == 1          # one step done: the counter the next step starts from
    step(m2, x, 1)
    got = [p.clone() for p in params(m2)] + [p.momentum.clone() for p in params(m2)]
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    MOLEModule.reset_instances()


def test_profiling_window_plans_from_measured_times():
    """schedule_policy / set_step / time_it / profile_prefetch on a small stack: inside the window the layers record
    forward and backward spans, the scheduler folds them and the measured fetch time into running means, and the
    plan it applies equals plan_prefetch fed the same numbers by hand; after the window prefetch_it() turns on and
    the prefetched steps give the results of the plain ones bit for bit."""
    from mole_amd import core
    from mole_amd.moe.layer import MOLEModule
    from mole_amd.utils.Uscheduler import UniScheduler, plan_prefetch
    print("profiling window", flush=True)
    S, M, E, k, Fd, n_layers, pool = 256, 64, 4, 2, 128, 3, 6
    MOLEModule.reset_instances(); UniScheduler.reset()
    torch.manual_seed(5)
    dist = {"local_rank": 0, "world_size": 1, "rank": 0}
    layers = [MOLEModule(E, 0, M, Fd, pool, k, 2, dist, "gelu", 1, False, True, dtype=torch.float32) for _ in range(n_layers)]
    x = torch.randn(S, M, generator=torch.Generator().manual_seed(1)).cuda()
    UniScheduler.schedule_policy(profile_step=4, prefetch_on=True, deactivate_first_prefetch=False, prefetch_floor=False,
                                 global_prefetch=True)

    def train_step(i):
        UniScheduler.set_step(i)
        xin = x.clone().requires_grad_(True)
        UniScheduler.prefetch_fwd()
        h = xin
        for m in layers:
            h = m(h, capacity_factor=0.0, time_it=UniScheduler.time_it(), prefetch=UniScheduler.prefetch_it())
        h.backward(torch.ones_like(h) * 1e-2)
        torch.cuda.synchronize(); core.synchronize_tran()
        plan = UniScheduler.profile_prefetch()
        grads = [t.grad_.clone() for m in layers for t in m.d_experts_param()]
        return h.detach().clone(), xin.grad.clone(), grads, plan

    results = [train_step(i) for i in range(7)]
    # steps 0 and 1 are inside the window but too early to be counted; 2 and 3 are measured; 4.. are not timed
    assert [r[3] is not None for r in results] == [False, False, True, True, False, False, False]
    assert len(UniScheduler.fwd_stat) == n_layers and len(UniScheduler.bwd_stat) == n_layers
    assert all(t > 0 for t in UniScheduler.fwd_stat + UniScheduler.bwd_stat) and UniScheduler.ftime > 0
    by_hand = plan_prefetch(pool, UniScheduler.fwd_stat, UniScheduler.bwd_stat, UniScheduler.ftime, [E] * n_layers,
                            prefetch_floor=False, deactivate_first_prefetch=False, global_prefetch=True)
    assert results[3][3] == by_hand == UniScheduler.last_plan
    assert [m.local_prefetch_fwd_count for m in layers] == [p["local_fwd"] for p in by_hand]
    assert UniScheduler.prefetch_it() and not UniScheduler.time_it()
    um = core.get_UniMem()
    assert um.virtual_offset() == 0
    for r in results[5:]:                 # prefetched steps against the plain step 0
        assert torch.equal(r[0], results[0][0]) and torch.equal(r[1], results[0][1])
        for a, b in zip(r[2], results[0][2]):
            assert torch.equal(a, b)
    MOLEModule.reset_instances(); UniScheduler.reset()
