"""Prefetch planning (mole_amd/utils/Uscheduler.py, following MOLE/utils/Uscheduler.py:259-343): the integer
logic runs on the host, so these tests need no GPU (the planner's C entry point is host code)."""
import pytest

from oracle import moe_oracle as O


def _plan(*a, **k):
    from mole_amd.utils.Uscheduler import plan_prefetch
    return plan_prefetch(*a, **k)


def test_local_counts_follow_time_over_fetch_time():
    # 3 layers, fetch time 2 ms: forward times 5, 1, 9 ms hide floor(2.5), floor(0.5), floor(4.5) fetches;
    # backward statistics come in backward order (last layer first)
    plan = _plan(4, [5e-3, 1e-3, 9e-3], [8e-3, 3e-3, 2e-3], 2e-3, [8, 8, 3])
    assert [p["local_fwd"] for p in plan] == [2, 0, min(4, 3, 4)]
    # layer i takes bwd_pf[n-1-i]: bwd_pf = [4, 1, 1] -> layer 0: 1, layer 1: 1, layer 2: min(4, 3 experts, pool 4)
    assert [p["local_bwd"] for p in plan] == [1, 1, 3]
    assert all(p["global_fwd"] == [] and p["global_bwd"] == [] for p in plan)
    # rounding up instead
    plan = _plan(4, [5e-3, 1e-3, 9e-3], [8e-3, 3e-3, 2e-3], 2e-3, [8, 8, 3], prefetch_floor=False)
    assert [p["local_fwd"] for p in plan] == [3, 1, 3]
    # the pool bounds every count
    plan = _plan(1, [5e-3, 1e-3, 9e-3], [8e-3, 3e-3, 2e-3], 2e-3, [8, 8, 3])
    assert [p["local_fwd"] for p in plan] == [1, 0, 1]


def test_forced_scheme_and_first_layer_switch():
    plan = _plan(8, [1.0, 1.0], [1.0, 1.0], 0.5, [4, 4], force=[[3, 1], [2, 4]], global_prefetch=True)
    assert [p["local_fwd"] for p in plan] == [3, 1]
    assert [p["local_bwd"] for p in plan] == [4, 2]             # backward counts are given in backward order
    assert all(p["global_fwd"] == [] for p in plan)             # a forced scheme switches cross-layer prefetch off
    plan = _plan(8, [1.0, 1.0], [1.0, 1.0], 0.5, [4, 4], deactivate_first_prefetch=True)
    assert [p["local_fwd"] for p in plan] == [0, 2]
    with pytest.raises(ValueError):
        _plan(8, [1.0], [1.0, 1.0], 0.5, [4, 4])
    with pytest.raises(ValueError):
        _plan(8, [1.0, 1.0], [1.0, 1.0], 0.0, [4, 4])


@pytest.mark.parametrize("pool,fwd,bwd,E", [(6, [3, 0, 5, 1], [2, 2, 0, 4], [4, 4, 4, 4]),
                                            (3, [9, 9, 9], [0, 1, 2], [2, 5, 1]),
                                            (10, [1, 7, 2, 2, 6], [5, 0, 0, 3, 3], [3, 3, 8, 2, 4])])
def test_cross_layer_plan_matches_the_oracle_planner(pool, fwd, bwd, E):
    """With cross-layer prefetch the counts come from fast_assign_prefetch, once on the forward budgets and once
    on the backward budgets over the layers in backward order; the oracle restates that function."""
    n = len(E)
    plan = _plan(pool, fwd, bwd, 1.0, E, global_prefetch=True)       # ftime 1: budgets = the given integers
    gp_f, lp_f = O.fast_assign_prefetch(pool, fwd, E)
    gp_b, lp_b = O.fast_assign_prefetch(pool, bwd, E[::-1])
    for i in range(n):
        assert plan[i]["local_fwd"] == lp_f[i]
        assert plan[i]["local_bwd"] == lp_b[n - 1 - i]
        assert plan[i]["global_fwd"] == sorted([list(x) for x in gp_f[i]], reverse=True)
        assert plan[i]["global_bwd"] == sorted([[n - 1 - x[0], x[1]] for x in gp_b[n - 1 - i]])
    # nothing is prefetched beyond what a layer owns
    for i in range(n):
        got = plan[i]["local_fwd"] + sum(c for p in plan for (layer, c) in p["global_fwd"] if layer == i)
        assert got <= E[i]
