"""Prefetch planning for a stack of offloaded MoE layers: the part of the reference's UniScheduler that turns
measured times into per-layer prefetch counts (MOLE/utils/Uscheduler.py:228-349).

    plan_prefetch(...)                 pure integer logic: per-layer local / cross-layer ("global") counts
    UniScheduler.set_prefetch_scheme   applies a plan to the MOLEModule instances (Uscheduler.py:259-343)
    UniScheduler.measure_fetch_time    seconds to fetch one expert, from MOLEModule.dummy_fetch (Uscheduler.py:231-238)
    UniScheduler.prefetch_fwd          what a training loop calls before the first layer (Uscheduler.py:345-349)

The rest of the reference's scheduler (argument parsing, optimizer set-up, checkpoint files, the timers that
produce the per-layer statistics) is not part of this package: the caller passes the per-layer forward and
backward times it measured.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

from .. import core


def plan_prefetch(pool_size: int, fwd_stat: Sequence[float], bwd_stat: Sequence[float], ftime: float,
                  d_experts: Sequence[int], prefetch_floor: bool = True, force: Optional[Sequence[Sequence[int]]] = None,
                  deactivate_first_prefetch: bool = False, global_prefetch: bool = False) -> List[dict]:
    """Per-layer prefetch counts (Uscheduler.py:259-343).

    fwd_stat[i]: forward time of layer i; bwd_stat[j]: backward time of the j-th layer in backward order (the
    last layer first), as the reference's timers report them; ftime: time to fetch one expert.  A layer can hide
    floor (or ceil) of time / ftime expert fetches for the layer after it.  `force` = [fwd counts, bwd counts]
    overrides the measured budgets and switches cross-layer prefetch off, as the reference's
    force_prefetch_scheme does.  Returns, per layer, local_fwd / local_bwd (experts of the layer itself fetched
    just before it runs) and global_fwd / global_bwd (lists of [other_layer, count] fetched on its behalf)."""
    n = len(d_experts)
    if len(fwd_stat) != n or len(bwd_stat) != n:
        raise ValueError("plan_prefetch: one forward and one backward time per layer")
    if ftime <= 0:
        raise ValueError("plan_prefetch: the fetch time must be positive")
    rnd = math.floor if prefetch_floor else math.ceil
    fwd_pf = [int(rnd(f / ftime)) for f in fwd_stat]
    bwd_pf = [int(rnd(b / ftime)) for b in bwd_stat]
    if force is not None:
        global_prefetch = False
        fwd_pf, bwd_pf = [int(v) for v in force[0]], [int(v) for v in force[1]]
        if len(fwd_pf) != n or len(bwd_pf) != n:
            raise ValueError("plan_prefetch: a forced scheme needs one count per layer in both directions")
    if deactivate_first_prefetch and n:
        fwd_pf[0] = 0
    pool = max(0, int(pool_size))
    E = [int(e) for e in d_experts]
    plan = [dict(local_fwd=0, local_bwd=0, global_fwd=[], global_bwd=[]) for _ in range(n)]
    if not global_prefetch:
        for i in range(n):
            plan[i]["local_fwd"] = min(fwd_pf[i], E[i], pool)
            plan[i]["local_bwd"] = min(bwd_pf[n - 1 - i], E[i], pool)
        return plan
    gp_fwd, lp_fwd = core.fast_assign_prefetch(pool, fwd_pf, E)
    gp_bwd, lp_bwd = core.fast_assign_prefetch(pool, bwd_pf, E[::-1])
    for i in range(n):
        plan[i]["local_fwd"] = lp_fwd[i]
        plan[i]["local_bwd"] = lp_bwd[n - 1 - i]
        plan[i]["global_fwd"] = sorted(gp_fwd[i], reverse=True)
        plan[i]["global_bwd"] = sorted([[n - 1 - x[0], x[1]] for x in gp_bwd[n - 1 - i]])
    return plan


class UniScheduler:
    """The prefetch-related static methods of the reference's UniScheduler, over MOLEModule._instance."""
    ftime: Optional[float] = None

    @staticmethod
    def _layers():
        from ..moe.layer import MOLEModule
        return MOLEModule._instance

    @staticmethod
    def measure_fetch_time(batch_size: int = 1) -> float:
        """Average seconds per expert of an un-hidden fetch over all layers with offloaded experts, folded into a
        running mean like the reference's ftime (Uscheduler.py:231-238)."""
        times = [m.dummy_fetch(batch_size) / max(1, min(batch_size, m.d_experts))
                 for m in UniScheduler._layers() if m.d_experts > 0 and m.pool_size >= 1]
        if not times:
            raise RuntimeError("no layer with offloaded experts to measure")
        ftime = sum(times) / len(times)
        UniScheduler.ftime = ftime if UniScheduler.ftime is None else (UniScheduler.ftime + ftime) / 2
        return UniScheduler.ftime

    @staticmethod
    def set_prefetch_scheme(fwd_stat, bwd_stat, ftime=None, prefetch_floor=True, force=None,
                            deactivate_first_prefetch=False, global_prefetch=False) -> List[dict]:
        layers = UniScheduler._layers()
        ftime = UniScheduler.ftime if ftime is None else ftime
        if ftime is None:
            raise RuntimeError("set_prefetch_scheme: no fetch time (call measure_fetch_time or pass ftime)")
        pool = max(0, layers[0].pool_size) if layers else 0
        plan = plan_prefetch(pool, fwd_stat, bwd_stat, ftime, [m.d_experts for m in layers], prefetch_floor, force,
                             deactivate_first_prefetch, global_prefetch)
        use_global = global_prefetch and force is None
        for m, p in zip(layers, plan):
            m.set_prefetch(p["local_fwd"], p["local_bwd"])
            m.global_prefetch = use_global
            m.global_prefetch_fwd_count = p["global_fwd"]
            m.global_prefetch_bwd_count = p["global_bwd"]
        return plan

    @staticmethod
    def prefetch_fwd():
        layers = UniScheduler._layers()
        if not layers:
            return
        if layers[0].global_prefetch:
            layers[0].global_prefetch_fwd()
        layers[0].local_prefetch_fwd()
