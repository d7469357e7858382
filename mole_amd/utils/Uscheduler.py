"""Prefetch planning for a stack of offloaded MoE layers: the part of the reference's UniScheduler that turns
measured times into per-layer prefetch counts (MOLE/utils/Uscheduler.py:228-349).

    plan_prefetch(...)                 pure integer logic: per-layer local / cross-layer ("global") counts
    UniScheduler.set_prefetch_scheme   applies a plan to the MOLEModule instances (Uscheduler.py:259-343)
    UniScheduler.measure_fetch_time    seconds to fetch one expert, from MOLEModule.dummy_fetch (Uscheduler.py:231-238)
    UniScheduler.prefetch_fwd          what a training loop calls before the first layer (Uscheduler.py:345-349)
    UniScheduler.schedule_policy / set_step / time_it / prefetch_it / profile_prefetch
                                       the profiling window (Uscheduler.py:56-63, 163-184, 228-258): during the first
                                       profile_step steps the layers run with time_it=True and record their forward
                                       and backward spans (utils/Utimer.py); profile_prefetch folds them and the
                                       measured fetch time into running means and plans the prefetch from them
    UniScheduler.save_states / load_states
                                       the checkpoint file (Uscheduler.py:67-92): torch.save([model_state,
                                       optim_state]) with one get_layer_state() dict per layer

The rest of the reference's scheduler (argument parsing, construction of the CPU optimizer) is not part of this
package; the optimizer state saved here is that of the in-pipeline Adam (the fp32 moments of the offloaded experts).
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch

from .. import core
from .Utimer import UATimer


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
    fwd_stat: Optional[List[float]] = None
    bwd_stat: Optional[List[float]] = None
    cur_step = -1
    profile_step = -1
    prefetch_on = False
    deactivate_first_prefetch = True
    prefetch_floor = False
    global_prefetch = False
    last_plan: Optional[List[dict]] = None

    @staticmethod
    def reset():
        """Forget policy, step counter and every measured time (a new run in the same process)."""
        UniScheduler.ftime = UniScheduler.fwd_stat = UniScheduler.bwd_stat = UniScheduler.last_plan = None
        UniScheduler.cur_step, UniScheduler.profile_step, UniScheduler.prefetch_on = -1, -1, False
        UniScheduler.deactivate_first_prefetch, UniScheduler.prefetch_floor, UniScheduler.global_prefetch = True, False, False
        UATimer.clear()

    # ---- the profiling window (Uscheduler.py:56-63, 163-184, 228-258) ------------------------------------
    @staticmethod
    def schedule_policy(profile_step, prefetch_on, deactivate_first_prefetch=True, prefetch_floor=False,
                        global_prefetch=False):
        UniScheduler.profile_step = profile_step
        UniScheduler.prefetch_on = prefetch_on
        UniScheduler.deactivate_first_prefetch = deactivate_first_prefetch
        UniScheduler.prefetch_floor = prefetch_floor
        UniScheduler.global_prefetch = global_prefetch

    @staticmethod
    def set_step(cur_step):
        """At the beginning of every step (Uscheduler.py:163-169): inside the profiling window the timers start
        afresh; the prefetch stack is emptied."""
        UniScheduler.cur_step = cur_step
        if UniScheduler.time_it():
            UATimer.clear()
        core.clear_virtual_mem()

    @staticmethod
    def time_it() -> bool:
        """Pass this as MOLEModule.forward(..., time_it=...): true during the profiling window (Uscheduler.py:171-177)."""
        return UniScheduler.cur_step < UniScheduler.profile_step

    @staticmethod
    def prefetch_it() -> bool:
        """Pass this as MOLEModule.forward(..., prefetch=...): true after the window when prefetch is on (Uscheduler.py:179-184)."""
        return UniScheduler.cur_step > UniScheduler.profile_step and UniScheduler.prefetch_on

    @staticmethod
    def profile_prefetch(force_prefetch_scheme=None):
        """At the end of a step inside the profiling window (Uscheduler.py:228-258): measure the time to fetch one
        expert, read the layers' forward and backward spans of this step, fold all three into running means
        (mean of the old value and the new one, as the reference does) and, with prefetch on, plan the prefetch
        from them.  The first two steps are skipped like the reference's (start-up costs would distort the means).
        Returns the plan, or None when nothing was planned."""
        if not UniScheduler.time_it() or UniScheduler.cur_step < 2:
            return None
        UniScheduler.measure_fetch_time(1)
        fwd, bwd = UATimer.stats()
        mean = lambda old, new: list(new) if old is None else [(a + b) / 2 for a, b in zip(old, new)]
        if fwd:
            UniScheduler.fwd_stat = mean(UniScheduler.fwd_stat, fwd)
        if bwd:
            UniScheduler.bwd_stat = mean(UniScheduler.bwd_stat, bwd)
        if not UniScheduler.prefetch_on or UniScheduler.fwd_stat is None or UniScheduler.bwd_stat is None:
            return None
        return UniScheduler.set_prefetch_scheme(UniScheduler.fwd_stat, UniScheduler.bwd_stat, None,
                                                UniScheduler.prefetch_floor, force_prefetch_scheme,
                                                UniScheduler.deactivate_first_prefetch, UniScheduler.global_prefetch)

    # ---- checkpoint files (Uscheduler.py:67-92) ----------------------------------------------------------
    @staticmethod
    def get_optim_state():
        """State of the in-pipeline Adam in the layout of the reference's MOLEMixedAdam.get_optim_state
        (MOLE/optim/mixed_optim.py:245-277): [expert_state, gate_state]; expert_state[4 l + p] = {"step",
        "exp_avg", "exp_avg_sq"} for parameter kind p of layer l (the order of the optimizer's parameter list,
        Uscheduler.py:104-112), the moments being the fp32 arrays of the layer's offloaded experts.  The gate is
        the caller's own optimizer's business here (gate_state None), and so are GPU-resident experts."""
        core.synchronize_tran()
        state = {}
        for l, m in enumerate(UniScheduler._layers()):
            if m.d_experts == 0 or not m.adv_adam:
                continue
            # set_adam hands over the counter before a step (the reference's optimizer does so every step), so after
            # that step the number of steps done is one more
            t = m.MOLECore.adam[2] + 1 if m.MOLECore.adam is not None else 0
            for p, c in enumerate(m.MOLECore.cpu):
                state[4 * l + p] = {"step": int(t), "exp_avg": c[2].clone(), "exp_avg_sq": c[3].clone()}
        return [state or None, None]

    @staticmethod
    def set_optim_state(states):
        core.synchronize_tran()
        expert_state = states[0] if states else None
        if not expert_state:
            return
        for l, m in enumerate(UniScheduler._layers()):
            if m.d_experts == 0 or not m.adv_adam:
                continue
            for p, c in enumerate(m.MOLECore.cpu):
                st = expert_state[4 * l + p]
                # the reference's state holds GPU-resident experts first: the offloaded ones are the last rows
                c[2].copy_(st["exp_avg"][-c[2].shape[0]:])
                c[3].copy_(st["exp_avg_sq"][-c[3].shape[0]:])
            if m.MOLECore.adam is not None:
                a = list(m.MOLECore.adam)
                a[2] = int(expert_state[4 * l]["step"])      # steps done = the counter before the next step
                m.MOLECore.adam = tuple(a)

    @staticmethod
    def save_states(state_file="MOLE_states", grad=False):
        """torch.save([model_state, optim_state], state_file + ".pt") (Uscheduler.py:67-75): model_state holds one
        MOLEModule.get_layer_state(grad) per layer, in layer order."""
        model_state = [m.get_layer_state(grad) for m in UniScheduler._layers()]
        torch.save([model_state, UniScheduler.get_optim_state()], state_file + ".pt")

    @staticmethod
    def load_states(state_file="MOLE_states", grad=False):
        """Inverse of save_states (Uscheduler.py:78-92).  The file is read with a loader that executes nothing
        from it (tensors, lists, dicts, numbers and None are all a state file holds)."""
        all_state = torch.load(state_file + ".pt", map_location="cpu", weights_only=True)
        model_state, optim_state = all_state[0], all_state[1]
        layers = UniScheduler._layers()
        if len(model_state) != len(layers):
            raise RuntimeError(f"load_states: the file holds {len(model_state)} layers, the model has {len(layers)}")
        for m, st in zip(layers, model_state):
            m.set_layer_state(st, grad)
        UniScheduler.set_optim_state(optim_state)
        return all_state

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
        UniScheduler.last_plan = plan
        return plan

    @staticmethod
    def prefetch_fwd():
        layers = UniScheduler._layers()
        if not layers:
            return
        if UniScheduler.profile_step >= 0 and not UniScheduler.prefetch_it():
            return            # a policy is set (schedule_policy) and this step does not prefetch (Uscheduler.py:345-349)
        if layers[0].global_prefetch:
            layers[0].global_prefetch_fwd()
        layers[0].local_prefetch_fwd()
