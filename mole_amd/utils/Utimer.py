"""Per-layer forward / backward times of the MoE layers, for the prefetch planner.

The reference's UATimer (MOLE/utils/Utimer.py:73-110) stops the host around every measured span
(`torch.cuda.synchronize()` + `time.time()`).  Here a span is a pair of events on the compute stream, recorded by
MOLEModule.forward (and the backward of its autograd node) when it is called with time_it=True: the host never
waits inside a step, and stats() reads the events once, after the step.
"""
import torch


class UATimer:
    _fwd = {}    # moe_id -> [start event, end event]
    _bwd = {}

    @staticmethod
    def clear():
        UATimer._fwd, UATimer._bwd = {}, {}

    @staticmethod
    def _mark(store, moe_id, which):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        store.setdefault(moe_id, [None, None])[which] = ev

    @staticmethod
    def track_fwd_start(moe_id=0):
        UATimer._mark(UATimer._fwd, moe_id, 0)

    @staticmethod
    def track_fwd_end(moe_id=0):
        UATimer._mark(UATimer._fwd, moe_id, 1)

    @staticmethod
    def track_bwd_start(moe_id=0):
        UATimer._mark(UATimer._bwd, moe_id, 0)

    @staticmethod
    def track_bwd_end(moe_id=0):
        UATimer._mark(UATimer._bwd, moe_id, 1)

    @staticmethod
    def stats():
        """(fwd_stat, bwd_stat) in seconds: forward times in layer order, backward times in the order the
        backward pass visits the layers (the last layer first), as UATimer.stats() of the reference lists them."""
        torch.cuda.synchronize()

        def spans(store, reverse):
            out = []
            for i in sorted(store, reverse=reverse):
                a, b = store[i]
                if a is None or b is None:
                    raise RuntimeError(f"UATimer: layer {i} has an unfinished span (time_it must cover forward and backward)")
                out.append(a.elapsed_time(b) * 1e-3)
            return out
        return spans(UATimer._fwd, False), spans(UATimer._bwd, True)
