"""Host side of the expert pipeline: the module the reference reaches as `UniMoE.core` (pybind,
MOLE/cpp/core.cpp:1347-1469), re-hosted in Python over the C ABI of libmole_hip.so.

What is mirrored (same names, same argument meaning):
  create_UniMem / clear_virtual_mem / view_pool_size / fetch_top_prefetched_batch /
  synchronize_tran / default_wait_tran / fast_assign_prefetch       core.cpp:1397-1432
  MOLECore(...).forward / .backward / .prefetch_fwd / .prefetch_bwd / .dummy_fetch /
  .set_GPUParamCore / .set_CPUParamCore                               core.cpp:1356-1388
  BatchFusedFWD  - the autograd.Function MOLE/moe/layer.py:453 calls but the reference snapshot
                   never defines; it forwards to MOLECore.forward / MOLECore.backward
                   (define.hpp:594-606).

The expert math itself (two grouped GEMMs forward, four backward, bias/GELU/GELU' epilogues) is
mole_ffn_fwd / mole_ffn_bwd; this file only decides which experts run from which memory:
GPU-resident ("static") experts in one grouped launch, offloaded ("dynamic") experts in chunks that
fit the free part of the slot pool (core.cpp:1020-1051), each chunk fetched on the copy stream and
handed to the compute stream through events (core.cpp:110-143, 212-249).
"""
from __future__ import annotations

import ctypes
import itertools
from ctypes import c_float, c_int, c_uint64, c_void_p
from typing import List, Optional

import torch

from . import _lib as L
from . import hip_ops as H

_DTYPES = {"torch.float32": torch.float32, "torch.bfloat16": torch.bfloat16}


# ---------------------------------------------------------------------------------------------
# slot pool (process-global, first caller wins: umemory.cpp:77-86)
# ---------------------------------------------------------------------------------------------
class UniMem:
    def __init__(self, device: int, pool_size: int, dtype: torch.dtype, F: int, M: int):
        self.device, self.pool_size, self.dtype, self.F, self.M = device, pool_size, dtype, F, M
        self._h = c_void_p()
        L.check(L.lib().mole_unimem_create(device, max(pool_size, 0), L.dtype_code(dtype), F, M, ctypes.byref(self._h)),
                "mole_unimem_create")

    def close(self):
        if self._h:
            L.check(L.lib().mole_unimem_destroy(self._h), "mole_unimem_destroy")
            self._h = c_void_p()

    def _int(self, fn) -> int:
        out = c_int()
        L.check(fn(self._h, ctypes.byref(out)), fn.__name__)
        return out.value

    def view_pool_size(self) -> int:
        return self._int(L.lib().mole_unimem_view_pool_size)

    def virtual_offset(self) -> int:
        return self._int(L.lib().mole_unimem_virtual_offset)

    def clear_virtual_mem(self):
        L.check(L.lib().mole_unimem_clear_virtual_mem(self._h), "mole_unimem_clear_virtual_mem")

    @staticmethod
    def _src(host_tensors):
        arr = (c_void_p * 4)()
        for i, t in enumerate(host_tensors):
            arr[i] = t.data_ptr()
        return arr

    def prefetch(self, layer: int, host_tensors, base: int, n: int):
        L.check(L.lib().mole_unimem_prefetch(self._h, layer, self._src(host_tensors), base, n), "mole_unimem_prefetch")

    def fetch_top(self, layer: int) -> int:
        out = c_int()
        L.check(L.lib().mole_unimem_fetch_top(self._h, layer, ctypes.byref(out)), "mole_unimem_fetch_top")
        return out.value

    def fetch(self, host_tensors, view_base: int, base: int, n: int, prefetched: int) -> List[int]:
        ptrs = (c_void_p * 4)()
        L.check(L.lib().mole_unimem_fetch(self._h, self._src(host_tensors), view_base, base, n, prefetched, ptrs),
                "mole_unimem_fetch")
        return [int(p) for p in ptrs]

    @staticmethod
    def _ids(ids):
        return (ctypes.c_int32 * max(len(ids), 1))(*[int(e) for e in ids])

    def prefetch_ids(self, layer: int, host_tensors, ids, tag: int = 0):
        """prefetch() for an explicit list of experts: ids[i] lands in the i-th reserved slot.  tag != 0: slots
        that were filled under the same tag from the same host expert keep what they hold."""
        L.check(L.lib().mole_unimem_prefetch_ids(self._h, layer, self._src(host_tensors), self._ids(ids), len(ids), tag),
                "mole_unimem_prefetch_ids")

    def fetch_ids(self, host_tensors, view_base: int, ids, prefetched: int, tag: int = 0) -> List[int]:
        """fetch() for an explicit list of experts (the first `prefetched` of them are already in their slots)."""
        ptrs = (c_void_p * 4)()
        L.check(L.lib().mole_unimem_fetch_ids(self._h, self._src(host_tensors), view_base, self._ids(ids), len(ids),
                                              prefetched, tag, ptrs), "mole_unimem_fetch_ids")
        return [int(p) for p in ptrs]

    def reuse_stats(self) -> int:
        """Bytes that were not copied because their slot still held the expert (since the last read)."""
        b = c_uint64()
        L.check(L.lib().mole_unimem_reuse_stats(self._h, ctypes.byref(b)), "mole_unimem_reuse_stats")
        return b.value

    def wait_params(self):
        L.check(L.lib().mole_unimem_wait_params(self._h, L.stream()), "mole_unimem_wait_params")

    def wait_slots(self, view_base: int, n: int):
        """The current stream waits for the experts in slots view_base.. (of the visible pool) to have arrived."""
        L.check(L.lib().mole_unimem_wait_slots(self._h, view_base, n, L.stream()), "mole_unimem_wait_slots")

    def release(self, view_base: int, n: int):
        L.check(L.lib().mole_unimem_release(self._h, view_base, n, L.stream()), "mole_unimem_release")

    def sync_tran(self):
        L.check(L.lib().mole_unimem_sync_tran(self._h), "mole_unimem_sync_tran")
        L.check(L.lib().mole_unimem_sync_tranback(self._h), "mole_unimem_sync_tranback")

    def store_grads(self, host_grads, dev_grads, base: int, n: int):
        """Device gradients of n experts -> experts [base, base+n) of the pinned host gradient arrays, on the
        pool's write-back stream, after the compute already enqueued on the current stream."""
        L.check(L.lib().mole_unimem_store_grads(self._h, self._src(host_grads), self._src(dev_grads), base, n, L.stream()),
                "mole_unimem_store_grads")
        out = c_void_p()
        L.check(L.lib().mole_unimem_tranback_stream(self._h, ctypes.byref(out)), "mole_unimem_tranback_stream")
        wb = torch.cuda.ExternalStream(int(out.value), device=dev_grads[0].device)
        for g in dev_grads:           # the allocator must not hand these blocks out again before the copy has run
            g.record_stream(wb)

    def store_grads_ids(self, host_grads, dev_grads, ids):
        """store_grads() with the i-th expert of dev_grads going to host expert ids[i]."""
        L.check(L.lib().mole_unimem_store_grads_ids(self._h, self._src(host_grads), self._src(dev_grads), self._ids(ids),
                                                    len(ids), L.stream()), "mole_unimem_store_grads_ids")
        wb = self._side_stream("mole_unimem_tranback_stream", dev_grads[0].device)
        for g in dev_grads:
            g.record_stream(wb)

    def zero_grads_ids(self, host_grads, ids):
        """Zeros to the listed experts of the pinned host gradient arrays, on the write-back stream."""
        if ids:
            L.check(L.lib().mole_unimem_zero_grads_ids(self._h, self._src(host_grads), self._ids(ids), len(ids)),
                    "mole_unimem_zero_grads_ids")

    @staticmethod
    def _arrays(tensors):
        n = len(tensors)
        ptrs, sizes = (c_void_p * n)(), (ctypes.c_size_t * n)()
        for i, t in enumerate(tensors):
            ptrs[i], sizes[i] = t.data_ptr(), t.numel() * t.element_size()
        return ptrs, sizes

    def _side_stream(self, getter: str, device) -> torch.cuda.Stream:
        out = c_void_p()
        L.check(getattr(L.lib(), getter)(self._h, ctypes.byref(out)), getter)
        return torch.cuda.ExternalStream(int(out.value), device=device)

    def load_state(self, dev_tensors, host_tensors, after_writeback: bool = False):
        """Pinned host arrays -> device tensors of the same sizes on the copy stream (after the compute already
        enqueued on the current stream, which then waits for the copies): optimizer moments and accumulated
        gradients of an expert batch (core.cpp:864-915).  after_writeback: the host arrays may still be the target
        of a write-back in flight (gradients of the previous micro-step), so the copies wait for that stream too."""
        dp, sizes = self._arrays(dev_tensors)
        hp, hs = self._arrays(host_tensors)
        if list(sizes) != list(hs):
            raise RuntimeError("UniMem.load_state: host and device sizes differ")
        L.check(L.lib().mole_unimem_load_state(self._h, dp, hp, sizes, len(dev_tensors), int(after_writeback), L.stream()),
                "mole_unimem_load_state")
        tran = self._side_stream("mole_unimem_tran_stream", dev_tensors[0].device)
        for t in dev_tensors:
            t.record_stream(tran)

    def store_state(self, host_tensors, dev_tensors):
        """Device tensors -> pinned host arrays on the write-back stream, after the compute already enqueued on
        the current stream (core.cpp:925-935)."""
        hp, hs = self._arrays(host_tensors)
        dp, sizes = self._arrays(dev_tensors)
        if list(sizes) != list(hs):
            raise RuntimeError("UniMem.store_state: host and device sizes differ")
        L.check(L.lib().mole_unimem_store_state(self._h, hp, dp, sizes, len(dev_tensors), L.stream()),
                "mole_unimem_store_state")
        wb = self._side_stream("mole_unimem_tranback_stream", dev_tensors[0].device)
        for t in dev_tensors:
            t.record_stream(wb)

    def writeback_stats(self):
        b, ms = c_uint64(), c_float()
        L.check(L.lib().mole_unimem_writeback_stats(self._h, ctypes.byref(b), ctypes.byref(ms)),
                "mole_unimem_writeback_stats")
        return b.value, ms.value

    def tran_stream_handle(self) -> int:
        out = c_void_p()
        L.check(L.lib().mole_unimem_tran_stream(self._h, ctypes.byref(out)), "mole_unimem_tran_stream")
        return int(out.value or 0)

    def tranback_stream_handle(self) -> int:
        out = c_void_p()
        L.check(L.lib().mole_unimem_tranback_stream(self._h, ctypes.byref(out)), "mole_unimem_tranback_stream")
        return int(out.value or 0)

    def copy_stats(self):
        b, ms = c_uint64(), c_float()
        L.check(L.lib().mole_unimem_copy_stats(self._h, ctypes.byref(b), ctypes.byref(ms)), "mole_unimem_copy_stats")
        return b.value, ms.value

    def slot_tensor(self, p_id: int, slot: int, n: int) -> int:
        """Device address of `slot` for parameter kind p_id (debug / tests)."""
        out = c_void_p()
        L.check(L.lib().mole_unimem_slot_ptr(self._h, p_id, slot, ctypes.byref(out)), "mole_unimem_slot_ptr")
        return int(out.value)


_UniMemInst: List[UniMem] = []


def create_UniMem(device, pool_size, dtype, sizes) -> UniMem:
    """create_UniMem(local_rank, pool_size, "torch.float32", [[F,M],[F],[F,M],[M]]) - layer.py:43-47.
    The pool is process-global and the first caller sizes it (umemory.cpp:77-86); a later caller whose experts
    have another shape or dtype, or who asks for more slots, would read and write the slots at the wrong strides,
    so that is refused here (the reference does not check)."""
    dt = _DTYPES[dtype] if isinstance(dtype, str) else dtype
    F, M = int(sizes[0][0]), int(sizes[0][1])
    if _UniMemInst:
        um = _UniMemInst[0]
        if int(pool_size) > 0 and (um.dtype, um.F, um.M) != (dt, F, M):
            raise RuntimeError(f"create_UniMem: the slot pool holds {um.dtype} experts of F={um.F}, M={um.M}; "
                               f"a layer with {dt}, F={F}, M={M} cannot share it")
        if int(pool_size) > um.pool_size:
            raise RuntimeError(f"create_UniMem: the slot pool has {um.pool_size} slots, {pool_size} were asked for")
        return um
    um = UniMem(int(device), int(pool_size), dt, F, M)
    _UniMemInst.append(um)
    return um


def get_UniMem() -> Optional[UniMem]:
    return _UniMemInst[0] if _UniMemInst else None


def destroy_UniMem():
    while _UniMemInst:
        _UniMemInst.pop().close()


def clear_virtual_mem():
    _UniMemInst[0].clear_virtual_mem()


def view_pool_size() -> int:
    return _UniMemInst[0].view_pool_size()


def fetch_top_prefetched_batch(moe_id: int) -> int:
    return _UniMemInst[0].fetch_top(moe_id)


def synchronize_tran():
    if _UniMemInst:
        _UniMemInst[0].sync_tran()


def default_wait_tran():
    if _UniMemInst:
        _UniMemInst[0].wait_params()


_multi_stream = [True]


def disable_multi_stream():
    """core.cpp:1402 / stream.cpp:84-95: every role runs on the compute stream.  Here: the copies still run on the
    pool's streams (the ordering events make that invisible to results), but ExpertStreamCtx hands out the compute
    stream for every role."""
    _multi_stream[0] = False


def multi_stream_enabled() -> bool:
    return _multi_stream[0]


def get_stream_cdata(device: int, idx: int) -> int:
    """Raw handle of the stream with the reference's role index (stream.hpp:30-66: tran = 1, comp = 2, comm = 3,
    tranback = 4; core.cpp:1401).  comp and comm are torch's current stream (one GPU: no exchange stream)."""
    um = get_UniMem()
    if idx == 1 and um is not None and _multi_stream[0]:
        return um.tran_stream_handle()
    if idx == 4 and um is not None and _multi_stream[0]:
        return um.tranback_stream_handle()
    return int(torch.cuda.current_stream(device).cuda_stream)


def default_wait_comp():
    """core.cpp:1403: the default stream waits for the compute stream - the same stream here, nothing to do."""
    return None


def default_wait_comm():
    """core.cpp:1404: likewise for the exchange stream, which one GPU does not have."""
    return None


class _DeviceSpan:
    """A stretch of device memory as an object torch.as_tensor() can wrap without copying."""

    def __init__(self, ptr: int, nbytes: int):
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (ptr, False), "version": 2}


def pool_prefetch(moe_id: int, batch_size: int):
    """core.cpp:1425 -> _UniMem::prefetch (umemory.cpp:131-154): reserve `batch_size` slots for layer `moe_id` on
    the prefetch stack and return the four slot tensors [batch_size, F, M], [batch_size, F], [batch_size, F, M],
    [batch_size, M] for the caller to fill (MOLECore.prefetch_fwd does reserve + copy in one call)."""
    um = get_UniMem()
    if batch_size == 0 or um is None:
        return []
    ptrs = (c_void_p * 4)()
    L.check(L.lib().mole_unimem_reserve(um._h, int(moe_id), int(batch_size), ptrs), "mole_unimem_reserve")
    es = torch.empty(0, dtype=um.dtype).element_size()
    shapes = [(batch_size, um.F, um.M), (batch_size, um.F), (batch_size, um.F, um.M), (batch_size, um.M)]
    out = []
    for ptr, shape in zip(ptrs, shapes):
        n = 1
        for d in shape:
            n *= d
        raw = torch.as_tensor(_DeviceSpan(int(ptr), n * es), device=torch.device("cuda", um.device))
        out.append(raw.view(um.dtype).view(shape))
    return out


def fast_assign_prefetch(P: int, Fv, Ev):
    """(GPscheme, LPscheme) as core.cpp:1302-1345: GPscheme[i] = [[later_layer, count], ...]."""
    n = len(Ev)
    IntN = c_int * max(n, 1)
    lp = IntN()
    cap = 4 * n + 4
    gp = (c_int * (3 * cap))()
    gpn = c_int()
    L.check(L.lib().mole_fast_assign_prefetch(int(P), IntN(*[int(v) for v in Fv]), IntN(*[int(v) for v in Ev]), n, lp, gp,
                                              cap, ctypes.byref(gpn)), "mole_fast_assign_prefetch")
    scheme = [[] for _ in range(n)]
    for i in range(gpn.value):
        scheme[gp[3 * i]].append([gp[3 * i + 1], gp[3 * i + 2]])
    return scheme, [lp[i] for i in range(n)]


# ---------------------------------------------------------------------------------------------
# per-layer core
# ---------------------------------------------------------------------------------------------
def plan_chunks(n_total: int, prefetched: int, view_pool_size: int, ebatch_size: int):
    """Chunks of the offloaded experts of one layer, in processing order -> [(first, size, already_prefetched,
    view_base)] (core.cpp:1020-1051).  The first `prefetched` experts already sit in slots 0.. of the visible
    pool, so a chunk that still holds some of them must start at slot == index: where the reference wraps
    view_base to 0 regardless (core.cpp:1026-1046) - which would run such a chunk on whatever slot 0 holds - the
    chunk is cut at the end of the visible pool instead, and the wrap happens once the prefetched experts are done."""
    if n_total == 0:
        return []
    vps = int(view_pool_size)
    if vps <= 0:
        raise RuntimeError("slot pool exhausted by prefetches: no slot left to run offloaded experts")
    if prefetched > vps:
        raise RuntimeError(f"{prefetched} prefetched experts cannot sit in a visible pool of {vps} slots")
    d_batch = min(max(int(ebatch_size), 1), vps)
    out, view_base, i = [], 0, 0
    while i < n_total:
        size = min(d_batch, n_total - i)
        if vps - view_base < size:
            if i < prefetched:
                size = vps - view_base
            else:
                view_base = 0
        out.append((i, size, max(0, min(size, prefetched - i)), view_base))
        view_base += size
        i += size
    return out


# Tags under which forward passes fill pool slots come from one counter for the whole process: a tag is never handed
# out twice while the pool lives, whatever layers are destroyed and rebuilt around it (a rebuilt layer can get the same
# pinned host addresses back from the allocator, and a repeated tag would then match a stale slot).
_PASS_TAGS = itertools.count(1)


class MOLECore:
    """Per-layer state and the expert-batch pipeline (define.hpp:338-607, core.cpp:991-1300).

    activated_only (default): offloaded experts that routing gave no row (kept_rows[e] == 0) are neither copied to
    the pool nor launched; their host gradient is zero.  The layer reads its E kept-row counts back once per
    forward (one small device-to-host copy, the only host synchronisation of the path), packs the activated
    experts into pool slots in processing order and hands the grouped FFN a compacted offsets / kept_rows pair.
    prefetch_bwd prefetches only experts the forward pass activated; prefetch_fwd, which runs before the layer's
    routing exists, prefetches the experts the previous step activated (none before the first step) - a wrong
    guess costs a copy, never a result.  The reference copies and runs every expert of every chunk in index
    order (core.cpp:41-57, 1025-1047); activated_only=False does the same.

    resident (default): what a layer's forward pass brought into the pool is not fetched again for its backward
    pass while it is still there.  Every forward pass copies under a tag of its own and the backward pass asks
    for its experts under the same tag; the pool skips a slot that still holds that expert under that tag.  When
    the pool has a slot for every offloaded expert of every layer (an MI355X holds 288 GB), each layer keeps a
    fixed stretch of slots, expert e at its base + e, nothing is ever displaced between a forward and its
    backward, and the host-to-device traffic of a step halves; with a smaller pool the slots are recycled
    through the prefetch stack as in the reference (umemory.cpp:131-183) and only what happens to survive (the last
    layer's experts, whose backward follows its forward directly) is reused.  The reference fetches the weights
    again for every backward (core.cpp:1203)."""

    def __init__(self, use_pool, mome_use_pool, vari_use_pool, grad_use_pool, s_experts, d_experts, ebatch_size,
                 world_size, act_name, adv_adam, acc_step, step, device, moe_id, total_experts,
                 gelu_bwd: str = "tanh", activated_only: bool = True, resident: bool = True):
        if world_size != 1:
            raise NotImplementedError("this build covers the single-GPU hot path (world_size == 1)")
        if act_name != "gelu":
            raise NotImplementedError("only act='gelu' is on the hot path")
        self.adv_adam = bool(adv_adam)
        self.adam = None            # set_adam(): (beta1, beta2, t, lr, lam, eps, adamW)
        self.hybrid_adam_count = d_experts
        self.use_pool, self.acc_step, self.step = bool(use_pool), int(acc_step), int(step)
        self.device, self.moe_id, self.total_experts = device, moe_id, total_experts
        self.s_experts, self.d_experts, self.ebatch_size = s_experts, d_experts, max(int(ebatch_size), 1)
        self.world_size, self.act_name = world_size, act_name
        self.gelu_bwd = L.GELU_BWD_TANH if gelu_bwd == "tanh" else L.GELU_BWD_EXACT
        self.gpu = [None] * 4       # (all_tensors, grad_tensors)
        self.cpu = [None] * 4       # (all_tensors, grad_)
        self._saved = None
        self.activated_only = bool(activated_only)
        self._pref = {"fwd": [], "bwd": []}   # experts prefetched so far for the next pass, in slot order
        self._active = None                   # offloaded experts the last forward gave rows to (None: not known)
        self._grad_is_zero = [False] * d_experts   # the expert's pinned host gradient is known to hold zeros
        self.lazy_zero = True
        self.resident = bool(resident)
        self._passes = 0            # forward passes so far: part of the tag under which a pass fills pool slots
        self._tag = 0               # tag of the pass in preparation or in flight (0: none yet)
        self._tag_used = True       # a forward pass has run under _tag: the next prefetch_fwd / forward takes a new one
        # Where a pass keeps its experts - a fixed stretch of slots (first slot) or the prefetch stack (None) - is
        # decided once per pass, by the first prefetch for it or by the forward itself, and carried to its backward.
        self._home_fwd = None       # decision for the coming forward pass (valid while experts are prefetched for it)
        self._home_pass = None      # decision of the last forward pass: its backward and the prefetches for it use it

    # the reference's counters of experts prefetched so far (define.hpp:352-353)
    @property
    def fwd_base(self) -> int:
        return len(self._pref["fwd"])

    @property
    def bwd_base(self) -> int:
        return len(self._pref["bwd"])

    # parameter stores -------------------------------------------------------------------------
    def set_GPUParamCore(self, p_id, all_tensors, grad_tensors, bias):
        self.gpu[p_id] = (all_tensors, grad_tensors)

    def set_CPUParamCore(self, p_id, all_tensors, grad_, momentum, variance, bias, p_id2=None):
        self.cpu[p_id] = (all_tensors, grad_, momentum, variance)

    def set_adam(self, beta1, beta2, t, lr, lam, eps, adamW, hybrid_adam_count=-1):
        """Hyper-parameters of the in-pipeline Adam (define.hpp:524-541); t is the optimizer's step counter
        before this step, hybrid_adam_count the number of leading offloaded experts updated on the GPU (-1: all)."""
        self.adam = (float(beta1), float(beta2), int(t), float(lr), float(lam), float(eps), bool(adamW))
        self.hybrid_adam_count = self.d_experts if hybrid_adam_count == -1 else int(hybrid_adam_count)

    def set_hybrid_adam_count(self, hybrid_adam_count):
        self.hybrid_adam_count = self.d_experts if hybrid_adam_count == -1 else int(hybrid_adam_count)

    def set_lazy_zero(self):
        """The host gradient arrays are to be taken as zero: the next write-back overwrites them
        (uparameter.cpp:68-83, core.cpp:1392)."""
        for c in self.cpu:
            if c is not None and c[1] is not None:
                c[1].lazy_zero = True

    def unset_lazy_zero(self):
        for c in self.cpu:
            if c is not None and c[1] is not None:
                c[1].lazy_zero = False

    def host_gradients_changed(self):
        """Call after writing the pinned host gradient arrays from outside the pipeline (loading a checkpoint):
        experts that get no rows in the next step are then zeroed again instead of being taken as already zero."""
        self._grad_is_zero = [False] * self.d_experts

    def _host(self):
        return [c[0] for c in self.cpu]

    # prefetch -----------------------------------------------------------------------------------
    def _forward_tag(self) -> int:
        """The tag of the coming (or running) forward pass: a new one unless a prefetch already took it."""
        if not self.resident:
            return 0
        if self._tag_used:
            self._passes += 1
            self._tag = next(_PASS_TAGS)
            self._tag_used = False
        return self._tag

    def _home_base(self):
        """First slot of this layer's fixed stretch of the pool, or None when the pool cannot give every offloaded
        expert of every layer a slot of its own (then the slots are recycled through the prefetch stack)."""
        if not self.resident or self.d_experts == 0 or not self.use_pool:
            return None
        um = get_UniMem()
        from .moe.layer import MOLEModule
        layers = [m.MOLECore for m in MOLEModule._instance]
        if um is None or self not in layers or not all(c.resident for c in layers):
            return None
        if sum(c.d_experts for c in layers) > um.pool_size or um.virtual_offset() != 0:
            return None
        return sum(c.d_experts for c in layers[:layers.index(self)])

    def _home_for(self, which: str):
        """The slot placement of the pass `which` is being prepared for: decided when nothing has been prefetched for
        the coming forward pass yet, then kept until its backward pass is done."""
        if which == "fwd":
            if not self._pref["fwd"]:
                self._home_fwd = self._home_base()
            return self._home_fwd
        return self._home_pass

    def _home_fetch(self, home: int, ids, tag: int):
        """Bring the experts `ids` into their own slots (home + e); runs of consecutive experts in one call."""
        um = get_UniMem()
        for (at, e0, n) in self._runs(list(ids)):
            um.fetch_ids(self._host(), home + e0, ids[at:at + n], 0, tag)

    def _prefetch(self, which: str, batch_size: int):
        if batch_size <= 0 or self.d_experts == 0:
            return
        done = self._pref[which]
        tag = self._forward_tag() if which == "fwd" else self._tag
        if not self.activated_only:
            todo = list(range(len(done), min(self.d_experts, len(done) + batch_size)))
        else:
            known = self._active if self._active is not None else []
            seen = set(done)
            todo = [e for e in known if e not in seen][:batch_size]
        if not todo:
            return
        home = self._home_for(which)
        if home is not None:
            self._home_fetch(home, todo, tag)
        elif not self.activated_only:
            get_UniMem().prefetch(self.moe_id, self._host(), todo[0], len(todo))
        else:
            get_UniMem().prefetch_ids(self.moe_id, self._host(), todo, tag)
        done.extend(todo)

    def prefetch_fwd(self, batch_size: int):
        self._prefetch("fwd", batch_size)

    def prefetch_bwd(self, batch_size: int):
        self._prefetch("bwd", batch_size)

    def dummy_fetch(self, batch_size: int):
        """Copy `batch_size` experts into slots 0.. without reserving them (core.cpp:25-39)."""
        if batch_size == 0:
            return
        um = get_UniMem()
        um.fetch(self._host(), -um.virtual_offset(), 0, batch_size, 0)

    # pipeline -----------------------------------------------------------------------------------
    def _take_prefetched(self, which: str, home):
        """The experts prefetched for this pass, in slot order; pops this layer's entry of the prefetch stack
        (experts with slots of their own never enter the stack)."""
        um = get_UniMem()
        if not self.use_pool or um is None or um.pool_size <= 0:
            raise RuntimeError("offloaded experts need the slot pool (pool_size >= 1, use_pool=True)")
        ids, self._pref[which] = self._pref[which], []
        if home is not None:
            return ids
        n = um.fetch_top(self.moe_id)
        if n != len(ids):
            raise RuntimeError(f"prefetch stack out of order: top holds {n}, layer expects {len(ids)}")
        return ids

    def _chunks(self, n_total: int, prefetched: int):
        um = get_UniMem()
        return plan_chunks(n_total, prefetched, um.view_pool_size(), self.ebatch_size)

    def _order(self, resident, wanted, offsets, kept_rows, host_meta):
        """Processing order of the offloaded experts - the resident (prefetched) ones in slot order, then the
        wanted ones not among them - and the matching offsets / kept_rows arrays on the device."""
        d, e0 = self.d_experts, self.s_experts
        inres = set(resident)
        order = list(resident) + [e for e in wanted if e not in inres]
        if order == list(range(d)):
            return order, offsets[e0:], kept_rows[e0:]
        if host_meta is None:     # no host copy of the counts: gather on the device
            sel = torch.tensor(order, dtype=torch.int64).to(offsets.device)
            return order, offsets[e0:e0 + d][sel].contiguous(), kept_rows[e0:e0 + d][sel].contiguous()
        off_h, kept_h = host_meta
        comp = torch.tensor([[off_h[e] for e in order], [kept_h[e] for e in order]], dtype=torch.int32)
        comp = comp.to(offsets.device)
        return order, comp[0], comp[1]

    def _home_chunks(self, home: int, wanted):
        """Expert ranges [e0, e0 + size) of at most ebatch_size experts that hold a wanted expert, with the device
        addresses of their slots."""
        um = get_UniMem()
        want = set(wanted)
        for e0 in range(0, self.d_experts, self.ebatch_size):
            size = min(self.ebatch_size, self.d_experts - e0)
            ids = [e for e in range(e0, e0 + size) if e in want]
            if ids:
                yield e0, size, ids, [um.slot_tensor(p, home + e0, size) for p in range(4)]

    def forward(self, dispatched_input: torch.Tensor, requires_grad: bool, offsets=None, kept_rows=None,
                return_saved: bool = False):
        """dispatched_input: [E, C, M] (reference layout; every row is computed, like the reference)
        or, with offsets/kept_rows from mole_route, any [rows, M] expert-contiguous buffer of which
        only the kept rows are computed.  Returns a tensor of the same shape."""
        x = dispatched_input
        shape = x.shape
        M = shape[-1]
        E = self.s_experts + self.d_experts
        routed = offsets is not None
        if not routed:
            assert x.dim() == 3 and shape[0] == E, f"expected [E={E}, C, M], got {tuple(shape)}"
            C = shape[1]
            offsets = torch.arange(E + 1, dtype=torch.int32, device=x.device) * C
            kept_rows = torch.full((E,), C, dtype=torch.int32, device=x.device)
        x2 = x.reshape(-1, M)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        rows = x2.shape[0]
        F = (self.gpu[0][0] if self.s_experts else self.cpu[0][0]).shape[1]
        h = torch.empty(rows, F, dtype=x.dtype, device=x.device)
        a = torch.empty(rows, F, dtype=x.dtype, device=x.device)
        out = torch.empty(rows, M, dtype=x.dtype, device=x.device)
        if self.s_experts:
            w1, b1, w2, b2 = (g[0] for g in self.gpu)
            H.ffn_fwd_into(x2, offsets, kept_rows, self.s_experts, rows, M, F, w1, b1, w2, b2, h, a, out)
        host_meta, tag = None, 0
        if self.d_experts:
            um = get_UniMem()
            home = self._home_for("fwd")
            self._home_pass = home
            resident = self._take_prefetched("fwd", home)
            tag = self._forward_tag()
            self._tag_used = True
            d, e0 = self.d_experts, self.s_experts
            if self.activated_only and routed:
                # the one host synchronisation of the path: E row counts (and row offsets) come back
                meta = torch.stack([offsets[e0:e0 + d], kept_rows[e0:e0 + d]]).cpu()
                host_meta = (meta[0].tolist(), meta[1].tolist())
                self._active = [e for e in range(d) if host_meta[1][e] > 0]
                wanted = self._active
            else:
                self._active = list(range(d))       # every expert runs
                wanted = range(d)
            if home is not None:
                # every expert has a slot of its own: the copies of all wanted experts are issued now, each chunk
                # waits for its own, and experts without rows are simply not copied (the kernel skips them)
                self._home_fetch(home, list(wanted), tag)
                for (c0, size, _, p) in self._home_chunks(home, wanted):
                    um.wait_slots(home + c0, size)
                    H.ffn_fwd_into(x2, offsets[e0 + c0:], kept_rows[e0 + c0:], size, rows, M, F, p[0], p[1], p[2], p[3], h, a, out)
                    um.release(home + c0, size)
            else:
                order, off_c, kept_c = self._order(resident, wanted, offsets, kept_rows, host_meta)
                for (lo, size, pref, view_base) in self._chunks(len(order), len(resident)):
                    p = um.fetch_ids(self._host(), view_base, order[lo:lo + size], pref, tag)
                    um.wait_slots(view_base, size)
                    H.ffn_fwd_into(x2, off_c[lo:], kept_c[lo:], size, rows, M, F, p[0], p[1], p[2], p[3], h, a, out)
                    um.release(view_base, size)
        saved = (x2, h, a, offsets, kept_rows, requires_grad, shape, host_meta, tag, self._home_pass)
        if return_saved:          # the caller (an autograd node) keeps the activations itself
            return out.view(shape), saved
        self._saved = saved       # reference behaviour: the core holds them until backward (define.hpp:594-606)
        return out.view(shape)

    def backward(self, all_output_grad: torch.Tensor, saved=None):
        if saved is None:
            saved, self._saved = self._saved, None
        if saved is None:
            raise RuntimeError("MOLECore.backward without a preceding forward")
        x2, h, a, offsets, kept_rows, need_gx, shape, host_meta, tag, home = saved
        M = shape[-1]
        go = all_output_grad.reshape(-1, M)
        if not go.is_contiguous():
            go = go.contiguous()
        rows = x2.shape[0]
        F = h.shape[1]
        t = torch.empty(rows, F, dtype=x2.dtype, device=x2.device)
        gx = torch.empty(rows, M, dtype=x2.dtype, device=x2.device) if need_gx else None
        acc = self.acc_step > 1
        if self.s_experts:
            w1, _, w2, _ = (g[0] for g in self.gpu)
            gw1, gb1, gw2, gb2 = (g[1] for g in self.gpu)
            H.ffn_bwd_into(go, x2, h, a, offsets, kept_rows, self.s_experts, rows, M, F, w1, w2, t, gw1, gb1, gw2, gb2,
                           gx, acc, self.gelu_bwd)
        if self.d_experts:
            um = get_UniMem()
            resident = self._take_prefetched("bwd", home)
            d, e0 = self.d_experts, self.s_experts
            host_grads = [c[1] for c in self.cpu]
            adam_now = self.adv_adam and (self.step + 1) % self.acc_step == 0
            adding = self.acc_step > 1 and not getattr(host_grads[0], "lazy_zero", True)
            if host_meta is not None:
                active = [e for e in range(d) if host_meta[1][e] > 0]
                # the optimizer moves every parameter it owns, also those whose gradient is zero
                wanted = list(range(d)) if adam_now else active
            else:
                active, wanted = list(range(d)), list(range(d))
            new_g = lambda n: [torch.empty((n, *hg.shape[1:]), dtype=hg.dtype, device=x2.device) for hg in host_grads]
            if home is not None:
                self._home_fetch(home, wanted, tag)       # what the forward left in place is not copied again
                for (c0, size, ids, p) in self._home_chunks(home, wanted):
                    um.wait_slots(home + c0, size)
                    g = new_g(size)
                    H.ffn_bwd_into(go, x2, h, a, offsets[e0 + c0:], kept_rows[e0 + c0:], size, rows, M, F, p[0], p[2], t,
                                   g[0], g[1], g[2], g[3], gx, False, self.gelu_bwd)
                    if adam_now:
                        self._instant_adam(p, g, list(range(c0, c0 + size)), adding)
                        um.release(home + c0, size)
                    else:
                        um.release(home + c0, size)
                        for (at, r0, n) in self._runs(ids):       # the experts of the chunk that got rows
                            self._store_grad(host_grads, [gg[r0 - c0:r0 - c0 + n] for gg in g], list(range(r0, r0 + n)), adding)
                seen = set(wanted)
            else:
                order, off_c, kept_c = self._order(resident, wanted, offsets, kept_rows, host_meta)
                for (lo, size, pref, view_base) in self._chunks(len(order), len(resident)):
                    ids = order[lo:lo + size]
                    p = um.fetch_ids(self._host(), view_base, ids, pref, tag)   # the reference fetches again (core.cpp:1203)
                    um.wait_slots(view_base, size)
                    g = new_g(size)
                    H.ffn_bwd_into(go, x2, h, a, off_c[lo:], kept_c[lo:], size, rows, M, F, p[0], p[2], t, g[0], g[1],
                                   g[2], g[3], gx, False, self.gelu_bwd)
                    if adam_now:
                        # the update reads the parameters in their pool slots, so the slots are released after it
                        self._instant_adam(p, g, ids, adding)
                        um.release(view_base, size)
                    else:
                        um.release(view_base, size)
                        self._store_grad(host_grads, g, ids, adding)
                seen = set(order)
            if host_meta is not None:
                # experts that got no row: their gradient is zero.  While sums are being built up that adds
                # nothing; otherwise the host array must read zero, which costs a copy only if it does not already
                act = set(active)
                if not adding:
                    stale = [e for e in range(d) if e not in seen and not self._grad_is_zero[e]]
                    um.zero_grads_ids(host_grads, stale)
                    for e in range(d):
                        self._grad_is_zero[e] = e not in act
                else:
                    for e in act:
                        self._grad_is_zero[e] = False
            else:
                self._grad_is_zero = [False] * d
            if adam_now:
                # the next prefetch reads the host parameters that the write-back stream is still filling
                # (the reference ends its backward with a synchronisation of the copy stream, core.cpp:1287)
                um.sync_tran()
        self.step += 1
        for c in self.cpu:
            if c is not None and hasattr(c[1], "lazy_zero"):
                c[1].lazy_zero = False
        return gx.view(shape) if need_gx else None

    @staticmethod
    def _runs(ids):
        """[(position of the run's first expert in ids, first expert, length)] of the runs of consecutive experts."""
        runs, i = [], 0
        while i < len(ids):
            j = i + 1
            while j < len(ids) and ids[j] == ids[j - 1] + 1:
                j += 1
            runs.append((i, ids[i], j - i))
            i = j
        return runs

    def _store_grad(self, host_grads, g, ids, adding):
        """Gradients of offloaded experts go back to their pinned host buffers (core.cpp:77-103,
        uparameter.cpp:68-83): overwrite, or add when accumulating and the buffer is not lazily zero."""
        if adding:
            for (at, e, n) in self._runs(ids):
                self._add_to_host([hg[e:e + n] for hg in host_grads], [gg[at:at + n] for gg in g])
        else:
            get_UniMem().store_grads_ids(host_grads, g, ids)

    @staticmethod
    def _add_to_host(host_slices, g):
        """host_slices += g without stopping the host: the sums of the earlier micro-steps come up on the copy
        stream (after any write-back into them still in flight), are added on the GPU and go back on the
        write-back stream.  The reference adds on the CPU after a blocking copy (data_transfer.cpp:9-12); the
        sum is the same single rounding of the same two operands."""
        um = get_UniMem()
        prev = [torch.empty_like(gg) for gg in g]
        um.load_state(prev, host_slices, after_writeback=True)
        for gg, pp in zip(g, prev):
            H.grad_add(gg, pp)
        um.store_state(host_slices, g)

    def _instant_adam(self, p_slots, g, ids, adding):
        """Adam on the GPU for the experts `ids` of the offloaded set (one chunk, in slot order), inside the
        backward pipeline (core.cpp:848-943): fetch their moments (and, when accumulating, the gradients of the
        earlier micro-steps) from pinned host memory, one fused update per parameter array, write parameters and
        moments back.  Only experts below hybrid_adam_count are updated here; the gradients of the others go to
        the host for the CPU optimizer.  The reference narrows the second weight from the first one when it cuts
        a batch at hybrid_adam_count (core.cpp:859); this follows the evident intent instead."""
        if self.adam is None:
            raise RuntimeError("in-pipeline Adam needs set_adam() before backward")
        if any(c[2] is None or c[3] is None for c in self.cpu):
            raise RuntimeError("in-pipeline Adam needs momentum and variance arrays (set_CPUParamCore)")
        um = get_UniMem()
        host_grads = [c[1] for c in self.cpu]
        es = g[0].element_size()
        for (at, e0, n_run) in self._runs(ids):
            n = max(0, min(n_run, self.hybrid_adam_count - e0))     # experts of the run updated on the GPU
            if n < n_run:          # beyond the GPU-updated prefix: gradients only
                rest = [gg[at + n:at + n_run] for gg in g]
                dst = [hg[e0 + n:e0 + n_run] for hg in host_grads]
                if adding:
                    self._add_to_host(dst, rest)
                else:
                    um.store_state(dst, rest)
            if n == 0:
                continue
            beta1, beta2, t, lr, lam, eps, adamw = self.adam
            dev = g[0].device
            m_host = [c[2][e0:e0 + n] for c in self.cpu]
            v_host = [c[3][e0:e0 + n] for c in self.cpu]
            m = [torch.empty(mh.shape, dtype=torch.float32, device=dev) for mh in m_host]
            v = [torch.empty(vh.shape, dtype=torch.float32, device=dev) for vh in v_host]
            loads_dev, loads_host = m + v, m_host + v_host
            if adding:
                g_prev = [torch.empty((n, *hg.shape[1:]), dtype=hg.dtype, device=dev) for hg in host_grads]
                loads_dev, loads_host = loads_dev + g_prev, loads_host + [hg[e0:e0 + n] for hg in host_grads]
            um.load_state(loads_dev, loads_host, after_writeback=adding)
            p_new = []
            for k in range(4):
                gk = g[k][at:at + n]
                if adding:
                    H.grad_add(gk, g_prev[k])
                out = torch.empty_like(gk)
                per_expert = gk[0].numel() * es
                H.adam_step(p_slots[k] + at * per_expert, gk, m[k], v[k], beta1, beta2, t + 1, lr, lam, eps, adamw, p_out=out)
                p_new.append(out)
            um.store_state([c[0][e0:e0 + n] for c in self.cpu] + m_host + v_host, p_new + m + v)


class BatchFusedFWD(torch.autograd.Function):
    """experts_output = BatchFusedFWD.apply(dispatched_input, module, dummy_param, time_it, prefetch)
    (MOLE/moe/layer.py:453-454).  `dummy_param` makes autograd record the node even when the input
    does not require grad (layer.py:80-81); expert gradients are written straight into the
    parameter stores' gradient buffers, as in the reference."""

    @staticmethod
    def forward(ctx, dispatched_input, module, dummy_param, time_it=False, prefetch=False, offsets=None, kept_rows=None):
        ctx.module = module
        ctx.prefetch = prefetch
        ctx.time_it = bool(time_it)
        out = module.MOLECore.forward(dispatched_input, dispatched_input.requires_grad, offsets, kept_rows)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        if ctx.time_it:       # the expert node's share of the layer's backward (the reference times the same span)
            from .utils.Utimer import UATimer
            UATimer.track_bwd_start(ctx.module.moe_id)
        gx = ctx.module.MOLECore.backward(grad_out)
        if ctx.time_it:
            UATimer.track_bwd_end(ctx.module.moe_id)
        dummy = torch.zeros_like(ctx.module.dummy_param) if ctx.module.dummy_param is not None else None
        return gx, None, dummy, None, None, None, None
