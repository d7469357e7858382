"""ctypes binding of libmole_hip.so (the C ABI declared in include/mole_hip.h).

The library is the product path: if it is missing this module raises, it never falls back to
another implementation.  torch is imported first so that the HIP runtime the process already
holds is the one the library binds to.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

import torch  # noqa: F401  (must precede the dlopen below)

LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "MOLE", "cpp", "libmole_hip.so")

MOLE_F32, MOLE_BF16 = 0, 1
LAYOUT_PADDED, LAYOUT_RAGGED = 0, 1
GELU_BWD_TANH, GELU_BWD_EXACT = 0, 1
MAX_TOPK, MAX_EXPERTS = 16, 1024
KERNEL_IDS = ("ffn_fwd1", "ffn_fwd2", "ffn_gw2", "ffn_da", "ffn_gw1", "ffn_gx", "ffn_gb", "dispatch_fwd", "dispatch_bwd",
              "combine_fwd", "combine_bwd", "route", "gemm_nt", "adam", "gate_fwd", "gate_bwd", "gate_wgrad", "probe")

_P = c_void_p
_SIGNATURES = {
    "mole_version": (c_int, []),
    "mole_last_error_string": (c_char_p, []),
    "mole_kernel_timing_enable": (c_int, [c_int]),
    "mole_kernel_timing_read": (c_int, [c_int, POINTER(c_int), POINTER(c_float)]),
    "mole_probe_mfma_operand_bytes": (c_size_t, []),
    "mole_probe_mfma": (c_int, [_P, c_int, c_int, _P, POINTER(c_double), _P]),
    "mole_probe_kloop": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "mole_probe_kloop_part": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "mole_softmax_fwd": (c_int, [_P, _P, c_int, c_int, _P, _P]),
    "mole_gate_fwd": (c_int, [_P, c_int, _P, _P, c_int, c_int, c_int, _P, _P]),
    "mole_softmax_bwd": (c_int, [_P, _P, c_int, c_int, _P, _P]),
    "mole_gate_bwd": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P, _P, _P, _P]),
    "mole_gate_wgrad_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mole_gate_wgrad": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_size_t, _P]),
    "mole_route_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mole_route": (c_int, [_P, c_int, c_int, c_int, c_double, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
                           _P, _P, c_size_t, _P]),
    "mole_gate_route_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mole_gate_route": (c_int, [_P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_double, c_int, c_int, c_int, _P, _P, _P, _P, _P,
                                _P, _P, _P, _P, _P, _P, c_size_t, _P]),
    "mole_route_static_max_bytes": (c_size_t, []),
    "mole_route_static": (c_int, [_P, c_int, c_int, c_int, c_double, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P,
                                  _P, _P]),
    "mole_dispatch_fwd": (c_int, [_P, c_int, _P, c_int, c_int, c_int, _P, _P]),
    "mole_dispatch_bwd": (c_int, [_P, c_int, _P, c_int, c_int, c_int, _P, _P, c_int, _P, _P, _P]),
    "mole_combine_fwd": (c_int, [_P, c_int, _P, _P, c_int, c_int, c_int, _P, _P]),
    "mole_combine_bwd": (c_int, [_P, _P, c_int, _P, _P, c_int, c_int, c_int, _P, _P, _P]),
    "mole_combine_bwd_gate": (c_int, [_P, _P, c_int, _P, _P, c_int, c_int, c_int, _P, _P, _P, c_int, c_int, c_int, _P, _P, _P, _P]),
    "mole_zero_pad_rows": (c_int, [_P, c_int, _P, _P, c_int, c_int, _P]),
    "mole_ffn_fwd": (c_int, [_P, c_int, _P, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P]),
    "mole_ffn_bwd": (c_int, [_P, _P, _P, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P,
                             _P, c_int, c_int, _P]),
    "mole_gemm_nt": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "mole_gemm_nn": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "mole_gemm_tn": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P]),
    "mole_unimem_create": (c_int, [c_int, c_int, c_int, c_int64, c_int64, POINTER(_P)]),
    "mole_unimem_destroy": (c_int, [_P]),
    "mole_unimem_clear_virtual_mem": (c_int, [_P]),
    "mole_unimem_view_pool_size": (c_int, [_P, POINTER(c_int)]),
    "mole_unimem_virtual_offset": (c_int, [_P, POINTER(c_int)]),
    "mole_unimem_slot_ptr": (c_int, [_P, c_int, c_int, POINTER(_P)]),
    "mole_unimem_prefetch": (c_int, [_P, c_int, POINTER(_P), c_int, c_int]),
    "mole_unimem_prefetch_ids": (c_int, [_P, c_int, POINTER(_P), POINTER(c_int32), c_int, c_uint64]),
    "mole_unimem_reserve": (c_int, [_P, c_int, c_int, POINTER(_P)]),
    "mole_unimem_fetch_top": (c_int, [_P, c_int, POINTER(c_int)]),
    "mole_unimem_fetch": (c_int, [_P, POINTER(_P), c_int, c_int, c_int, c_int, POINTER(_P)]),
    "mole_unimem_fetch_ids": (c_int, [_P, POINTER(_P), c_int, POINTER(c_int32), c_int, c_int, c_uint64, POINTER(_P)]),
    "mole_unimem_wait_params": (c_int, [_P, _P]),
    "mole_unimem_wait_slots": (c_int, [_P, c_int, c_int, _P]),
    "mole_unimem_release": (c_int, [_P, c_int, c_int, _P]),
    "mole_unimem_sync_tran": (c_int, [_P]),
    "mole_unimem_tran_stream": (c_int, [_P, POINTER(_P)]),
    "mole_unimem_copy_stats": (c_int, [_P, POINTER(c_uint64), POINTER(c_float)]),
    "mole_unimem_reuse_stats": (c_int, [_P, POINTER(c_uint64)]),
    "mole_unimem_store_grads": (c_int, [_P, POINTER(_P), POINTER(_P), c_int, c_int, _P]),
    "mole_unimem_store_grads_ids": (c_int, [_P, POINTER(_P), POINTER(_P), POINTER(c_int32), c_int, _P]),
    "mole_unimem_zero_grads_ids": (c_int, [_P, POINTER(_P), POINTER(c_int32), c_int]),
    "mole_unimem_sync_tranback": (c_int, [_P]),
    "mole_unimem_tranback_stream": (c_int, [_P, POINTER(_P)]),
    "mole_unimem_writeback_stats": (c_int, [_P, POINTER(c_uint64), POINTER(c_float)]),
    "mole_unimem_load_state": (c_int, [_P, POINTER(_P), POINTER(_P), POINTER(c_size_t), c_int, c_int, _P]),
    "mole_unimem_store_state": (c_int, [_P, POINTER(_P), POINTER(_P), POINTER(c_size_t), c_int, _P]),
    "mole_adam_step": (c_int, [_P, _P, _P, _P, _P, c_size_t, c_int, c_float, c_float, c_int, c_float, c_float, c_float,
                               c_int, _P]),
    "mole_grad_add": (c_int, [_P, _P, c_size_t, c_int, _P]),
    "mole_fast_assign_prefetch": (c_int, [c_int, POINTER(c_int), POINTER(c_int), c_int, POINTER(c_int),
                                          POINTER(c_int), c_int, POINTER(c_int)]),
}
EXPORTS = tuple(_SIGNATURES)

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension is the only implementation of the MoE hot path. "
                "Build it with `python -m mole_amd.build` (needs hipcc, no GPU).")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library does not export it
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().mole_last_error_string().decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed (code {rc}): {last_error()}")


def kernel_timing_enable(on: bool) -> None:
    check(lib().mole_kernel_timing_enable(int(on)), "mole_kernel_timing_enable")


def kernel_timing_read() -> dict:
    """{kernel name: (launches, total ms)} since the last read; waits for the recorded events."""
    n = len(KERNEL_IDS)
    counts, ms = (c_int * n)(), (c_float * n)()
    check(lib().mole_kernel_timing_read(n, counts, ms), "mole_kernel_timing_read")
    return {KERNEL_IDS[i]: (counts[i], ms[i]) for i in range(n)}


def ptr(t):
    """Raw device/host pointer of a tensor; integers (addresses from the slot pool) pass through."""
    if t is None:
        return None
    if isinstance(t, int):
        return c_void_p(t)
    return c_void_p(t.data_ptr())


def stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return MOLE_F32
    if dt == torch.bfloat16:
        return MOLE_BF16
    raise TypeError(f"mole_amd supports float32 and bfloat16, got {dt}")
