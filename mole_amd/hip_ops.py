"""Tensor-level wrappers of the C ABI: allocate outputs with torch, pass raw pointers, run on
torch's current HIP stream.  No math happens here."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib as L


def _dev(t: torch.Tensor) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError("mole_amd: tensors must live on the GPU (there is no CPU path)")
    if not t.is_contiguous():
        raise RuntimeError("mole_amd: tensors must be contiguous")
    return t


def gemm_nt(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """c[rows,N] = a[rows,K] @ b[N,K].T in fp32 (gate logits)."""
    _dev(a), _dev(b)
    rows, K = a.shape
    N = b.shape[0]
    c = torch.empty(rows, N, dtype=torch.float32, device=a.device)
    L.check(L.lib().mole_gemm_nt(L.ptr(a), L.ptr(b), L.dtype_code(a.dtype), rows, N, K, L.ptr(c), L.stream()), "mole_gemm_nt")
    return c


def gemm_nn(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """c[rows,N] = a[rows,K] @ b[K,N] in the operands' dtype."""
    _dev(a), _dev(b)
    rows, K = a.shape
    N = b.shape[1]
    c = torch.empty(rows, N, dtype=a.dtype, device=a.device)
    L.check(L.lib().mole_gemm_nn(L.ptr(a), L.ptr(b), L.dtype_code(a.dtype), rows, N, K, L.ptr(c), L.stream()), "mole_gemm_nn")
    return c


def softmax_fwd(logits: torch.Tensor, logit_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(logits)
    S, E = logits.shape
    scores = torch.empty_like(logits)
    L.check(L.lib().mole_softmax_fwd(L.ptr(logits), L.ptr(logit_bias), S, E, L.ptr(scores), L.stream()), "mole_softmax_fwd")
    return scores


def gate_fwd(x: torch.Tensor, wg: torch.Tensor, logit_bias: Optional[torch.Tensor] = None,
             fused: Optional[bool] = None) -> torch.Tensor:
    """scores [S,E] fp32 = softmax(x @ wg.T + logit_bias): one fused kernel for small gates (bf16 tokens with
    M % 128 == 0 and E <= 64, where a block of 16-64 tokens re-reads all of wg, which only pays while wg is small, or
    fp32 tokens with M % 4 == 0 and E <= 32), the NT GEMM followed by the softmax kernel otherwise.  fused=True asks for the
    one-kernel path where the kernel allows it (bf16: any E <= 256)."""
    _dev(x), _dev(wg)
    S, M = x.shape
    E = wg.shape[0]
    if fused is None:
        fused = wg.dtype == torch.float32 and (
            (x.dtype == torch.bfloat16 and M % 128 == 0 and E <= 64) or (x.dtype == torch.float32 and M % 4 == 0 and E <= 32))
    if fused:
        scores = torch.empty(S, E, dtype=torch.float32, device=x.device)
        L.check(L.lib().mole_gate_fwd(L.ptr(x), L.dtype_code(x.dtype), L.ptr(wg), L.ptr(logit_bias), S, E, M, L.ptr(scores),
                                      L.stream()), "mole_gate_fwd")
        return scores
    w = wg if wg.dtype == x.dtype else wg.to(x.dtype)
    return softmax_fwd(gemm_nt(x, w.contiguous()), logit_bias)


def gate_bwd(dgates: torch.Tensor, scores: torch.Tensor, idx: torch.Tensor, normalize_gate: bool,
             through_softmax: bool = True, counts0: Optional[torch.Tensor] = None,
             d_l_aux: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d(logits) (through_softmax) or d(scores) from d(gates); with counts0 [E] int32 and d_l_aux [1] fp32 (both on
    the device) the result also carries the gradient of l_aux = E/S^2 sum_e (sum_i scores[i,e]) counts0[e]."""
    _dev(dgates), _dev(scores), _dev(idx)
    S, E = scores.shape
    k = idx.shape[0]
    if (counts0 is None) != (d_l_aux is None):
        raise RuntimeError("gate_bwd: counts0 and d_l_aux go together")
    if d_l_aux is not None:
        _dev(counts0)
        d_l_aux = _dev(d_l_aux.reshape(1).float())
    dlogits = torch.empty_like(scores)
    L.check(L.lib().mole_gate_bwd(L.ptr(dgates), L.ptr(scores), L.ptr(idx), S, E, k, int(normalize_gate), int(through_softmax),
                                  L.ptr(counts0), L.ptr(d_l_aux), L.ptr(dlogits), L.stream()), "mole_gate_bwd")
    return dlogits


def softmax_bwd(dscores: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
    """dlogits = scores * (dscores - sum_e dscores scores)."""
    _dev(dscores), _dev(scores)
    S, E = scores.shape
    dlogits = torch.empty_like(scores)
    L.check(L.lib().mole_softmax_bwd(L.ptr(dscores), L.ptr(scores), S, E, L.ptr(dlogits), L.stream()), "mole_softmax_bwd")
    return dlogits


def gemm_tn(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """c[Mo,N] = a[rows,Mo].T @ b[rows,N] in the operands' dtype."""
    _dev(a), _dev(b)
    rows, Mo = a.shape
    N = b.shape[1]
    c = torch.empty(Mo, N, dtype=a.dtype, device=a.device)
    L.check(L.lib().mole_gemm_tn(L.ptr(a), L.ptr(b), L.dtype_code(a.dtype), rows, Mo, N, L.ptr(c), L.stream()), "mole_gemm_tn")
    return c


def _pad_cols(t: torch.Tensor, mult: int) -> torch.Tensor:
    """t [rows, n] with zero columns appended up to a multiple of `mult` (a copy only when needed)."""
    n = t.shape[1]
    if n % mult == 0:
        return t.contiguous()
    out = torch.zeros(t.shape[0], (n + mult - 1) // mult * mult, dtype=t.dtype, device=t.device)
    out[:, :n] = t
    return out


def gate_input_grad(dlogits: torch.Tensor, wg: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """dx [S,M] = dlogits[S,E] @ wg[E,M] in `dtype` on the grouped-GEMM tiles (the gate's share of the input
    gradient when it is not folded into the dispatch backward).  E is padded with zeros to the tile's granule."""
    epc = 8 if dtype == torch.bfloat16 else 4
    M = wg.shape[1]
    if M % epc:
        raise RuntimeError(f"gate_input_grad: M={M} must be a multiple of {epc}")
    a = _pad_cols(dlogits.to(dtype), epc)
    w = wg.to(dtype)
    if a.shape[1] != w.shape[0]:
        wp = torch.zeros(a.shape[1], M, dtype=dtype, device=w.device)
        wp[:w.shape[0]] = w
        w = wp
    return gemm_nn(a, w.contiguous())


def gate_wgrad(dlogits: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """dWg [E,M] fp32 = dlogits[S,E]^T @ x[S,M], deterministic (partial sums over token chunks, added in a fixed
    order): on the matrix cores for bf16 tokens (E <= 256, M % 64 == 0), on the VALU for small gates (E <= 32) in
    either dtype.  What neither kernel covers is a plain library GEMM (plumbing)."""
    _dev(dlogits), _dev(x)
    S, E = dlogits.shape
    M = x.shape[1]
    mfma = x.dtype == torch.bfloat16 and E <= 256 and M % 64 == 0 and S > 0
    if not mfma and (E > 32 or M % 4 != 0):
        # shapes neither gate kernel takes: the transposed product of the grouped-GEMM tiles (one tile per block,
        # the contraction over all tokens inside it), E padded to the tile's granule
        epc = 8 if x.dtype == torch.bfloat16 else 4
        if M % epc:
            raise RuntimeError(f"gate_wgrad: M={M} must be a multiple of {epc}")
        return gemm_tn(_pad_cols(dlogits.to(x.dtype), epc), x)[:E].float()
    dwg = torch.empty(E, M, dtype=torch.float32, device=x.device)
    nbytes = L.lib().mole_gate_wgrad_workspace_bytes(S, E, M)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    L.check(L.lib().mole_gate_wgrad(L.ptr(dlogits), L.ptr(x), L.dtype_code(x.dtype), S, E, M, L.ptr(dwg), L.ptr(ws), nbytes,
                                    L.stream()), "mole_gate_wgrad")
    return dwg


@dataclass
class Route:
    """Device-side result of mole_route (what tutel's extract_critical returns, plus the ragged
    bookkeeping).  Nothing here forces a host synchronisation."""
    S: int
    E: int
    k: int
    layout: int
    idx: torch.Tensor        # [k,S] int32
    loc: torch.Tensor        # [k,S] int32
    gates: torch.Tensor      # [k,S] fp32
    row: torch.Tensor        # [k,S] int32
    counts: torch.Tensor     # [k,E] int32
    kept_rows: torch.Tensor  # [E] int32
    offsets: torch.Tensor    # [E+1] int32
    capacity: torch.Tensor   # [1] int32
    l_aux: torch.Tensor      # [1] fp32
    normalize_gate: bool = True


def route(scores: torch.Tensor, top_k: int, capacity_factor: float = 1.0, normalize_gate: bool = True,
          alignment: int = 1, layout: int = L.LAYOUT_RAGGED) -> Route:
    _dev(scores)
    if scores.dtype != torch.float32:
        raise TypeError("mole_route takes fp32 scores")
    S, E = scores.shape
    k = min(int(top_k), E)
    dev = scores.device
    i32 = dict(dtype=torch.int32, device=dev)
    idx, loc, row = (torch.empty(k, S, **i32) for _ in range(3))
    gates = torch.empty(k, S, dtype=torch.float32, device=dev)
    meta = torch.empty(k * E + E + (E + 1) + 1, **i32)
    counts = meta[:k * E].view(k, E)
    kept = meta[k * E:k * E + E]
    offsets = meta[k * E + E:k * E + 2 * E + 1]
    cap = meta[k * E + 2 * E + 1:]
    l_aux = torch.empty(1, dtype=torch.float32, device=dev)
    nbytes = L.lib().mole_route_workspace_bytes(S, E, k)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    L.check(L.lib().mole_route(L.ptr(scores), S, E, k, float(capacity_factor), int(normalize_gate), int(alignment),
                               int(layout), L.ptr(idx), L.ptr(loc), L.ptr(gates), L.ptr(row), L.ptr(counts),
                               L.ptr(kept), L.ptr(offsets), L.ptr(cap), L.ptr(l_aux), L.ptr(ws), nbytes, L.stream()),
            "mole_route")
    return Route(S, E, k, layout, idx, loc, gates, row, counts, kept, offsets, cap, l_aux, normalize_gate)


def gate_route_fused(x: torch.Tensor, wg: torch.Tensor) -> bool:
    """Whether gate_route() takes (x, wg) in its one-call form."""
    return (x.dtype == torch.bfloat16 and wg.dtype == torch.float32 and wg.shape[0] <= 64 and x.shape[1] % 128 == 0
            and x.shape[0] >= 1)


def gate_route(x: torch.Tensor, wg: torch.Tensor, logit_bias: Optional[torch.Tensor], top_k: int,
               capacity_factor: float = 1.0, normalize_gate: bool = True, alignment: int = 1,
               layout: int = L.LAYOUT_RAGGED):
    """(scores, Route) = (gate_fwd(x, wg, logit_bias), route(scores, ...)): for small gates on bf16 tokens one call whose
    gate kernel also does the routing's first stage (mole_gate_route), otherwise the two calls."""
    _dev(x), _dev(wg)
    if not gate_route_fused(x, wg):
        scores = gate_fwd(x, wg, logit_bias)
        return scores, route(scores, top_k, capacity_factor, normalize_gate, alignment, layout)
    S, M = x.shape
    E = wg.shape[0]
    k = min(int(top_k), E)
    dev = x.device
    i32 = dict(dtype=torch.int32, device=dev)
    scores = torch.empty(S, E, dtype=torch.float32, device=dev)
    idx, loc, row = (torch.empty(k, S, **i32) for _ in range(3))
    gates = torch.empty(k, S, dtype=torch.float32, device=dev)
    meta = torch.empty(k * E + E + (E + 1) + 1, **i32)
    counts = meta[:k * E].view(k, E)
    kept = meta[k * E:k * E + E]
    offsets = meta[k * E + E:k * E + 2 * E + 1]
    cap = meta[k * E + 2 * E + 1:]
    l_aux = torch.empty(1, dtype=torch.float32, device=dev)
    nbytes = L.lib().mole_gate_route_workspace_bytes(S, E, k)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    L.check(L.lib().mole_gate_route(L.ptr(x), L.dtype_code(x.dtype), L.ptr(wg), L.ptr(logit_bias), S, E, M, k,
                                    float(capacity_factor), int(normalize_gate), int(alignment), int(layout), L.ptr(scores),
                                    L.ptr(idx), L.ptr(loc), L.ptr(gates), L.ptr(row), L.ptr(counts), L.ptr(kept), L.ptr(offsets),
                                    L.ptr(cap), L.ptr(l_aux), L.ptr(ws), nbytes, L.stream()), "mole_gate_route")
    return scores, Route(S, E, k, layout, idx, loc, gates, row, counts, kept, offsets, cap, l_aux, normalize_gate)


def dispatch_fwd(x: torch.Tensor, row: torch.Tensor, total_rows: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(x), _dev(row)
    S, M = x.shape
    k = row.shape[0]
    xd = out if out is not None else torch.empty(total_rows, M, dtype=x.dtype, device=x.device)
    if xd.numel() == 0:          # every pair was dropped: nothing to scatter
        return xd
    L.check(L.lib().mole_dispatch_fwd(L.ptr(x), L.dtype_code(x.dtype), L.ptr(row), S, M, k, L.ptr(xd), L.stream()),
            "mole_dispatch_fwd")
    return xd


def dispatch_bwd(dxd: torch.Tensor, row: torch.Tensor, dlogits: Optional[torch.Tensor] = None,
                 wg: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dx = gather-sum of dxd rows (+ dlogits @ wg, the gate's share of the input gradient).  Small gates
    are folded into the gather kernel; for larger ones the product runs first on the grouped-GEMM tiles."""
    _dev(dxd), _dev(row)
    k, S = row.shape
    M = dxd.shape[-1]
    if dxd.numel() == 0:         # every pair was dropped: the kernel still wants one (unused) row to read
        dxd = torch.zeros(1, M, dtype=dxd.dtype, device=dxd.device)
    dx = torch.empty(S, M, dtype=dxd.dtype, device=dxd.device)
    E = 0
    dx_add = None
    if dlogits is not None:
        _dev(dlogits), _dev(wg)
        E = wg.shape[0]
        if wg.dtype != torch.float32 or dlogits.dtype != torch.float32:
            raise TypeError("gate tensors are fp32")
        epc = 8 if dxd.dtype == torch.bfloat16 else 4
        if E > 32 and M % epc == 0:
            dx_add = gate_input_grad(dlogits, wg, dxd.dtype)
            dlogits, wg, E = None, None, 0
    L.check(L.lib().mole_dispatch_bwd(L.ptr(dxd), L.dtype_code(dxd.dtype), L.ptr(row), S, M, k, L.ptr(dlogits), L.ptr(wg),
                                      E, L.ptr(dx_add), L.ptr(dx), L.stream()), "mole_dispatch_bwd")
    return dx


def combine_fwd(o: torch.Tensor, row: torch.Tensor, gates: torch.Tensor) -> torch.Tensor:
    _dev(o), _dev(row), _dev(gates)
    k, S = row.shape
    M = o.shape[-1]
    if o.numel() == 0:           # every pair was dropped: all tokens output zeros
        return torch.zeros(S, M, dtype=o.dtype, device=o.device)
    y = torch.empty(S, M, dtype=o.dtype, device=o.device)
    L.check(L.lib().mole_combine_fwd(L.ptr(o), L.dtype_code(o.dtype), L.ptr(row), L.ptr(gates), S, M, k, L.ptr(y), L.stream()),
            "mole_combine_fwd")
    return y


def combine_bwd(dy: torch.Tensor, o: torch.Tensor, row: torch.Tensor, gates: torch.Tensor,
                d_o: Optional[torch.Tensor] = None):
    _dev(dy), _dev(o), _dev(row), _dev(gates)
    k, S = row.shape
    M = o.shape[-1]
    if d_o is None:
        d_o = torch.empty_like(o)
    if o.numel() == 0:
        return d_o, torch.zeros(k, S, dtype=torch.float32, device=o.device)
    dgates = torch.empty(k, S, dtype=torch.float32, device=o.device)
    L.check(L.lib().mole_combine_bwd(L.ptr(dy), L.ptr(o), L.dtype_code(o.dtype), L.ptr(row), L.ptr(gates), S, M, k,
                                     L.ptr(d_o), L.ptr(dgates), L.stream()), "mole_combine_bwd")
    return d_o, dgates


def combine_bwd_gate(dy: torch.Tensor, o: torch.Tensor, row: torch.Tensor, gates: torch.Tensor, scores: torch.Tensor,
                     idx: torch.Tensor, normalize_gate: bool, through_softmax: bool = True,
                     counts0: Optional[torch.Tensor] = None, d_l_aux: Optional[torch.Tensor] = None):
    """combine_bwd and gate_bwd in one kernel (gates of up to 256 experts): returns d_o and d(logits) (or d(scores)
    when not through_softmax).  Larger gates, and the case where every pair was dropped, take the two calls."""
    S, E = scores.shape
    if E > 256 or o.numel() == 0:
        d_o, dgates = combine_bwd(dy, o, row, gates)
        return d_o, gate_bwd(dgates, scores, idx, normalize_gate, through_softmax, counts0, d_l_aux)
    _dev(dy), _dev(o), _dev(row), _dev(gates), _dev(scores), _dev(idx)
    k = row.shape[0]
    M = o.shape[-1]
    if (counts0 is None) != (d_l_aux is None):
        raise RuntimeError("combine_bwd_gate: counts0 and d_l_aux go together")
    if d_l_aux is not None:
        _dev(counts0)
        d_l_aux = _dev(d_l_aux.reshape(1).float())
    d_o = torch.empty_like(o)
    dlogits = torch.empty_like(scores)
    L.check(L.lib().mole_combine_bwd_gate(L.ptr(dy), L.ptr(o), L.dtype_code(o.dtype), L.ptr(row), L.ptr(gates), S, M, k,
                                          L.ptr(d_o), L.ptr(scores), L.ptr(idx), E, int(normalize_gate), int(through_softmax),
                                          L.ptr(counts0), L.ptr(d_l_aux), L.ptr(dlogits), L.stream()), "mole_combine_bwd_gate")
    return d_o, dlogits


def zero_pad_rows(buf: torch.Tensor, kept_rows: torch.Tensor, offsets: torch.Tensor) -> None:
    _dev(buf)
    E = kept_rows.shape[0]
    M = buf.shape[-1]
    L.check(L.lib().mole_zero_pad_rows(L.ptr(buf), L.dtype_code(buf.dtype), L.ptr(kept_rows), L.ptr(offsets), E, M, L.stream()),
            "mole_zero_pad_rows")


def ffn_fwd_into(xd, offsets, kept_rows, E, max_rows, M, F, w1, b1, w2, b2, h, a, out) -> None:
    """mole_ffn_fwd on caller-provided buffers.  Weights may be tensors or raw device addresses
    (slot-pool pointers); offsets/kept_rows may be views starting at the first expert of a chunk."""
    L.check(L.lib().mole_ffn_fwd(L.ptr(xd), L.dtype_code(xd.dtype), L.ptr(offsets), L.ptr(kept_rows), int(E), int(max_rows),
                                 int(M), int(F), L.ptr(w1), L.ptr(b1), L.ptr(w2), L.ptr(b2), L.ptr(h), L.ptr(a), L.ptr(out),
                                 L.stream()), "mole_ffn_fwd")


def ffn_bwd_into(go, xd, h, a, offsets, kept_rows, E, max_rows, M, F, w1, w2, t, g_w1, g_b1, g_w2, g_b2, gx,
                 accumulate: bool, gelu_bwd: int) -> None:
    L.check(L.lib().mole_ffn_bwd(L.ptr(go), L.ptr(xd), L.ptr(h), L.ptr(a), L.dtype_code(xd.dtype), L.ptr(offsets),
                                 L.ptr(kept_rows), int(E), int(max_rows), int(M), int(F), L.ptr(w1), L.ptr(w2), L.ptr(t),
                                 L.ptr(g_w1), L.ptr(g_b1), L.ptr(g_w2), L.ptr(g_b2), L.ptr(gx), int(accumulate),
                                 int(gelu_bwd), L.stream()), "mole_ffn_bwd")


def ffn_fwd(xd, offsets, kept_rows, w1, b1, w2, b2, max_rows: Optional[int] = None):
    """Returns (out [rows,M], h [rows,F], a [rows,F])."""
    for t in (xd, offsets, kept_rows, w1, b1, w2, b2):
        _dev(t)
    rows, M = xd.shape
    E, F, _ = w1.shape
    max_rows = rows if max_rows is None else max_rows
    h = torch.empty(rows, F, dtype=xd.dtype, device=xd.device)
    a = torch.empty(rows, F, dtype=xd.dtype, device=xd.device)
    out = torch.empty(rows, M, dtype=xd.dtype, device=xd.device)
    ffn_fwd_into(xd, offsets, kept_rows, E, max_rows, M, F, w1, b1, w2, b2, h, a, out)
    return out, h, a


def ffn_bwd(go, xd, h, a, offsets, kept_rows, w1, w2, g_w1, g_b1, g_w2, g_b2, need_gx: bool = True,
            accumulate: bool = False, gelu_bwd: int = L.GELU_BWD_TANH, max_rows: Optional[int] = None):
    """Writes (or accumulates into) g_w1, g_b1, g_w2, g_b2; returns gx [rows,M] or None."""
    for t in (go, xd, h, a, offsets, kept_rows, w1, w2, g_w1, g_b1, g_w2, g_b2):
        _dev(t)
    rows, M = xd.shape
    E, F, _ = w1.shape
    max_rows = rows if max_rows is None else max_rows
    t = torch.empty(rows, F, dtype=xd.dtype, device=xd.device)
    gx = torch.empty(rows, M, dtype=xd.dtype, device=xd.device) if need_gx else None
    ffn_bwd_into(go, xd, h, a, offsets, kept_rows, E, max_rows, M, F, w1, w2, t, g_w1, g_b1, g_w2, g_b2, gx, accumulate,
                 gelu_bwd)
    return gx


def grad_add(acc: torch.Tensor, add: torch.Tensor) -> None:
    """acc += add, element by element in the tensors' dtype (one rounding): gradient sums over micro-steps."""
    _dev(acc); _dev(add)
    if acc.dtype != add.dtype or acc.numel() != add.numel() or not (acc.is_contiguous() and add.is_contiguous()):
        raise RuntimeError("mole_amd.grad_add: acc and add must be contiguous and agree in dtype and size")
    L.check(L.lib().mole_grad_add(L.ptr(acc), L.ptr(add), acc.numel(), L.dtype_code(acc.dtype), L.stream()), "mole_grad_add")


def adam_step(p, g, m, v, beta1: float, beta2: float, t: int, lr: float, lam: float, eps: float, adamw: bool,
              p_out=None) -> None:
    """One fused Adam / AdamW step (define.hpp:543-579) over all elements of p: m and v (fp32) are updated in
    place, the new parameters go to p_out (p itself when None).  t is the step count already incremented.
    p may be a raw device address (a slot of the parameter pool) holding g.numel() elements of g's dtype."""
    for x in (g, m, v):
        _dev(x)
    if isinstance(p, int):
        if p_out is None:
            p_out = p
    else:
        _dev(p)
        if p.dtype != g.dtype or p.numel() != g.numel():
            raise RuntimeError("mole_amd.adam_step: p and g must agree in dtype and size")
        p_out = p if p_out is None else p_out
    if not isinstance(p_out, int):
        _dev(p_out)
        if p_out.dtype != g.dtype or p_out.numel() != g.numel():
            raise RuntimeError("mole_amd.adam_step: p_out and g must agree in dtype and size")
    if m.dtype != torch.float32 or v.dtype != torch.float32:
        raise RuntimeError("mole_amd.adam_step: m and v are fp32")
    n = g.numel()
    if not (m.numel() == v.numel() == n):
        raise RuntimeError("mole_amd.adam_step: g, m, v must have the same number of elements")
    L.check(L.lib().mole_adam_step(L.ptr(p), L.ptr(g), L.ptr(m), L.ptr(v), L.ptr(p_out), n, L.dtype_code(g.dtype),
                                   float(beta1), float(beta2), int(t), float(lr), float(lam), float(eps), int(bool(adamw)),
                                   L.stream()), "mole_adam_step")
