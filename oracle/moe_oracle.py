"""CPU oracle for the single-GPU MoE-layer hot path of MOLE.  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it.  Nothing under mole_amd/ imports it.

It restates, on the CPU (numpy for the integer work, torch-CPU library routines for the
floating-point work), what the reference computes along the path

    gate -> extract_critical -> fast_encode -> grouped expert FFN -> fast_decode
    (reference: MOLE/moe/layer.py:429-476)

Sources followed, function by function (paths are inside the reference tree):

  gate_scores          MOLE/utils/Ugate.py:5-14 (Linear without bias, softmax over experts)
  extract_critical     call site MOLE/moe/layer.py:445-446.  The implementation lives in the
                       third-party package `tutel` (github.com/microsoft/tutel,
                       tutel/impls/fast_dispatch.py), an empty, UNPINNED git submodule of the
                       reference (.gitmodules:4-6): its published algorithm is restated here.
  fast_encode          call site MOLE/moe/layer.py:448-449 (tutel GatingEncoder)
  fast_decode          call site MOLE/moe/layer.py:457-458 (tutel GatingDecoder)
  gshard_loss          stored at MOLE/moe/layer.py:447 (tutel/impls/losses.py)
  ffn_fwd              MOLE/cpp/core.cpp:344-356 (_BatchRecord::bffn_fwd, GELU branch)
  ffn_bwd              MOLE/cpp/core.cpp:381-414 (_BatchRecord::bffn_bwd) and 457-491 (+= variant)
  d_gelu_tanh          MOLE/cpp/gelu.cu:3-14
  UniMemModel          MOLE/cpp/umemory.cpp:92-183, MOLE/cpp/core.cpp:41-75, 1017-1051
  fast_assign_prefetch MOLE/cpp/core.cpp:1302-1345
  adam_step            MOLE/cpp/define.hpp:543-579 (_MOLECore::adam, used by instant_adam,
                       MOLE/cpp/core.cpp:848-943)

Parity status.
  * ffn_fwd / ffn_bwd / d_gelu_tanh / gate_scores reduce to torch library routines and closed
    forms; tests/test_oracle_*.py pin them (torch autograd, fp64, closed-form spot values).
  * extract_critical / fast_encode / fast_decode / gshard_loss: the reference holds no source,
    no test and no fixture for them (tutel is absent and unpinned), so parity with the exact
    tutel commit the reference's authors used is UNPINNED.  What is pinned is the published
    algorithm: brute-force top-k with the (score desc, index asc) order, stable-sort closed form
    for locations, integer closed form for capacity, permutation invariants, adjointness of
    encode/decode backward, torch autograd on a dense one-hot formulation.
  * UniMemModel / fast_assign_prefetch are integer state machines restated from the C++; fast_assign_prefetch is
    also checked against the reference's own function, compiled from where it lies by oracle/build_ref.py into
    oracle/_ref/libmole_ref.so (tests/test_oracle_ref.py: every small input and thousands of random ones).
  * adam_step is pinned against torch.optim.Adam and torch.optim.AdamW over several steps in fp64
    and against hand-computed first-step values (tests/test_oracle_adam.py).

Floating point: everything is evaluated in the dtype of the inputs (fp32 by default; pass fp64
tensors for an error budget).  bf16 inputs are compared by up-casting the *same rounded values*
to fp32 first.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

FP32_EPS = float(np.finfo(np.float32).eps)  # 1.1920929e-07, torch.finfo(torch.float32).eps


# --------------------------------------------------------------------------------------------
# A1  gate  (MOLE/utils/Ugate.py:11-14)
# --------------------------------------------------------------------------------------------
def gate_scores(x: torch.Tensor, wg: torch.Tensor, logit_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """scores = softmax(x @ wg.T (+ logit_bias), dim=-1); x [S,M], wg [E,M] -> [S,E].

    The reference gate has no bias (Ugate.py:9); `logit_bias` [E] is the hook the imbalanced
    benchmark configuration needs and defaults to None.
    """
    logits = F.linear(x, wg)
    if logit_bias is not None:
        logits = logits + logit_bias
    return F.softmax(logits, dim=-1)


# --------------------------------------------------------------------------------------------
# A2-A6  routing  (tutel.impls.fast_dispatch.extract_critical; call: MOLE/moe/layer.py:445-446)
# --------------------------------------------------------------------------------------------
@dataclass
class Critical:
    """What extract_critical returns, plus the ragged bookkeeping derived from it."""
    num_experts: int
    indices_s: List[np.ndarray]      # k x [S] int32
    locations_s: List[np.ndarray]    # k x [S] int32
    gates_s: List[np.ndarray]        # k x [S] float32
    capacity: int
    counts: np.ndarray               # [k,E] int32   per-choice per-expert token counts
    kept_rows: np.ndarray            # [E]   int32   n[e] = min(sum_j counts[j,e], capacity)
    offsets: np.ndarray              # [E+1] int32   ragged row offsets (prefix sum of kept_rows)
    l_aux: float = 0.0

    @property
    def top_k(self) -> int:
        return len(self.indices_s)

    def tutel_tuple(self):
        return (self.num_experts, self.indices_s, self.locations_s, self.gates_s, self.capacity)

    def rows(self, ragged: bool) -> np.ndarray:
        """[k,S] int32 destination row of every (choice, token) pair, -1 when dropped.

        ragged=False is the reference layout row = e*C + loc into an [E*C, M] buffer;
        ragged=True packs experts back to back: row = offsets[e] + loc.
        """
        out = np.full((self.top_k, len(self.indices_s[0])), -1, dtype=np.int32)
        for j in range(self.top_k):
            e = self.indices_s[j].astype(np.int64)
            loc = self.locations_s[j].astype(np.int64)
            base = self.offsets[e].astype(np.int64) if ragged else e * self.capacity
            keep = loc < self.capacity
            out[j, keep] = (base + loc)[keep].astype(np.int32)
        return out


def topk_lowest_index_ties(scores: np.ndarray, k: int) -> np.ndarray:
    """[S,k] int32: experts sorted by (score descending, expert index ascending).

    torch.topk leaves the order of equal scores unspecified; the rule of record is "ties go to the
    lowest expert index".  NaN compares greater than every number (torch.topk's convention) and
    NaNs tie with each other.
    """
    scores = np.asarray(scores)
    S, E = scores.shape
    isn = np.isnan(scores)
    val = np.where(isn, np.inf, scores)
    idx = np.broadcast_to(np.arange(E), (S, E))
    # np.lexsort: last key is the primary one.  ~isn puts NaN (False) first.
    order = np.lexsort((idx, -val, ~isn), axis=-1)
    return order[:, :k].astype(np.int32)


def _one_hot(idx: np.ndarray, E: int) -> np.ndarray:
    m = np.zeros((idx.shape[0], E), dtype=np.int32)
    m[np.arange(idx.shape[0]), idx] = 1
    return m


def compute_capacity(S: int, E: int, k: int, capacity_factor: float, max_loc_plus_one: int,
                     alignment: int = 1) -> int:
    """Capacity rule of extract_critical: k*int(cf*ceil(S/E)) for cf>0; max(loc)+1 for cf==0;
    min of both for cf<0; then rounded up to `alignment`."""
    spe = (S + E - 1) // E
    if capacity_factor > 0:
        cap = k * int(capacity_factor * spe)
    else:
        cap = int(max_loc_plus_one)
        if capacity_factor < 0:
            cap = min(cap, k * int(-capacity_factor * spe))
    rem = cap % alignment
    if rem > 0:
        cap += alignment - rem
    return cap


def extract_critical(scores, top_k: int, capacity_factor: float = 1.0, normalize_gate: bool = True,
                     alignment: int = 1) -> Critical:
    """Restatement of tutel's extract_critical (non-batch-prioritised, single group).

    indices  : top-k of every row, ties to the lowest expert index.
    gates    : score at the chosen expert; for k>1 and normalize_gate divided by
               clamp(sum_j gate_j, min=fp32 eps), the sum taken left to right in fp32.
    locations: cumsum(one_hot, dim=0) - 1 masked to the chosen column; choice j additionally
               offset by the counts of all earlier choices ("k-major": every first choice of an
               expert is placed before any second choice).
    capacity : see compute_capacity.  A pair is kept iff location < capacity.
    """
    scores = np.ascontiguousarray(np.asarray(scores, dtype=np.float32))
    S, E = scores.shape
    k = min(int(top_k), E)
    topk = topk_lowest_index_ties(scores, k)
    indices_s = [np.ascontiguousarray(topk[:, j]) for j in range(k)]
    masks = [_one_hot(ix, E) for ix in indices_s]
    rows = np.arange(S)
    gates_s = [scores[rows, ix].astype(np.float32) for ix in indices_s]

    counts = np.stack([m.sum(axis=0) for m in masks]).astype(np.int32) if S > 0 else np.zeros((k, E), np.int32)
    locations_s = []
    acc_base = np.zeros((1, E), dtype=np.int64)
    for j in range(k):
        loc = np.cumsum(masks[j], axis=0, dtype=np.int64) - 1
        if j > 0:
            acc_base = acc_base + masks[j - 1].sum(axis=0, keepdims=True)
            loc = loc + acc_base
        locations_s.append((loc * masks[j]).sum(axis=1).astype(np.int32))
    if k > 1 and normalize_gate:
        denom = np.zeros(S, dtype=np.float32)
        for g in gates_s:                       # python sum(): left to right, fp32
            denom = (denom + g).astype(np.float32)
        denom = np.maximum(denom, np.float32(FP32_EPS))
        gates_s = [(g / denom).astype(np.float32) for g in gates_s]

    max_loc_p1 = int(max(int(l.max()) for l in locations_s)) + 1 if S > 0 else 0
    cap = compute_capacity(S, E, k, capacity_factor, max_loc_p1, alignment)
    kept = np.minimum(counts.sum(axis=0), cap).astype(np.int32)
    offsets = np.zeros(E + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(kept)
    l_aux = gshard_loss(scores, indices_s[0]) if S > 0 else 0.0
    return Critical(E, indices_s, locations_s, gates_s, cap, counts, kept, offsets, l_aux)


def gshard_loss(scores: np.ndarray, top1_idx: np.ndarray) -> float:
    """l_aux = E/S^2 * sum_e (sum_i scores[i,e]) * (#tokens whose first choice is e)."""
    scores = np.asarray(scores, dtype=np.float64)
    S, E = scores.shape
    me = scores.sum(axis=0)
    ce = np.bincount(np.asarray(top1_idx, dtype=np.int64), minlength=E).astype(np.float64)
    return float((me * ce).sum() * (E / (S * S)))


def gshard_loss_bwd(S: int, counts0: np.ndarray, d_l_aux: float = 1.0) -> torch.Tensor:
    """d l_aux / d scores, [S,E]: E/S^2 * counts0[e] for every token (the counts are integers and carry no
    gradient; tutel detaches them the same way by building them from the top-k indices)."""
    E = len(counts0)
    row = torch.from_numpy(np.asarray(counts0, dtype=np.float64)) * (d_l_aux * E / (S * S))
    return row.unsqueeze(0).expand(S, E).clone()


# --------------------------------------------------------------------------------------------
# A7 / A8  dispatch (encode) and combine (decode), forward and backward
# --------------------------------------------------------------------------------------------
def fast_encode(x: torch.Tensor, crit: Critical, ragged: bool = False) -> torch.Tensor:
    """GatingEncoder forward with is_postscore=True: D[row(j,i),:] += x[i,:] on a zeroed buffer.

    Returns [E, C, M] (reference layout) or, with ragged=True, [R, M] with R = offsets[-1].
    Destination rows are unique, so the += is a copy.
    """
    S, M = x.shape
    nrows = int(crit.offsets[-1]) if ragged else crit.num_experts * crit.capacity
    d = torch.zeros(nrows, M, dtype=x.dtype)
    rows = crit.rows(ragged)
    for j in range(crit.top_k):
        keep = torch.from_numpy(rows[j] >= 0)
        dst = torch.from_numpy(rows[j][rows[j] >= 0].astype(np.int64))
        d.index_add_(0, dst, x[keep])
    return d if ragged else d.view(crit.num_experts, crit.capacity, M)


def fast_encode_bwd(dd: torch.Tensor, crit: Critical, ragged: bool = False) -> torch.Tensor:
    """dx[i,:] = sum_j kept(j,i) * dD[row(j,i),:]."""
    dd2 = dd.reshape(-1, dd.shape[-1])
    rows = crit.rows(ragged)
    S = rows.shape[1]
    dx = torch.zeros(S, dd2.shape[1], dtype=dd.dtype)
    for j in range(crit.top_k):
        keep = torch.from_numpy(rows[j] >= 0)
        src = torch.from_numpy(rows[j][rows[j] >= 0].astype(np.int64))
        dx[keep] += dd2[src]
    return dx


def fast_decode(o: torch.Tensor, crit: Critical, ragged: bool = False) -> torch.Tensor:
    """GatingDecoder forward: y[i,:] = sum_j kept(j,i) * gate_j[i] * O[row(j,i),:]."""
    o2 = o.reshape(-1, o.shape[-1])
    rows = crit.rows(ragged)
    S = rows.shape[1]
    y = torch.zeros(S, o2.shape[1], dtype=o.dtype)
    for j in range(crit.top_k):
        keep = torch.from_numpy(rows[j] >= 0)
        src = torch.from_numpy(rows[j][rows[j] >= 0].astype(np.int64))
        g = torch.from_numpy(crit.gates_s[j]).to(o.dtype)[keep]
        y[keep] += g[:, None] * o2[src]
    return y


def fast_decode_bwd(dy: torch.Tensor, o: torch.Tensor, crit: Critical, ragged: bool = False):
    """dO[row(j,i),:] = gate_j[i]*dy[i,:] (zero elsewhere); dgate_j[i] = <dy[i,:], O[row(j,i),:]>
    (zero for dropped pairs).  Returns (dO shaped like o, dgates [k,S])."""
    o2 = o.reshape(-1, o.shape[-1])
    rows = crit.rows(ragged)
    k, S = rows.shape
    do = torch.zeros_like(o2)
    dg = torch.zeros(k, S, dtype=o.dtype)
    for j in range(k):
        keep = torch.from_numpy(rows[j] >= 0)
        dst = torch.from_numpy(rows[j][rows[j] >= 0].astype(np.int64))
        g = torch.from_numpy(crit.gates_s[j]).to(o.dtype)[keep]
        do[dst] = g[:, None] * dy[keep]
        dg[j, keep] = (dy[keep] * o2[dst]).sum(dim=1)
    return do.view_as(o), dg


def gate_normalize_bwd(dgates: torch.Tensor, scores: torch.Tensor, crit: Critical,
                       normalize_gate: bool = True) -> torch.Tensor:
    """Back-propagate d(loss)/d(gate_j[i]) to d(loss)/d(scores[i,e]) (dense [S,E]).

    gate_j = graw_j / max(sum_j' graw_j', eps) with graw_j = scores[i, idx_j[i]].
    """
    k, S = dgates.shape
    E = scores.shape[1]
    ar = torch.arange(S)
    idx = [torch.from_numpy(ix.astype(np.int64)) for ix in crit.indices_s]
    graw = torch.stack([scores[ar, ix] for ix in idx])                 # [k,S]
    dscores = torch.zeros(S, E, dtype=scores.dtype)
    if k > 1 and normalize_gate:
        denom = graw[0].clone()
        for j in range(1, k):
            denom = denom + graw[j]
        clamped = denom < FP32_EPS
        den = torch.clamp(denom, min=FP32_EPS)
        dot = (dgates * graw).sum(dim=0) / (den * den)                 # sum_j dgate_j*graw_j / den^2
        dot = torch.where(clamped, torch.zeros_like(dot), dot)          # clamp passes no gradient
        dgraw = dgates / den - dot
    else:
        dgraw = dgates
    for j in range(k):
        dscores[ar, idx[j]] += dgraw[j]
    return dscores


def softmax_bwd(dscores: torch.Tensor, scores: torch.Tensor) -> torch.Tensor:
    """dlogits = scores * (dscores - sum_e dscores*scores)."""
    return scores * (dscores - (dscores * scores).sum(dim=-1, keepdim=True))


# --------------------------------------------------------------------------------------------
# A9-A12  expert FFN forward / backward  (MOLE/cpp/core.cpp:344-356, 381-414, 457-491)
# --------------------------------------------------------------------------------------------
SQRT_2_OVER_PI = 0.79788456080286535587989211986876


def d_gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """Derivative of the tanh-approximate GELU, term by term as in MOLE/cpp/gelu.cu:3-14."""
    x2mul = x * x * 0.044715
    tan_h = torch.tanh(SQRT_2_OVER_PI * (x + x * x2mul))
    dg1 = 0.5 * (1.0 + tan_h)
    dg2 = x * 0.5 * SQRT_2_OVER_PI * (1 - tan_h * tan_h)
    dg3 = dg2 * 3 * x2mul
    return dg1 + dg2 + dg3


def d_gelu_exact(x: torch.Tensor) -> torch.Tensor:
    """Derivative of the erf GELU: Phi(x) + x*phi(x) (what at::gelu_backward multiplies by,
    the path taken when USE_MOLE_GELU is undefined, MOLE/cpp/core.cpp:396)."""
    cdf = 0.5 * (1.0 + torch.erf(x / math.sqrt(2.0)))
    pdf = torch.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)
    return cdf + x * pdf


def ffn_fwd(x: torch.Tensor, w1, b1, w2, b2):
    """Padded batched forward, [E,C,M] -> [E,C,M]; returns (out, x1) with x1 the saved
    pre-activation (core.cpp:350-355).  w1 [E,F,M], b1 [E,F], w2 [E,F,M] (used as x2 @ w2), b2 [E,M].
    """
    x1 = torch.baddbmm(b1.unsqueeze(1), x, w1.permute(0, 2, 1))
    x2 = F.gelu(x1)
    out = torch.baddbmm(b2.unsqueeze(1), x2, w2)
    return out, x1


def ffn_bwd(go: torch.Tensor, x, x1, w1, w2, gelu_bwd: str = "tanh", input_requires_grad: bool = True):
    """Padded batched backward (core.cpp:386-414).  gelu_bwd="tanh" is the reference's compiled
    default (define.hpp:6 defines USE_MOLE_GELU -> gelu.cu derivative); "exact" is the erf
    derivative.  Returns (g_w1, g_b1, g_w2, g_b2, x_grad)."""
    x3 = F.gelu(x1)
    g_w2 = torch.matmul(x3.permute(0, 2, 1), go)
    t = torch.matmul(go, w2.permute(0, 2, 1))
    t = t * (d_gelu_tanh(x1) if gelu_bwd == "tanh" else d_gelu_exact(x1))
    g_b2 = go.sum(dim=1)
    g_w1 = torch.matmul(t.permute(0, 2, 1), x)
    g_b1 = t.sum(dim=1)
    x_grad = torch.matmul(t, w1) if input_requires_grad else None
    return g_w1, g_b1, g_w2, g_b2, x_grad


def ffn_fwd_ragged(xd: torch.Tensor, offsets: Sequence[int], w1, b1, w2, b2):
    """Same math over expert-contiguous ragged rows: rows offsets[e]:offsets[e+1] belong to
    expert e.  Returns (out [R,M], x1 [R,F])."""
    R = xd.shape[0]
    Fdim = w1.shape[1]
    out = torch.zeros(R, w2.shape[2], dtype=xd.dtype)
    x1 = torch.zeros(R, Fdim, dtype=xd.dtype)
    for e in range(w1.shape[0]):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            h = torch.addmm(b1[e], xd[lo:hi], w1[e].t())
            x1[lo:hi] = h
            out[lo:hi] = torch.addmm(b2[e], F.gelu(h), w2[e])
    return out, x1


def ffn_bwd_ragged(go: torch.Tensor, xd, x1, offsets: Sequence[int], w1, w2, gelu_bwd: str = "tanh"):
    """Ragged backward; experts without rows get zero gradients."""
    E, Fdim, M = w1.shape
    g_w1 = torch.zeros_like(w1)
    g_w2 = torch.zeros_like(w2)
    g_b1 = torch.zeros(E, Fdim, dtype=w1.dtype)
    g_b2 = torch.zeros(E, M, dtype=w1.dtype)
    gx = torch.zeros_like(xd)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi <= lo:
            continue
        h = x1[lo:hi]
        g = go[lo:hi]
        g_w2[e] = F.gelu(h).t() @ g
        t = g @ w2[e].t()
        t = t * (d_gelu_tanh(h) if gelu_bwd == "tanh" else d_gelu_exact(h))
        g_b2[e] = g.sum(dim=0)
        g_w1[e] = t.t() @ xd[lo:hi]
        g_b1[e] = t.sum(dim=0)
        gx[lo:hi] = t @ w1[e]
    return g_w1, g_b1, g_w2, g_b2, gx


# --------------------------------------------------------------------------------------------
# whole layer, forward + backward  (MOLE/moe/layer.py:429-476 and its autograd)
# --------------------------------------------------------------------------------------------
@dataclass
class LayerResult:
    scores: torch.Tensor
    crit: Critical
    y: torch.Tensor
    dx: Optional[torch.Tensor] = None
    dwg: Optional[torch.Tensor] = None
    g_w1: Optional[torch.Tensor] = None
    g_b1: Optional[torch.Tensor] = None
    g_w2: Optional[torch.Tensor] = None
    g_b2: Optional[torch.Tensor] = None
    extras: dict = field(default_factory=dict)


def moe_layer(x, wg, w1, b1, w2, b2, top_k: int, capacity_factor: float = 1.0, dy=None,
              logit_bias=None, normalize_gate: bool = True, gelu_bwd: str = "tanh",
              scores_override=None, d_l_aux: float = 0.0) -> LayerResult:
    """One MoE layer forward (and backward when dy is given) on the ragged layout.

    The ragged layout computes exactly the kept rows; the reference's padded [E,C,M] layout gives
    the same y and the same gradients because padded rows are never read by decode and receive
    zero output gradient (tests pin that equivalence).  `scores_override` lets a test feed the
    scores produced on the GPU so that routing is compared bit for bit on identical inputs.  d_l_aux is the
    weight with which l_aux enters the loss (loss = <dy, y> + d_l_aux * l_aux): its gradient reaches dx and dwg
    through the scores.
    """
    scores = gate_scores(x, wg, logit_bias) if scores_override is None else scores_override
    crit = extract_critical(scores.detach().numpy(), top_k, capacity_factor, normalize_gate)
    xd = fast_encode(x, crit, ragged=True)
    o, x1 = ffn_fwd_ragged(xd, crit.offsets, w1, b1, w2, b2)
    y = fast_decode(o, crit, ragged=True)
    res = LayerResult(scores, crit, y, extras={"xd": xd, "o": o, "x1": x1})
    if dy is None:
        return res
    do, dgates = fast_decode_bwd(dy, o, crit, ragged=True)
    g_w1, g_b1, g_w2, g_b2, gxd = ffn_bwd_ragged(do, xd, x1, crit.offsets, w1, w2, gelu_bwd)
    dx = fast_encode_bwd(gxd, crit, ragged=True)
    dscores = gate_normalize_bwd(dgates, scores, crit, normalize_gate)
    if d_l_aux != 0.0 and x.shape[0] > 0:
        dscores = dscores + gshard_loss_bwd(x.shape[0], crit.counts[0], d_l_aux).to(dscores.dtype)
    dlogits = softmax_bwd(dscores, scores)
    dx = dx + dlogits @ wg
    res.dx, res.dwg = dx, dlogits.t() @ x
    res.g_w1, res.g_b1, res.g_w2, res.g_b2 = g_w1, g_b1, g_w2, g_b2
    res.extras.update({"do": do, "dgates": dgates, "gxd": gxd, "dlogits": dlogits})
    return res


# --------------------------------------------------------------------------------------------
# A14  slot-pool prefetch bookkeeping  (MOLE/cpp/umemory.cpp, MOLE/cpp/core.cpp)
# --------------------------------------------------------------------------------------------
class UniMemModel:
    """Integer model of _UniMem's prefetch stack (umemory.cpp:109-183).

    prefetch(layer, n)  reserves slots [virtual_offset, virtual_offset+n), merges with the top
                        stack entry when it belongs to the same layer, advances virtual_offset
                        and shrinks the visible pool (umemory.cpp:131-154).
    fetch_top(layer)    pops the top entry when it belongs to `layer`, rewinds virtual_offset and
                        returns the number of prefetched experts, else 0 (umemory.cpp:169-183).
    fetch_batch(a, b)   slots [a+virtual_offset, b+virtual_offset) (umemory.cpp:92-107).
    """

    def __init__(self, pool_size: int):
        self.pool_size = pool_size
        self.clear_virtual_mem()

    def clear_virtual_mem(self):
        self.stk: List[List[int]] = []
        self.virtual_offset = 0
        self.view_pool_size = self.pool_size

    def prefetch(self, layer: int, n: int) -> Tuple[int, int]:
        if n == 0:
            return (self.virtual_offset, self.virtual_offset)
        if self.stk and self.stk[-1][0] == layer:
            self.stk[-1][1] += n
        else:
            self.stk.append([layer, n])
        lo = self.virtual_offset
        self.virtual_offset += n
        self.view_pool_size -= n
        return (lo, lo + n)

    def fetch_top(self, layer: int) -> int:
        if self.stk and self.stk[-1][0] == layer:
            n = self.stk.pop()[1]
            self.virtual_offset -= n
            self.view_pool_size += n
            return n
        return 0

    def fetch_batch(self, start: int, end: int) -> Tuple[int, int]:
        return (start + self.virtual_offset, end + self.virtual_offset)


def plan_offloaded_chunks(d_experts: int, ebatch_size: int, use_pool: bool, view_pool_size: int,
                          prefetched: int, as_reference: bool = False):
    """Chunking of the offloaded experts of one layer into batch records and launch groups
    (core.cpp:1020-1051).  Returns a list of groups, each a list of
    (expert_base, size, already_prefetched, view_base).

    as_reference=True restates the reference literally.  It wraps view_base to 0 whenever the next chunk does not
    fit the visible pool, also while that chunk still holds prefetched experts (core.cpp:1026-1046), which then
    are looked for in slots that hold other experts - e.g. (d=6, ebatch=2, pool=5, prefetched=5) yields the chunk
    (4, 2, 1, 0): expert 4 is taken to be in slot 0, which holds expert 0.  The default cuts such a chunk at the
    end of the visible pool instead, so that prefetched experts are always used where they lie;
    simulate_chunk_slots() checks exactly that."""
    groups, cur = [], []
    d_batch = min(ebatch_size, 10000 if not use_pool else view_pool_size)
    view_base = 0
    i = 0
    while i < d_experts:
        size = min(d_batch, d_experts - i)
        if use_pool and view_pool_size - view_base < size:
            if i < prefetched and not as_reference:
                size = view_pool_size - view_base
            else:
                view_base = 0
                groups.append(cur)
                cur = []
        cur_pref = min(size, prefetched - i) if prefetched > i else 0
        cur.append((i, size, cur_pref, view_base))
        view_base += size
        i += d_batch if as_reference else size
    if cur:
        groups.append(cur)
    return groups


def simulate_chunk_slots(chunks, prefetched: int, pool_size: int) -> bool:
    """Plays a chunk plan [(expert_base, size, already_prefetched, view_base)] against the slot pool: slots
    0..prefetched-1 start out holding experts 0..prefetched-1, each chunk copies its not-yet-prefetched experts
    into its slots and then runs on what the slots hold.  True iff every chunk finds exactly its own experts."""
    slots = [None] * pool_size
    for e in range(prefetched):
        slots[e] = e
    for (base, size, pref, vb) in chunks:
        if vb < 0 or vb + size > pool_size:
            return False
        for j in range(pref, size):
            slots[vb + j] = base + j
        if any(slots[vb + j] != base + j for j in range(size)):
            return False
    return True


def fast_assign_prefetch(P: int, Fv: Sequence[int], Ev: Sequence[int]):
    """Greedy cross-layer prefetch assignment (core.cpp:1302-1345).

    P pool slots; Fv[i] experts fetchable under layer i's compute; Ev[i] offloaded experts of
    layer i.  Returns (GPscheme, LPscheme): LPscheme[i] = experts layer i prefetches for itself,
    GPscheme[i] = list of [later_layer, count] that layer i prefetches on behalf of later layers.
    """
    n = len(Ev)
    gp = [[] for _ in range(n)]
    lp = [0] * n
    stk: List[List[int]] = []
    p_cur = P
    for i in range(n):
        fetchable = min(p_cur, Fv[i])
        if fetchable <= Ev[i]:
            need = Ev[i] - fetchable
            lp[i] = fetchable
            while stk and need > 0:
                top_id, top = stk[-1]
                if top > need:
                    stk[-1][1] = top - need
                    gp[top_id].append([i, need])
                    p_cur += need
                    need = 0
                else:
                    gp[top_id].append([i, top])
                    stk.pop()
                    need -= top
                    p_cur += top
        else:
            new_gp = fetchable - Ev[i]
            p_cur -= new_gp
            stk.append([i, new_gp])
            lp[i] = Ev[i]
    return gp, lp


# ---------------------------------------------------------------------------------------------
# in-pipeline Adam (MOLE/cpp/define.hpp:543-579)
# ---------------------------------------------------------------------------------------------
def adam_step(p: torch.Tensor, m: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta1: float, beta2: float,
              t_stored: int, lr: float, lam: float, eps: float, adamW: bool, scalar=np.float32):
    """One update as _MOLECore::adam evaluates it, tensor op by tensor op, in the dtype of the inputs.
    t_stored is the counter set_adam() stored; the update uses t_stored + 1 (define.hpp:547).
    The hyper-parameters are C++ floats in the reference (define.hpp:521), so 1 - beta, lam * lr and
    1 - lam * lr are formed in single precision (scalar=np.float32); std::pow(float, int) promotes to double,
    and so does 1 - pow.  scalar=np.float64 gives the textbook double-precision constants.
    Returns (p_new, m_new, v_new); the inputs are left untouched."""
    f = scalar
    beta1, beta2, lr, lam, eps = f(beta1), f(beta2), f(lr), f(lam), f(eps)
    one = f(1)
    t = t_stored + 1
    if adamW:
        p = p * float(one - lam * lr)
    else:
        g = g + float(lam) * p
    m = float(beta1) * m + float(one - beta1) * g
    v = float(beta2) * v + float(one - beta2) * g * g
    mt = m / (1.0 - float(beta1) ** t)
    vt = v / (1.0 - float(beta2) ** t)
    p = p - float(lr) * mt / (vt.sqrt() + float(eps))
    return p, m, v
