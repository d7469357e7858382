"""Routing / dispatch / combine with the interface of tutel.impls.fast_dispatch, the third-party
module MOLE/moe/layer.py:4 imports and calls at layer.py:445-446 (extract_critical), 448-449
(fast_encode) and 457-458 (fast_decode).  Same names, same argument spelling (`critial_data`),
same return structure; every step runs in the HIP kernels behind mole_route / mole_dispatch_* /
mole_combine_* and is differentiable the way tutel's GatingEncoder / GatingDecoder are.
"""
from __future__ import annotations

import torch

from .. import _lib as L
from .. import hip_ops as H


class Critical(tuple):
    """(num_global_experts, indices_s, locations_s, gates_s, capacity) - tutel's critical data -
    carrying the device-side route (row permutation, kept rows, offsets) as `.route`."""
    route: H.Route = None


class _RouteFn(torch.autograd.Function):
    """scores [S,E] -> gates [k,S] and l_aux; differentiable through the gate normalisation and through
    l_aux = E/S^2 sum_e (sum_i scores[i,e]) counts[0,e] (tutel's gshard_loss, whose gradient the reference's
    loss reaches through autograd)."""

    @staticmethod
    def forward(ctx, scores, top_k, capacity_factor, normalize_gate, alignment, layout, holder):
        r = H.route(scores.detach().contiguous(), top_k, capacity_factor, normalize_gate, alignment, layout)
        holder.append(r)
        ctx.save_for_backward(scores, r.idx, r.counts)
        ctx.normalize_gate = normalize_gate
        ctx.mark_non_differentiable(r.idx, r.loc)
        return r.gates, r.idx, r.loc, r.l_aux.view(())

    @staticmethod
    def backward(ctx, dgates, _di, _dl, d_l_aux):
        scores, idx, counts = ctx.saved_tensors
        if dgates is None:
            dgates = torch.zeros(idx.shape, dtype=torch.float32, device=scores.device)
        aux = {} if d_l_aux is None else dict(counts0=counts[0].contiguous(), d_l_aux=d_l_aux)
        dscores = H.gate_bwd(dgates.contiguous(), scores.detach().contiguous(), idx, ctx.normalize_gate,
                             through_softmax=False, **aux)
        return dscores, None, None, None, None, None, None


def extract_critical(scores, top_k, loss_fn=None, capacity_factor=1.0, batch_prioritized_routing=False,
                     normalize_gate=True, alignment=1, group=None, inequivalent_tokens=False,
                     layout=L.LAYOUT_PADDED):
    """Returns ((E, indices_s, locations_s, gates_s, capacity), l_aux) like tutel.

    capacity_factor <= 0 makes the capacity data dependent; only then is the device read back
    (one .item()), exactly where tutel synchronises too."""
    if batch_prioritized_routing or inequivalent_tokens or group is not None:
        raise NotImplementedError("only the plain single-group routing of the MOLE layer is implemented")
    S, E = scores.shape
    k = min(int(top_k), E)
    holder = []
    gates, idx, loc, l_aux_diff = _RouteFn.apply(scores.float(), k, float(capacity_factor), bool(normalize_gate),
                                                 int(alignment), int(layout), holder)
    r = holder[0]
    if capacity_factor > 0:
        cap = k * int(capacity_factor * ((S + E - 1) // E))
        rem = cap % alignment
        cap += (alignment - rem) if rem > 0 else 0
    else:
        cap = int(r.capacity.item())
    crit = Critical((E, [idx[j] for j in range(k)], [loc[j] for j in range(k)], [gates[j] for j in range(k)], cap))
    crit.route = r
    crit.gates = gates
    l_aux = l_aux_diff if loss_fn is None else loss_fn(scores, idx.t())
    return crit, l_aux


def _route_of(crit, S):
    """Row permutation of a critical tuple; rebuilt from (indices, locations, capacity) when the
    tuple did not come from extract_critical above."""
    r = getattr(crit, "route", None)
    if r is not None and r.layout == L.LAYOUT_PADDED:
        return r.row, r.kept_rows, r.offsets
    E, indices_s, locations_s, _, cap = crit[:5]
    idx = torch.stack([t.to(torch.int32) for t in indices_s])
    loc = torch.stack([t.to(torch.int32) for t in locations_s])
    row = torch.where(loc < cap, idx * cap + loc, torch.full_like(loc, -1)).contiguous()
    kept = torch.zeros(E, dtype=torch.int32, device=idx.device)
    kept.scatter_add_(0, idx.flatten().long(), (loc < cap).flatten().to(torch.int32))
    offsets = torch.arange(E + 1, dtype=torch.int32, device=idx.device) * cap
    return row, kept, offsets


class _EncodeFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, row, kept, offsets, total_rows):
        xd = torch.empty(total_rows, x.shape[1], dtype=x.dtype, device=x.device)
        H.dispatch_fwd(x.contiguous(), row, total_rows, out=xd)
        H.zero_pad_rows(xd, kept, offsets)
        ctx.save_for_backward(row)
        return xd

    @staticmethod
    def backward(ctx, dxd):
        (row,) = ctx.saved_tensors
        return H.dispatch_bwd(dxd.contiguous(), row), None, None, None, None


class _DecodeFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, o, gates, row, kept, offsets):
        ctx.save_for_backward(o, gates, row, kept, offsets)
        return H.combine_fwd(o, row, gates.detach().float().contiguous())

    @staticmethod
    def backward(ctx, dy):
        o, gates, row, kept, offsets = ctx.saved_tensors
        d_o, dgates = H.combine_bwd(dy.contiguous(), o, row, gates.detach().float().contiguous())
        H.zero_pad_rows(d_o, kept, offsets)
        return d_o, dgates.to(gates.dtype), None, None, None


def fast_encode(data, critial_data, is_postscore=True):
    """[S, M] -> [E, C, M] zero-padded (tutel GatingEncoder, gates not applied)."""
    if not is_postscore:
        raise NotImplementedError("MOLE encodes with is_postscore=True (gates applied at decode)")
    E, cap = critial_data[0], critial_data[4]
    x = data.reshape(-1, data.shape[-1])
    row, kept, offsets = _route_of(critial_data, x.shape[0])
    xd = _EncodeFn.apply(x, row, kept, offsets, E * cap)
    return xd.view(E, cap, x.shape[1])


def fast_decode(data, critial_data, is_postscore=True):
    """[E, C, M] -> [S, M], gate-weighted sum over the k choices (tutel GatingDecoder)."""
    if not is_postscore:
        raise NotImplementedError("MOLE decodes with is_postscore=True")
    E, cap = critial_data[0], critial_data[4]
    o = data.reshape(E * cap, data.shape[-1])
    S = critial_data[1][0].shape[0]
    row, kept, offsets = _route_of(critial_data, S)
    gates = getattr(critial_data, "gates", None)
    if gates is None:
        gates = torch.stack(list(critial_data[3]))
    return _DecodeFn.apply(o.contiguous(), gates, row, kept, offsets)
