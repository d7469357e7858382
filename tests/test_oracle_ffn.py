"""Pins the FFN / GELU / whole-layer / prefetch parts of the oracle against torch autograd,
fp64 closed forms and brute force."""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def test_d_gelu_tanh_is_autograd_of_tanh_gelu_and_spot_values():
    x = torch.linspace(-6, 6, 4001, dtype=torch.float64, requires_grad=True)
    F.gelu(x, approximate="tanh").sum().backward()
    torch.testing.assert_close(O.d_gelu_tanh(x.detach()), x.grad, rtol=1e-12, atol=1e-12)
    assert float(O.d_gelu_tanh(torch.tensor(0.0))) == 0.5
    assert abs(float(O.d_gelu_tanh(torch.tensor(10.0, dtype=torch.float64))) - 1.0) < 1e-12
    assert abs(float(O.d_gelu_tanh(torch.tensor(-10.0, dtype=torch.float64)))) < 1e-12


def test_d_gelu_exact_is_autograd_of_erf_gelu():
    x = torch.linspace(-6, 6, 4001, dtype=torch.float64, requires_grad=True)
    F.gelu(x).sum().backward()
    torch.testing.assert_close(O.d_gelu_exact(x.detach()), x.grad, rtol=1e-12, atol=1e-12)
    # the two derivatives differ by more than the fp32 tolerance: the switch matters
    d = (O.d_gelu_exact(x.detach()) - O.d_gelu_tanh(x.detach())).abs().max()
    assert 1e-4 < float(d) < 5e-3


def _rand_ffn(E, C, M, Fd, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=dtype)
    return r(E, C, M), r(E, Fd, M) * 0.1, r(E, Fd) * 0.1, r(E, Fd, M) * 0.1, r(E, M) * 0.1, r(E, C, M)


def test_ffn_fwd_matches_per_expert_linear_layers():
    x, w1, b1, w2, b2, _ = _rand_ffn(3, 5, 8, 12)
    out, x1 = O.ffn_fwd(x, w1, b1, w2, b2)
    for e in range(3):
        h = F.linear(x[e], w1[e], b1[e])
        torch.testing.assert_close(x1[e], h)
        torch.testing.assert_close(out[e], F.linear(F.gelu(h), w2[e].t(), b2[e]))


def test_ffn_bwd_exact_matches_autograd_and_tanh_variant_differs_only_by_the_derivative():
    x, w1, b1, w2, b2, go = _rand_ffn(3, 5, 8, 12)
    leaves = [t.clone().requires_grad_(True) for t in (x, w1, b1, w2, b2)]
    out, x1 = O.ffn_fwd(*leaves)
    (out * go).sum().backward()
    g_w1, g_b1, g_w2, g_b2, gx = O.ffn_bwd(go, x, x1.detach(), w1, w2, gelu_bwd="exact")
    for got, leaf in zip((gx, g_w1, g_b1, g_w2, g_b2), leaves):
        torch.testing.assert_close(got, leaf.grad, rtol=1e-10, atol=1e-10)
    # tanh variant == autograd of a layer whose activation has erf forward and tanh-GELU backward
    class MixedGelu(torch.autograd.Function):
        @staticmethod
        def forward(ctx, h):
            ctx.save_for_backward(h)
            return F.gelu(h)
        @staticmethod
        def backward(ctx, g):
            (h,) = ctx.saved_tensors
            with torch.enable_grad():
                hh = h.detach().requires_grad_(True)
                F.gelu(hh, approximate="tanh").backward(g)
            return hh.grad
    leaves = [t.clone().requires_grad_(True) for t in (x, w1, b1, w2, b2)]
    h = torch.baddbmm(leaves[2].unsqueeze(1), leaves[0], leaves[1].permute(0, 2, 1))
    out2 = torch.baddbmm(leaves[4].unsqueeze(1), MixedGelu.apply(h), leaves[3])
    (out2 * go).sum().backward()
    got = O.ffn_bwd(go, x, x1.detach(), w1, w2, gelu_bwd="tanh")
    for g, leaf in zip((got[4], got[0], got[1], got[2], got[3]), leaves):
        torch.testing.assert_close(g, leaf.grad, rtol=1e-10, atol=1e-10)


def test_ragged_ffn_equals_padded_ffn_on_kept_rows():
    E, C, M, Fd = 4, 6, 8, 10
    x, w1, b1, w2, b2, go = _rand_ffn(E, C, M, Fd, seed=2)
    n = [6, 0, 3, 1]
    off = np.concatenate([[0], np.cumsum(n)])
    xd = torch.cat([x[e, :n[e]] for e in range(E)])
    god = torch.cat([go[e, :n[e]] for e in range(E)])
    out_p, x1_p = O.ffn_fwd(x, w1, b1, w2, b2)
    out_r, x1_r = O.ffn_fwd_ragged(xd, off, w1, b1, w2, b2)
    torch.testing.assert_close(out_r, torch.cat([out_p[e, :n[e]] for e in range(E)]))
    # padded backward with zero grad on the padded rows == ragged backward
    gop = go.clone()
    for e in range(E):
        gop[e, n[e]:] = 0
    xp = x.clone()
    ref = O.ffn_bwd(gop, xp, x1_p, w1, w2, "tanh")
    got = O.ffn_bwd_ragged(god, xd, x1_r, off, w1, w2, "tanh")
    for a, b in zip(got[:4], ref[:4]):
        torch.testing.assert_close(a, b, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(got[4], torch.cat([ref[4][e, :n[e]] for e in range(E)]), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("k,cf", [(1, 1.25), (2, 1.0), (2, 0.0), (3, 0.0)])
def test_whole_layer_against_dense_autograd(k, cf):
    """The explicit forward/backward of the oracle layer == torch autograd through a dense
    formulation (one-hot dispatch/combine matrices held constant, gates differentiable)."""
    torch.manual_seed(11 + k)
    S, M, E, Fd = 40, 8, 5, 12
    dt = torch.float64
    x = torch.randn(S, M, dtype=dt)
    wg = torch.randn(E, M, dtype=dt) * 0.5
    w1, b1 = torch.randn(E, Fd, M, dtype=dt) * 0.2, torch.randn(E, Fd, dtype=dt) * 0.1
    w2, b2 = torch.randn(E, Fd, M, dtype=dt) * 0.2, torch.randn(E, M, dtype=dt) * 0.1
    dy = torch.randn(S, M, dtype=dt)
    aux_w = 0.7 * k                      # the load-balancing loss enters the loss with this weight
    res = O.moe_layer(x, wg, w1, b1, w2, b2, k, cf, dy=dy, gelu_bwd="exact", d_l_aux=aux_w)
    crit = res.crit
    # dense autograd version
    leaves = [t.clone().requires_grad_(True) for t in (x, wg, w1, b1, w2, b2)]
    xq, wgq, w1q, b1q, w2q, b2q = leaves
    scores = torch.softmax(xq @ wgq.t(), dim=-1)
    idx = torch.from_numpy(np.stack(crit.indices_s).astype(np.int64))
    graw = scores.gather(1, idx.t()).t()
    gates = graw / torch.clamp(graw.sum(0, keepdim=True), min=O.FP32_EPS) if k > 1 else graw
    rows = crit.rows(True)
    y = torch.zeros(S, M, dtype=dt)
    for j in range(k):
        for i in range(S):
            if rows[j, i] < 0:
                continue
            e = int(crit.indices_s[j][i])
            h = F.linear(xq[i], w1q[e], b1q[e])
            y = y + F.one_hot(torch.tensor(i), S).to(dt)[:, None] * (gates[j, i] * (F.gelu(h) @ w2q[e] + b2q[e]))[None, :]
    # gates pass through fp32 inside extract_critical (as in the reference), hence 1e-6
    torch.testing.assert_close(res.y, y.detach(), rtol=1e-6, atol=1e-7)
    # l_aux by its definition (mean score per expert times the fraction of first choices, times E), differentiable
    # in the scores only: autograd through it pins gshard_loss_bwd, a term the layer's own loss does not exercise
    frac = torch.bincount(idx[0], minlength=E).to(dt) / S
    l_aux = E * (scores.mean(dim=0) * frac).sum()
    assert abs(float(l_aux.detach()) - crit.l_aux) < 1e-6
    ((y * dy).sum() + aux_w * l_aux).backward()
    for got, leaf in zip((res.dx, res.dwg, res.g_w1, res.g_b1, res.g_w2, res.g_b2), leaves):
        torch.testing.assert_close(got, leaf.grad, rtol=1e-5, atol=1e-6)


def test_padded_reference_layout_gives_the_same_layer_output():
    torch.manual_seed(5)
    S, M, E, Fd, k = 64, 8, 4, 16, 2
    x, wg = torch.randn(S, M), torch.randn(E, M)
    w1, b1, w2, b2 = torch.randn(E, Fd, M) * .2, torch.randn(E, Fd) * .1, torch.randn(E, Fd, M) * .2, torch.randn(E, M) * .1
    res = O.moe_layer(x, wg, w1, b1, w2, b2, k, 1.0)
    d = O.fast_encode(x, res.crit, ragged=False)
    out, _ = O.ffn_fwd(d, w1, b1, w2, b2)
    y = O.fast_decode(out, res.crit, ragged=False)
    torch.testing.assert_close(y, res.y, rtol=1e-5, atol=1e-6)


# ---- prefetch bookkeeping ------------------------------------------------------------------
def test_unimem_stack_model():
    m = O.UniMemModel(8)
    assert m.prefetch(0, 3) == (0, 3)
    assert m.prefetch(0, 2) == (3, 5)            # same layer merges
    assert m.prefetch(1, 2) == (5, 7)
    assert m.view_pool_size == 1 and m.virtual_offset == 7
    assert m.fetch_top(0) == 0                    # layer 0 is not on top
    assert m.fetch_top(1) == 2 and m.virtual_offset == 5
    assert m.fetch_batch(0, 2) == (5, 7)          # popped layer's slots line up with its prefetch
    assert m.fetch_top(0) == 5 and m.virtual_offset == 0 and m.view_pool_size == 8
    assert m.fetch_top(0) == 0


def test_chunk_plan_covers_every_expert_once_and_respects_the_pool():
    for d, eb, pool, pref in itertools.product([0, 1, 5, 8], [1, 2, 4], [1, 3, 8], [0, 1, 3]):
        pref = min(pref, d, pool)
        groups = O.plan_offloaded_chunks(d, eb, True, pool, pref)
        seen = []
        for g in groups:
            used = 0
            for (base, size, p, vb) in g:
                assert vb == used and vb + size <= pool
                used += size
                seen += list(range(base, base + size))
                assert p == max(0, min(size, pref - base))
        assert seen == list(range(d))


def test_chunk_plans_use_prefetched_experts_where_they_lie():
    """Brute force over (experts, batch, pool, prefetched): played against a model of the slots, every chunk of
    the oracle's plan and of the product's plan finds its own experts in its slots; the literal reference plan
    does not (two hand-checked cases), which is why neither follows it there."""
    from mole_amd import core
    bad_ref = 0
    for d, eb, pool in itertools.product(range(0, 9), range(1, 6), range(1, 8)):
        for pref in range(0, min(d, pool) + 1):
            flat = [c for g in O.plan_offloaded_chunks(d, eb, True, pool, pref) for c in g]
            assert O.simulate_chunk_slots(flat, pref, pool), (d, eb, pool, pref, flat)
            assert [e for (b, n, _, _) in flat for e in range(b, b + n)] == list(range(d))
            mine = core.plan_chunks(d, pref, pool, eb)
            assert O.simulate_chunk_slots(mine, pref, pool), (d, eb, pool, pref, mine)
            assert [e for (b, n, _, _) in mine for e in range(b, b + n)] == list(range(d))
            for (b, n, p, vb) in mine:
                assert n <= min(eb, pool) and (p == 0 or vb == b)
            ref = [c for g in O.plan_offloaded_chunks(d, eb, True, pool, pref, as_reference=True) for c in g]
            bad_ref += not O.simulate_chunk_slots(ref, pref, pool)
    assert bad_ref > 0
    ref = [c for g in O.plan_offloaded_chunks(6, 2, True, 5, 5, as_reference=True) for c in g]
    assert (4, 2, 1, 0) in ref and not O.simulate_chunk_slots(ref, 5, 5)
    ref = [c for g in O.plan_offloaded_chunks(6, 3, True, 4, 4, as_reference=True) for c in g]
    assert (3, 3, 1, 0) in ref and not O.simulate_chunk_slots(ref, 4, 4)
    assert core.plan_chunks(6, 5, 5, 2) == [(0, 2, 2, 0), (2, 2, 2, 2), (4, 1, 1, 4), (5, 1, 0, 0)]
    with pytest.raises(RuntimeError):
        core.plan_chunks(3, 0, 0, 2)


def _brute_assign_ok(P, Fv, Ev, gp, lp):
    """Check the schedule invariants instead of retyping the greedy: pool never over-committed,
    nobody prefetches more than its layer time allows, nothing beyond a layer's expert count."""
    n = len(Ev)
    got = list(lp)
    for i in range(n):
        for (tgt, cnt) in gp[i]:
            assert tgt > i and cnt > 0
            got[tgt] += cnt
    for i in range(n):
        assert got[i] <= Ev[i]
        assert lp[i] + sum(c for _, c in gp[i]) <= Fv[i]
    # pool occupancy: an entry prefetched at layer i for layer t lives from i until t runs
    for t in range(n):
        live = lp[t] + sum(c for i in range(t) for (tt, c) in gp[i] if tt >= t)
        assert live <= P


def test_fast_assign_prefetch_invariants_and_special_cases():
    rng = np.random.default_rng(0)
    for _ in range(300):
        n = int(rng.integers(1, 7))
        P = int(rng.integers(1, 10))
        Fv = [int(v) for v in rng.integers(0, 10, n)]
        Ev = [int(v) for v in rng.integers(0, 8, n)]
        gp, lp = O.fast_assign_prefetch(P, Fv, Ev)
        _brute_assign_ok(P, Fv, Ev, gp, lp)
    # no slack anywhere -> purely local prefetch
    gp, lp = O.fast_assign_prefetch(4, [2, 2, 2], [3, 3, 3])
    assert lp == [2, 2, 2] and gp == [[], [], []]
    # layer 0 has slack 3, layer 1 can only fetch 1 of its 4 -> layer 0 fetches 3 for layer 1
    gp, lp = O.fast_assign_prefetch(8, [5, 1], [2, 4])
    assert lp == [2, 1] and gp[0] == [[1, 3]]
