"""Pins the routing half of the oracle (extract_critical / encode / decode) against brute force,
closed forms and invariants, none of which retype the oracle's own formulas."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


def brute_topk(scores, k):
    out = []
    for row in scores:
        order = sorted(range(len(row)), key=lambda e: (-float(row[e]), e))
        out.append(order[:k])
    return np.array(out, dtype=np.int32)


def brute_locations(indices_s, E):
    """Sequential simulation: all first choices in token order, then all second choices, ..."""
    fill = [0] * E
    locs = []
    for idx in indices_s:
        loc = np.zeros(len(idx), dtype=np.int32)
        for i, e in enumerate(idx):
            loc[i] = fill[e]
            fill[e] += 1
        locs.append(loc)
    return locs


def stable_sort_locations(indices_s, E):
    """Closed form: rank inside the expert in token order via a stable sort + earlier-choice counts."""
    base = np.zeros(E, dtype=np.int64)
    locs = []
    for idx in indices_s:
        order = np.argsort(idx, kind="stable")
        sorted_e = idx[order]
        starts = np.searchsorted(sorted_e, np.arange(E), side="left")
        rank = np.empty(len(idx), dtype=np.int64)
        rank[order] = np.arange(len(idx)) - starts[sorted_e]
        locs.append((rank + base[idx]).astype(np.int32))
        base += np.bincount(idx, minlength=E)
    return locs


@pytest.mark.parametrize("S,E,k", [(1, 1, 1), (7, 3, 2), (64, 8, 2), (257, 16, 1), (100, 5, 5), (300, 64, 8)])
def test_topk_matches_brute_force(S, E, k):
    rng = np.random.default_rng(S * 131 + E)
    scores = rng.random((S, E), dtype=np.float32)
    np.testing.assert_array_equal(O.topk_lowest_index_ties(scores, k), brute_topk(scores, k))


def test_topk_exact_ties_go_to_lowest_index():
    scores = np.array([[0.25, 0.25, 0.25, 0.25],
                       [0.1, 0.4, 0.4, 0.1],
                       [0.0, 0.0, 1.0, 0.0],
                       [0.3, 0.2, 0.3, 0.2]], dtype=np.float32)
    got = O.topk_lowest_index_ties(scores, 3)
    np.testing.assert_array_equal(got, [[0, 1, 2], [1, 2, 0], [2, 0, 1], [0, 2, 1]])
    # duplicated gate columns produce bit-identical scores for whole columns
    rng = np.random.default_rng(0)
    x = torch.from_numpy(rng.standard_normal((50, 16)).astype(np.float32))
    wg = torch.from_numpy(rng.standard_normal((6, 16)).astype(np.float32))
    wg[4] = wg[1]
    s = O.gate_scores(x, wg).numpy()
    assert (s[:, 4] == s[:, 1]).all()
    t = O.topk_lowest_index_ties(s, 6)
    pos1 = np.argmax(t == 1, axis=1)
    pos4 = np.argmax(t == 4, axis=1)
    assert (pos4 == pos1 + 1).all()


def test_topk_nan_is_largest():
    scores = np.array([[0.1, np.nan, 0.7, np.nan, np.inf]], dtype=np.float32)
    np.testing.assert_array_equal(O.topk_lowest_index_ties(scores, 4), [[1, 3, 4, 2]])
    tt = torch.topk(torch.from_numpy(scores), 4, dim=1).indices.numpy()
    assert set(tt[0, :2]) == {1, 3} and tt[0, 2] == 4   # torch agrees on NaN > inf > finite


@pytest.mark.parametrize("S,E,k,cf", [(64, 8, 2, 1.0), (500, 16, 1, 1.25), (333, 7, 3, 0.0),
                                      (1000, 64, 2, 0.0), (129, 4, 2, -0.5), (2048, 256, 8, 0.0)])
def test_extract_critical_pinned(S, E, k, cf):
    rng = np.random.default_rng(7 * S + E + k)
    logits = rng.standard_normal((S, E)).astype(np.float32) + np.log(np.arange(1, E + 1, dtype=np.float32) ** -1.2)
    scores = torch.softmax(torch.from_numpy(logits), dim=-1).numpy()
    c = O.extract_critical(scores, k, cf)
    bt = brute_topk(scores, k)
    for j in range(k):
        np.testing.assert_array_equal(c.indices_s[j], bt[:, j])
        assert c.indices_s[j].dtype == np.int32 and c.locations_s[j].dtype == np.int32
    # counts: library routine
    for j in range(k):
        np.testing.assert_array_equal(c.counts[j], np.bincount(bt[:, j], minlength=E))
        assert c.counts[j].sum() == S
    # locations: sequential simulation and stable-sort closed form
    for ref in (brute_locations(c.indices_s, E), stable_sort_locations(c.indices_s, E)):
        for j in range(k):
            np.testing.assert_array_equal(c.locations_s[j], ref[j])
    # (expert, location) pairs are distinct and gap-free per expert
    pairs = np.stack([np.concatenate(c.indices_s), np.concatenate(c.locations_s)], axis=1)
    assert len(np.unique(pairs, axis=0)) == S * k
    tot = c.counts.sum(axis=0)
    for e in range(E):
        np.testing.assert_array_equal(np.sort(pairs[pairs[:, 0] == e, 1]), np.arange(tot[e]))
    # capacity closed form
    spe = -(-S // E)
    if cf > 0:
        assert c.capacity == k * int(cf * spe)
    elif cf == 0:
        assert c.capacity == tot.max()
        assert (c.rows(True) >= 0).all()       # nothing dropped
    else:
        assert c.capacity == min(tot.max(), k * int(-cf * spe))
    np.testing.assert_array_equal(c.kept_rows, np.minimum(tot, c.capacity))
    assert c.offsets[0] == 0 and c.offsets[-1] == c.kept_rows.sum()
    # gates: gather closed form, normalised to one
    g = np.stack([scores[np.arange(S), bt[:, j]] for j in range(k)])
    if k > 1:
        np.testing.assert_allclose(np.stack(c.gates_s).sum(0), 1.0, rtol=1e-6)
        np.testing.assert_allclose(np.stack(c.gates_s), g / g.sum(0, keepdims=True), rtol=1e-6)
    else:
        np.testing.assert_array_equal(c.gates_s[0], g[0])
    # dispatch permutation: kept rows are a bijection onto 0..R-1 (ragged) and inside e*C..e*C+n[e] (padded)
    rr = c.rows(True)
    kept = rr[rr >= 0]
    np.testing.assert_array_equal(np.sort(kept), np.arange(c.offsets[-1]))
    rp = c.rows(False)
    for j in range(k):
        m = rp[j] >= 0
        assert ((rp[j][m] // max(c.capacity, 1)) == c.indices_s[j][m]).all()


def test_capacity_special_cases_of_the_benchmark_configs():
    assert O.compute_capacity(16384, 16, 1, 1.25, 0) == 1280
    assert O.compute_capacity(4096, 8, 2, 1.0, 0) == 1024
    assert O.compute_capacity(10, 4, 2, 0.0, 7, alignment=4) == 8
    assert O.compute_capacity(10, 4, 1, -1.0, 7) == 3
    # the product is a Python (double precision) one: int(0.02 * 50) is 1; in single precision it would be 0
    assert O.compute_capacity(200, 4, 1, 0.02, 0) == 1
    assert O.compute_capacity(200, 4, 1, 0.001, 0) == 0


def test_capacity_drop_is_lowest_index_first_and_first_choice_first():
    S, E, k = 40, 2, 2
    scores = np.zeros((S, E), dtype=np.float32)
    scores[:, 0], scores[:, 1] = 0.9, 0.1       # everyone: first choice 0, second choice 1
    c = O.extract_critical(scores, k, 0.5)      # C = 2*int(0.5*20) = 20
    assert c.capacity == 20
    rows = c.rows(False)
    assert (rows[0][:20] >= 0).all() and (rows[0][20:] == -1).all()
    assert (rows[1][:20] >= 0).all() and (rows[1][20:] == -1).all()
    # second choices of expert 0 would come after ALL first choices of expert 0 (k-major)
    scores2 = scores.copy()
    scores2[30:, 0], scores2[30:, 1] = 0.1, 0.9
    c2 = O.extract_critical(scores2, k, 0.0)
    assert c2.locations_s[1][30] == 30          # 30 first-choice tokens of expert 0 precede it


def _dense_combine_weights(c, S, E, nrows, ragged, dtype):
    """[S, nrows] matrix W with W[i, row(j,i)] = gate_j[i]: the one-hot formulation of decode."""
    W = torch.zeros(S, nrows, dtype=dtype)
    rows = c.rows(ragged)
    for j in range(c.top_k):
        for i in range(S):
            if rows[j, i] >= 0:
                W[i, rows[j, i]] = float(c.gates_s[j][i])
    return W


@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("S,E,k,cf", [(48, 4, 2, 1.0), (37, 5, 3, 0.0), (64, 8, 1, 0.5)])
def test_encode_decode_against_dense_one_hot_and_autograd(S, E, k, cf, ragged):
    torch.manual_seed(S + E)
    M = 6
    scores = torch.softmax(torch.randn(S, E), dim=-1).numpy()
    c = O.extract_critical(scores, k, cf)
    nrows = int(c.offsets[-1]) if ragged else E * c.capacity
    x = torch.randn(S, M, dtype=torch.float64)
    W = _dense_combine_weights(c, S, E, nrows, ragged, torch.float64)
    P = (W != 0).to(torch.float64)             # dispatch one-hot [S, nrows]
    d = O.fast_encode(x, c, ragged).reshape(nrows, M)
    torch.testing.assert_close(d, P.t() @ x)
    o = torch.randn(nrows, M, dtype=torch.float64)
    y = O.fast_decode(o, c, ragged)
    torch.testing.assert_close(y, W @ o)
    # backward of decode from autograd of the dense formulation
    Wp = W.clone().requires_grad_(True)
    op = o.clone().requires_grad_(True)
    dy = torch.randn(S, M, dtype=torch.float64)
    ((Wp @ op) * dy).sum().backward()
    do, dg = O.fast_decode_bwd(dy, o, c, ragged)
    torch.testing.assert_close(do, op.grad)
    rows = c.rows(ragged)
    for j in range(k):
        for i in range(S):
            want = Wp.grad[i, rows[j, i]] if rows[j, i] >= 0 else 0.0
            assert abs(float(dg[j, i]) - float(want)) < 1e-12
    # adjointness pins encode backward: <encode(x), D'> == <x, encode_bwd(D')>
    dd = torch.randn(nrows, M, dtype=torch.float64)
    lhs = (d * dd).sum()
    rhs = (x * O.fast_encode_bwd(dd, c, ragged)).sum()
    torch.testing.assert_close(lhs, rhs)
    # decode(encode(x)) with unit gates = (#kept choices) * x
    c1 = O.extract_critical(scores, k, cf, normalize_gate=False)
    c1.gates_s = [np.ones_like(g) for g in c1.gates_s]
    kept = (c1.rows(ragged) >= 0).sum(0)
    torch.testing.assert_close(O.fast_decode(O.fast_encode(x, c1, ragged), c1, ragged),
                               torch.from_numpy(kept).to(torch.float64)[:, None] * x)


def test_gate_normalize_and_softmax_backward_against_autograd():
    torch.manual_seed(3)
    S, E, k = 33, 6, 3
    logits = torch.randn(S, E, dtype=torch.float64, requires_grad=True)
    scores = torch.softmax(logits, dim=-1)
    c = O.extract_critical(scores.detach().numpy(), k, 0.0)
    idx = torch.from_numpy(np.stack(c.indices_s).astype(np.int64))       # [k,S]
    graw = scores.gather(1, idx.t()).t()                                  # [k,S]
    gates = graw / torch.clamp(graw.sum(0, keepdim=True), min=O.FP32_EPS)
    dg = torch.randn(k, S, dtype=torch.float64)
    (gates * dg).sum().backward()
    ds = O.gate_normalize_bwd(dg, scores.detach(), c)
    torch.testing.assert_close(O.softmax_bwd(ds, scores.detach()), logits.grad)


def test_l_aux_closed_form():
    S, E = 12, 3
    scores = np.full((S, E), 1.0 / E, dtype=np.float32)
    idx = np.array([0] * 6 + [1] * 4 + [2] * 2)
    # me = S/E for every e, sum_e ce = S  ->  l_aux = E/S^2 * (S/E) * S = 1
    assert abs(O.gshard_loss(scores, idx) - 1.0) < 1e-6


def test_empty_and_single_expert_inputs():
    c = O.extract_critical(np.zeros((0, 4), np.float32), 2, 1.0)
    assert c.capacity == 0 and c.offsets[-1] == 0
    c = O.extract_critical(np.ones((5, 1), np.float32), 2, 0.0)   # k clipped to E
    assert c.top_k == 1 and c.capacity == 5
    np.testing.assert_array_equal(c.locations_s[0], np.arange(5))
