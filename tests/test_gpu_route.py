"""HIP routing (mole_route, mole_softmax_fwd, mole_gate_bwd) against the CPU oracle, through the C ABI.
Integer outputs are compared bit for bit; gates too (same fp32 operations in the same order)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import crit_to_numpy, rel_err, zipf_scores

pytestmark = pytest.mark.gpu


def _compare(scores, k, cf, layout_ragged, normalize=True, alignment=1):
    from mole_amd import hip_ops as H, _lib as L
    r = H.route(scores.cuda(), k, cf, normalize, alignment, L.LAYOUT_RAGGED if layout_ragged else L.LAYOUT_PADDED)
    got = crit_to_numpy(r)
    c = O.extract_critical(scores.numpy(), k, cf, normalize, alignment)
    kk = c.top_k
    np.testing.assert_array_equal(got["idx"], np.stack(c.indices_s))
    np.testing.assert_array_equal(got["counts"], c.counts)
    np.testing.assert_array_equal(got["loc"], np.stack(c.locations_s))
    assert got["capacity"] == c.capacity
    np.testing.assert_array_equal(got["kept"], c.kept_rows)
    want_off = c.offsets if layout_ragged else np.arange(c.num_experts + 1, dtype=np.int32) * c.capacity
    np.testing.assert_array_equal(got["offsets"], want_off)
    np.testing.assert_array_equal(got["row"], c.rows(layout_ragged))
    np.testing.assert_array_equal(got["gates"], np.stack(c.gates_s))
    assert abs(got["l_aux"] - c.l_aux) <= 1e-5 * max(1.0, abs(c.l_aux))
    assert kk == r.k


@pytest.mark.parametrize("S,E,k,cf", [
    (1, 1, 1, 1.0), (5, 3, 2, 0.0), (255, 8, 2, 1.0), (256, 8, 2, 1.0), (257, 8, 2, 0.5),
    (1000, 16, 1, 1.25), (777, 5, 5, 0.0), (4096, 64, 2, 0.0), (3000, 100, 4, -0.5),
    (2048, 256, 8, 0.0), (600, 1024, 16, 0.0), (4096, 8, 2, 1.0),
    (200, 4, 1, 0.02),      # 0.02 * 50 is 1 in double precision and 0.99999998 in single: the capacity must be 1
])
@pytest.mark.parametrize("ragged", [True, False])
def test_route_matches_oracle(S, E, k, cf, ragged):
    print(f"route S={S} E={E} k={k} cf={cf} ragged={ragged}", flush=True)
    _compare(zipf_scores(S, E, seed=S + E + k), k, cf, ragged)


def test_route_ties_nan_alignment_and_unnormalised():
    print("route ties", flush=True)
    _compare(zipf_scores(1500, 16, seed=3, ties=True), 4, 0.0, True)
    _compare(torch.full((700, 32), 1.0 / 32), 3, 1.0, False)            # every score equal
    s = zipf_scores(300, 8, seed=9)
    s[5, 3] = float("nan"); s[17, :] = float("nan"); s[40, 0] = float("inf")
    from mole_amd import hip_ops as H
    r = H.route(s.cuda(), 2, 0.0)
    c = O.extract_critical(s.numpy(), 2, 0.0)
    np.testing.assert_array_equal(r.idx.cpu().numpy(), np.stack(c.indices_s))
    np.testing.assert_array_equal(r.loc.cpu().numpy(), np.stack(c.locations_s))
    _compare(zipf_scores(900, 8, seed=4), 2, 0.0, True, normalize=False)
    _compare(zipf_scores(900, 8, seed=5), 2, 0.0, False, alignment=64)


@pytest.mark.parametrize("name,S,E,k,cf", [("c2", 16384, 16, 1, 1.25), ("c3", 8192, 64, 2, 0.0),
                                           ("c5", 32768, 256, 8, 0.0)])
def test_route_full_size_configs(name, S, E, k, cf):
    print(f"route full {name}", flush=True)
    _compare(zipf_scores(S, E, seed=1), k, cf, True)


@pytest.mark.parametrize("S,E", [(100, 8), (513, 16), (64, 100), (300, 256)])
def test_softmax_and_gate_bwd(S, E):
    from mole_amd import hip_ops as H
    print(f"softmax/gate_bwd S={S} E={E}", flush=True)
    g = torch.Generator().manual_seed(S)
    logits = torch.randn(S, E, generator=g) * 3
    bias = torch.randn(E, generator=g)
    sc = H.softmax_fwd(logits.cuda(), bias.cuda())
    want = torch.softmax(logits + bias, dim=-1)
    assert rel_err(sc, want) < 1e-6
    assert rel_err(H.softmax_fwd(logits.cuda()), torch.softmax(logits, dim=-1)) < 1e-6
    for k, norm in [(1, True), (min(3, E), True), (min(3, E), False)]:
        scores = sc.cpu()
        c = O.extract_critical(scores.numpy(), k, 0.0, norm)
        dg = torch.randn(c.top_k, S, generator=g)
        want_dl = O.softmax_bwd(O.gate_normalize_bwd(dg, scores, c, norm), scores)
        idx = torch.from_numpy(np.stack(c.indices_s)).cuda()
        got = H.gate_bwd(dg.cuda(), sc, idx, norm)
        assert rel_err(got, want_dl) < 1e-5
        # the load-balancing loss rides along: d l_aux / d scores = E/S^2 counts0[e] on every token
        w = 0.37 * (k + 1)
        extra = O.gshard_loss_bwd(S, c.counts[0], w).float()
        want_aux = O.softmax_bwd(O.gate_normalize_bwd(dg, scores, c, norm) + extra, scores)
        counts0 = torch.from_numpy(c.counts[0].astype(np.int32)).cuda()
        got = H.gate_bwd(dg.cuda(), sc, idx, norm, counts0=counts0, d_l_aux=torch.tensor([w], device="cuda"))
        assert rel_err(got, want_aux) < 1e-5
        got = H.gate_bwd(dg.cuda(), sc, idx, norm, through_softmax=False, counts0=counts0,
                         d_l_aux=torch.tensor([w], device="cuda"))
        assert rel_err(got, O.gate_normalize_bwd(dg, scores, c, norm) + extra) < 1e-5
    # the softmax's backward as its own entry point
    ds = torch.randn(S, E, generator=g)
    assert rel_err(H.softmax_bwd(ds.cuda(), sc), O.softmax_bwd(ds, sc.cpu())) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,E,M", [(1, 1, 4), (100, 8, 64), (1000, 16, 1024), (333, 32, 520), (70, 5, 2048),
                                   (16384, 16, 1024), (700, 64, 192), (4100, 256, 2048), (129, 100, 320)])
def test_gate_wgrad(S, E, M, dtype):
    from mole_amd import hip_ops as H
    print(f"gate_wgrad S={S} E={E} M={M} {dtype}", flush=True)
    g = torch.Generator().manual_seed(S + E)
    dl = torch.randn(S, E, generator=g) * 0.1
    x = torch.randn(S, M, generator=g).to(dtype)
    got = H.gate_wgrad(dl.cuda(), x.cuda())
    want = dl.double().t() @ x.double()
    # fp32 sums of exact products (VALU kernel) or of products with dlogits split into two bf16 parts (matrix
    # cores, bf16 tokens); fp32 tokens with a large gate take the transposed product of the grouped-GEMM tiles
    assert got.shape == (E, M)
    assert rel_err(got, want) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,Mo,N", [(1, 4, 8), (300, 64, 192), (1000, 8, 520), (129, 128, 256), (0, 8, 16)])
def test_gemm_tn_and_gate_input_grad(rows, Mo, N, dtype):
    """c = a^T . b on the grouped-GEMM tiles (the gate weight gradient of shapes its own kernels do not take) and
    the gate's input gradient dlogits . Wg with E padded to the tile granule."""
    from mole_amd import hip_ops as H
    print(f"gemm_tn rows={rows} Mo={Mo} N={N} {dtype}", flush=True)
    g = torch.Generator().manual_seed(rows + Mo)
    ep = 8 if dtype == torch.bfloat16 else 4
    Mo = (Mo + ep - 1) // ep * ep
    a = torch.randn(rows, Mo, generator=g).to(dtype)
    b = torch.randn(rows, N, generator=g).to(dtype)
    got = H.gemm_tn(a.cuda(), b.cuda())
    want = a.double().t() @ b.double()
    t = 1e-5 if dtype == torch.float32 else 1e-2
    if rows == 0:
        assert float(got.abs().max()) == 0.0
        return
    assert rel_err(got, want) < t
    for E in (3, 8, 37):
        dl = torch.randn(rows, E, generator=g) * 0.1
        wg = torch.randn(E, N, generator=g) * 0.05
        got = H.gate_input_grad(dl.cuda(), wg.cuda(), dtype)
        want = dl.to(dtype).double() @ wg.to(dtype).double()
        assert got.shape == (rows, N) and got.dtype == dtype
        assert rel_err(got, want) < t


@pytest.mark.parametrize("S,E,M,bias", [(100, 16, 128, False), (1000, 8, 256, True), (513, 64, 384, False),
                                        (300, 256, 1024, True), (64, 100, 128, True), (16384, 16, 1024, False),
                                        (333, 12, 1280, True), (47, 16, 640, False)])
def test_fused_gate_forward(S, E, M, bias):
    """mole_gate_fwd (bf16 tokens) against the oracle's gate on the same rounded operands, and against the
    unfused GEMM + softmax path it replaces."""
    from mole_amd import hip_ops as H
    print(f"gate_fwd S={S} E={E} M={M} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(S + E)
    x = torch.randn(S, M, generator=g).bfloat16()
    wg = torch.randn(E, M, generator=g) * 0.05
    b = torch.log(torch.arange(1, E + 1, dtype=torch.float32) ** -1.2) if bias else None
    got = H.gate_fwd(x.cuda(), wg.cuda(), b.cuda() if bias else None, fused=True).cpu()
    want = O.gate_scores(x.float(), wg.bfloat16().float(), b)
    assert got.shape == (S, E)
    assert rel_err(got, want) < 1e-4
    assert float((got.sum(-1) - 1).abs().max()) < 1e-5
    unfused = H.softmax_fwd(H.gemm_nt(x.cuda(), wg.bfloat16().cuda()), b.cuda() if bias else None).cpu()
    assert rel_err(got, unfused) < 1e-5


@pytest.mark.parametrize("S,E,M,bias", [(4096, 8, 512, False), (777, 3, 260, True), (1000, 32, 1024, True),
                                        (5, 17, 4, False), (300, 16, 2048, False)])
def test_fused_gate_forward_fp32_tokens(S, E, M, bias):
    """mole_gate_fwd for fp32 tokens and small gates (one wave per token, fp32 FMAs) against the oracle's gate and
    against the GEMM + softmax path it replaces."""
    from mole_amd import hip_ops as H
    print(f"gate_fwd fp32 S={S} E={E} M={M} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(S + E)
    x = torch.randn(S, M, generator=g)
    wg = torch.randn(E, M, generator=g) * 0.05
    b = torch.log(torch.arange(1, E + 1, dtype=torch.float32) ** -1.2) if bias else None
    got = H.gate_fwd(x.cuda(), wg.cuda(), b.cuda() if bias else None).cpu()          # the fused kernel by default
    assert got.shape == (S, E)
    assert rel_err(got, O.gate_scores(x, wg, b)) < 1e-5
    assert float((got.sum(-1) - 1).abs().max()) < 1e-5
    unfused = H.gate_fwd(x.cuda(), wg.cuda(), b.cuda() if bias else None, fused=False).cpu()
    assert rel_err(got, unfused) < 1e-5


def test_route_random_sweep():
    """Sixty seeded random (S, E, k, capacity factor, alignment) combinations, both layouts, bit for bit."""
    rng = np.random.default_rng(2024)
    cfs = [0.0, 0.01, 0.02, 0.05, 0.1, 0.3, 0.5, 0.7, 1.0, 1.25, 2.0, 3.3, -0.3, -1.0]
    for case in range(60):
        E = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 17, 32, 60, 64, 128]))
        k = int(rng.integers(1, min(E, 8) + 1))
        S = int(rng.integers(1, 1500))
        cf = float(rng.choice(cfs))
        align = int(rng.choice([1, 1, 1, 2, 8]))
        print(f"route sweep {case}: S={S} E={E} k={k} cf={cf} align={align}", flush=True)
        _compare(zipf_scores(S, E, seed=case, ties=(case % 5 == 0)), k, cf, bool(case % 2), normalize=bool(case % 3), alignment=align)


@pytest.mark.parametrize("S,E,M,k,cf,bias,normalize,ragged", [
    (16384, 16, 1024, 1, 1.25, False, True, True), (1000, 8, 256, 2, 1.0, True, True, True),
    (33, 20, 128, 2, 0.0, False, True, False), (777, 32, 384, 4, 0.5, True, False, True),
    (64, 3, 128, 3, 1.0, False, True, True), (1, 5, 128, 1, 1.0, False, True, True),
    (4095, 17, 256, 5, -0.5, True, True, False), (8192, 32, 2048, 2, 0.0, False, True, True),
    (8192, 64, 2048, 2, 1.0, False, True, True), (16500, 48, 1024, 3, 1.25, True, True, True), (301, 33, 128, 8, 0.5, True, False, False),
])
def test_gate_and_route_in_one_call(S, E, M, k, cf, bias, normalize, ragged):
    """mole_gate_route (the gate kernel does the routing's first stage on the scores it has just formed) against
    mole_gate_fwd followed by mole_route: the same scores and the same routing, bit for bit; l_aux, whose column sums
    are taken over blocks of 32 instead of 64 tokens, to fp32 rounding.  The two-call path is the one compared with the
    oracle above; duplicated Wg rows make exact ties in every token's scores."""
    from mole_amd import hip_ops as H, _lib as L
    print(f"gate_route S={S} E={E} M={M} k={k} cf={cf} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(S * 7 + E)
    x = torch.randn(S, M, generator=g).bfloat16().cuda()
    wg = torch.randn(E, M, generator=g) * 0.05
    if E >= 4:
        wg[E - 1] = wg[0]                      # exact ties: the lower index must win in both paths
    wg = wg.cuda()
    lb = (torch.randn(E, generator=g) * 0.5).cuda() if bias else None
    if bias and E >= 4:
        lb[E - 1] = lb[0]
    layout = L.LAYOUT_RAGGED if ragged else L.LAYOUT_PADDED
    assert H.gate_route_fused(x, wg)
    scores, r = H.gate_route(x, wg, lb, k, cf, normalize, 1, layout)
    scores2 = H.gate_fwd(x, wg, lb)
    r2 = H.route(scores2, k, cf, normalize, 1, layout)
    assert torch.equal(scores, scores2)
    a, b = crit_to_numpy(r), crit_to_numpy(r2)
    for name in ("idx", "loc", "gates", "row", "counts", "kept", "offsets"):
        np.testing.assert_array_equal(a[name], b[name], err_msg=name)
    assert a["capacity"] == b["capacity"]
    assert abs(a["l_aux"] - b["l_aux"]) <= 1e-5 * max(1.0, abs(b["l_aux"]))
