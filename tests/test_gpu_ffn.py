"""HIP grouped expert FFN forward/backward (MFMA kernels) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import rel_err, tol

pytestmark = pytest.mark.gpu


def _make(E, M, Fd, rows_per_expert, dtype, seed=0, pad_between=0):
    g = torch.Generator().manual_seed(seed)
    n = np.array(rows_per_expert, dtype=np.int32)
    off = np.zeros(E + 1, dtype=np.int32)
    off[1:] = np.cumsum(n + pad_between)
    R = int(off[-1])
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).to(dtype)
    d = dict(xd=r(max(R, 1), M), w1=r(E, Fd, M, sc=0.05), b1=r(E, Fd, sc=0.05), w2=r(E, Fd, M, sc=0.05),
             b2=r(E, M, sc=0.05), go=r(max(R, 1), M), n=n, off=off, R=R)
    return d


def _oracle_fwd_bwd(d, gelu_bwd):
    """fp32 oracle on the same (rounded) inputs, per expert over its kept rows only."""
    f = {k: (v.float() if torch.is_tensor(v) else v) for k, v in d.items()}
    E = f["w1"].shape[0]
    R, M, Fd = d["R"], f["w1"].shape[2], f["w1"].shape[1]
    out = torch.zeros(max(R, 1), M); h = torch.zeros(max(R, 1), Fd)
    gx = torch.zeros(max(R, 1), M)
    g_w1 = torch.zeros_like(f["w1"]); g_w2 = torch.zeros_like(f["w2"])
    g_b1 = torch.zeros(E, Fd); g_b2 = torch.zeros(E, M)
    for e in range(E):
        lo, hi = int(d["off"][e]), int(d["off"][e]) + int(d["n"][e])
        if hi <= lo:
            continue
        o_e, h_e = O.ffn_fwd(f["xd"][lo:hi][None], f["w1"][e:e + 1], f["b1"][e:e + 1], f["w2"][e:e + 1], f["b2"][e:e + 1])
        out[lo:hi], h[lo:hi] = o_e[0], h_e[0]
        a, b, c_, dd, ee = O.ffn_bwd(f["go"][lo:hi][None], f["xd"][lo:hi][None], h_e, f["w1"][e:e + 1], f["w2"][e:e + 1], gelu_bwd)
        g_w1[e], g_b1[e], g_w2[e], g_b2[e], gx[lo:hi] = a[0], b[0], c_[0], dd[0], ee[0]
    return out, h, gx, g_w1, g_b1, g_w2, g_b2


CASES = [
    # E, M, F, rows per expert, gap between experts (padded layout has gaps)
    (1, 64, 128, [5], 0),
    (4, 64, 128, [130, 0, 7, 64], 0),
    (3, 136, 264, [257, 31, 129], 3),
    (8, 256, 512, [100, 200, 0, 1, 300, 128, 127, 129], 0),
    (2, 512, 2048, [1024, 1000], 24),
    # more experts than one wave of the tile search covers, most of them nearly empty
    (150, 64, 256, [(7 * e) % 23 if e % 3 else 0 for e in range(149)] + [700], 0),
    # an expert with more rows than four 320-row tiles, and column counts that are not whole tiles
    (3, 264, 520, [1500, 3, 321], 5),
    # more than 16 rounds of tiles (the grouped kernel then numbers them in plain expert order)
    (150, 64, 4096, [257 + (11 * e) % 90 for e in range(150)], 0),
    # experts of eight or more m-tiles (their tiles are numbered in groups of 8 n-tiles, the last group short: 9 and
    # 11 n-tiles here) beside experts that keep the plain order, one of them with a remainder tile of its own class
    (4, 64, 2304, [2100, 300, 0, 2600], 0),
    (3, 128, 2816, [2049, 1793, 2305], 8),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gelu_bwd", ["tanh", "exact"])
@pytest.mark.parametrize("E,M,Fd,rows,gap", CASES)
def test_ffn_fwd_bwd_matches_oracle(E, M, Fd, rows, gap, gelu_bwd, dtype):
    from mole_amd import hip_ops as H, _lib as L
    print(f"ffn E={E} M={M} F={Fd} rows={rows} gap={gap} {gelu_bwd} {dtype}", flush=True)
    d = _make(E, M, Fd, rows, dtype, seed=E * 7 + M, pad_between=gap)
    c = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in d.items()}
    off = torch.from_numpy(d["off"]).cuda(); n = torch.from_numpy(d["n"]).cuda()
    out, h, a = H.ffn_fwd(c["xd"], off, n, c["w1"], c["b1"], c["w2"], c["b2"])
    w_out, w_h, w_gx, w_gw1, w_gb1, w_gw2, w_gb2 = _oracle_fwd_bwd(d, gelu_bwd)
    t = tol(dtype)
    mask = torch.zeros(max(d["R"], 1), dtype=torch.bool)
    for e in range(E):
        mask[int(d["off"][e]):int(d["off"][e]) + int(d["n"][e])] = True
    assert rel_err(h.cpu()[mask], w_h[mask]) < t
    assert rel_err(out.cpu()[mask], w_out[mask]) < t
    assert rel_err(a.cpu()[mask], torch.nn.functional.gelu(w_h[mask])) < t
    g_w1 = torch.full_like(c["w1"], 9.0); g_w2 = torch.full_like(c["w2"], 9.0)
    g_b1 = torch.full_like(c["b1"], 9.0); g_b2 = torch.full_like(c["b2"], 9.0)
    mode = L.GELU_BWD_TANH if gelu_bwd == "tanh" else L.GELU_BWD_EXACT
    gx = H.ffn_bwd(c["go"], c["xd"], h, a, off, n, c["w1"], c["w2"], g_w1, g_b1, g_w2, g_b2, True, False, mode)
    # the backward consumes the GPU's own saved h (rounded to the storage dtype), so compare against the
    # oracle evaluated on that same h for the tight fp32 bound
    assert rel_err(gx.cpu()[mask], w_gx[mask]) < t
    assert rel_err(g_w2, w_gw2) < t
    assert rel_err(g_b2, w_gb2) < t
    assert rel_err(g_w1, w_gw1) < t
    assert rel_err(g_b1, w_gb1) < t
    # accumulate variant (bffn_bwd_acc): a second call adds the same gradients again
    # (bf16: the running sum is rounded to bf16 after every call)
    H.ffn_bwd(c["go"], c["xd"], h, a, off, n, c["w1"], c["w2"], g_w1, g_b1, g_w2, g_b2, False, True, mode)
    assert rel_err(g_w1, 2 * w_gw1) < t and rel_err(g_b2, 2 * w_gb2) < t
    assert rel_err(g_w2, 2 * w_gw2) < t and rel_err(g_b1, 2 * w_gb1) < t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_nt_gate_logits(dtype):
    from mole_amd import hip_ops as H
    print(f"gemm_nt {dtype}", flush=True)
    g = torch.Generator().manual_seed(1)
    for rows, N, K in [(1, 1, 8), (300, 16, 512), (1000, 256, 1024), (129, 100, 264)]:
        a = torch.randn(rows, K, generator=g).to(dtype); b = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
        c = H.gemm_nt(a.cuda(), b.cuda())
        want = a.float() @ b.float().t()
        assert rel_err(c, want) < (1e-5 if dtype == torch.float32 else 1e-4)   # fp32 accumulation of exact products


@pytest.mark.parametrize("dtype,step", [(torch.bfloat16, 8), (torch.float32, 16), (torch.float32, 4)])
@pytest.mark.parametrize("seed", range(6))
def test_ffn_random_shapes(seed, dtype, step):
    """Random expert counts, loads and widths through the grouped kernels: 8-aligned widths for the bf16 direct-to-LDS
    kernel, 16-aligned ones for the fp32 one (whole stages of K), 4-aligned ones for the mix of the fp32 kernel (weight
    gradients) and the generic one (row-ragged products whose K is not whole stages)."""
    from mole_amd import hip_ops as H, _lib as L
    rng = np.random.default_rng(100 + seed)
    E = int(rng.integers(1, 40))
    M = int(rng.integers(1, 40)) * step
    Fd = int(rng.integers(1, 80)) * step
    rows = [int(r) for r in rng.choice([0, 1, 31, 32, 33, 63, 64, 65, 127, 129, 255, 256, 257, 320, 321, 640, 700], size=E)]
    gap = int(rng.integers(0, 3))
    print(f"ffn random seed={seed} {dtype} E={E} M={M} F={Fd} rows={rows} gap={gap}", flush=True)
    d = _make(E, M, Fd, rows, dtype, seed=seed, pad_between=gap)
    c = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in d.items()}
    off = torch.from_numpy(d["off"]).cuda(); n = torch.from_numpy(d["n"]).cuda()
    out, h, a = H.ffn_fwd(c["xd"], off, n, c["w1"], c["b1"], c["w2"], c["b2"])
    w_out, w_h, w_gx, w_gw1, w_gb1, w_gw2, w_gb2 = _oracle_fwd_bwd(d, "tanh")
    t = tol(dtype)
    mask = torch.zeros(max(d["R"], 1), dtype=torch.bool)
    for e in range(E):
        mask[int(d["off"][e]):int(d["off"][e]) + int(d["n"][e])] = True
    if mask.any():
        assert rel_err(h.cpu()[mask], w_h[mask]) < t
        assert rel_err(out.cpu()[mask], w_out[mask]) < t
    g_w1 = torch.full_like(c["w1"], 9.0); g_w2 = torch.full_like(c["w2"], 9.0)
    g_b1 = torch.full_like(c["b1"], 9.0); g_b2 = torch.full_like(c["b2"], 9.0)
    gx = H.ffn_bwd(c["go"], c["xd"], h, a, off, n, c["w1"], c["w2"], g_w1, g_b1, g_w2, g_b2, True, False, L.GELU_BWD_TANH)
    if mask.any():
        assert rel_err(gx.cpu()[mask], w_gx[mask]) < t
        assert rel_err(g_w2, w_gw2) < t and rel_err(g_b2, w_gb2) < t
        assert rel_err(g_w1, w_gw1) < t and rel_err(g_b1, w_gb1) < t
    else:   # no rows at all: every gradient is exactly zero
        for gt in (g_w1, g_b1, g_w2, g_b2):
            assert float(gt.float().abs().max()) == 0.0


def test_ffn_benchmark_size_against_fp32_products():
    """The benchmark's own shape (16 experts of 1024 -> 4096 -> 1024 in bf16, 16384 rows at uneven loads up to the
    capacity of 1280): forward and backward of three experts against fp32 torch products of the same rounded
    operands on the GPU (the CPU oracle would take minutes at this size), plus bias gradients of all experts."""
    from mole_amd import hip_ops as H, _lib as L
    E, M, Fd = 16, 1024, 4096
    g = torch.Generator().manual_seed(5)
    loads = torch.clamp((torch.randn(E, generator=g) * 120 + 1024).int(), min=1, max=1280)
    off = torch.zeros(E + 1, dtype=torch.int32)
    off[1:] = torch.cumsum(loads, 0)
    R = int(off[-1])
    print(f"ffn benchmark size: loads {loads.tolist()} R={R}", flush=True)
    dev, dt = "cuda", torch.bfloat16
    gd = torch.Generator(device=dev).manual_seed(6)
    rnd = lambda *s, sc=1.0: (torch.randn(*s, generator=gd, device=dev) * sc).to(dt)
    xd, go = rnd(R, M), rnd(R, M, sc=0.02)
    w1, b1, w2, b2 = rnd(E, Fd, M, sc=0.03), rnd(E, Fd, sc=0.03), rnd(E, Fd, M, sc=0.03), rnd(E, M, sc=0.03)
    offd, nd = off.cuda(), loads.int().cuda()
    out, h, a = H.ffn_fwd(xd, offd, nd, w1, b1, w2, b2)
    g_w1, g_b1, g_w2, g_b2 = torch.empty_like(w1), torch.empty_like(b1), torch.empty_like(w2), torch.empty_like(b2)
    gx = H.ffn_bwd(go, xd, h, a, offd, nd, w1, w2, g_w1, g_b1, g_w2, g_b2, True, False, L.GELU_BWD_EXACT)
    torch.cuda.synchronize()
    t = tol(dt)
    for e in (0, 7, 15):
        lo, hi = int(off[e]), int(off[e + 1])
        x32, go32 = xd[lo:hi].float(), go[lo:hi].float()
        h32 = x32 @ w1[e].float().t() + b1[e].float()
        a32 = torch.nn.functional.gelu(h32)
        o32 = a32 @ w2[e].float() + b2[e].float()
        assert rel_err(h[lo:hi], h32) < t and rel_err(a[lo:hi], a32) < t and rel_err(out[lo:hi], o32) < t
        # backward from the kernel's own (bf16) h, as the kernel sees it
        hs = h[lo:hi].float()
        hs.requires_grad_(True)
        torch.nn.functional.gelu(hs).backward(go32 @ w2[e].float().t())
        t32 = hs.grad
        assert rel_err(g_w2[e], a[lo:hi].float().t() @ go32) < t
        assert rel_err(g_w1[e], t32.t() @ x32) < t
        assert rel_err(gx[lo:hi], t32 @ w1[e].float()) < t
        assert rel_err(g_b1[e], t32.sum(0)) < t
    # bias gradient of the second linear for every expert: plain column sums of go
    want_b2 = torch.stack([go[int(off[e]):int(off[e + 1])].float().sum(0) for e in range(E)])
    assert rel_err(g_b2, want_b2) < t


def test_ffn_imbalanced_full_size_against_fp32_products():
    """The imbalanced configuration at its real shape (64 experts of 2048 -> 8192 -> 2048 in bf16, 16384 kept rows,
    expert loads from a Zipf-biased top-2 routing: a handful of rows up to well over a thousand): the lightest, a
    middle and the heaviest expert against fp32 torch products of the same rounded operands, forward and backward."""
    from mole_amd import hip_ops as H, _lib as L
    from tests.util import zipf_scores
    S, E, k, M, Fd = 8192, 64, 2, 2048, 8192
    r = H.route(zipf_scores(S, E, seed=11).cuda(), k, 0.0)
    loads = r.kept_rows.cpu()
    off = r.offsets.cpu()
    R = int(off[-1])
    assert R == S * k
    order = torch.argsort(loads)
    picks = [int(order[0]), int(order[E // 2]), int(order[-1])]
    print(f"ffn imbalanced full size: loads min {int(loads.min())} median {int(loads.median())} max {int(loads.max())}, "
          f"experts {picks}", flush=True)
    dev, dt = "cuda", torch.bfloat16
    gd = torch.Generator(device=dev).manual_seed(12)
    rnd = lambda *s, sc=1.0: (torch.randn(*s, generator=gd, device=dev) * sc).to(dt)
    xd, go = rnd(R, M), rnd(R, M, sc=0.02)
    w1, b1, w2, b2 = rnd(E, Fd, M, sc=0.02), rnd(E, Fd, sc=0.02), rnd(E, Fd, M, sc=0.02), rnd(E, M, sc=0.02)
    out, h, a = H.ffn_fwd(xd, r.offsets, r.kept_rows, w1, b1, w2, b2)
    g_w1, g_b1, g_w2, g_b2 = torch.empty_like(w1), torch.empty_like(b1), torch.empty_like(w2), torch.empty_like(b2)
    gx = H.ffn_bwd(go, xd, h, a, r.offsets, r.kept_rows, w1, w2, g_w1, g_b1, g_w2, g_b2, True, False, L.GELU_BWD_TANH)
    torch.cuda.synchronize()
    t = tol(dt)
    c = 0.7978845608028654
    for e in picks:
        lo, hi = int(off[e]), int(off[e + 1])
        if hi == lo:
            assert float(g_w1[e].float().abs().max()) == 0.0 and float(g_w2[e].float().abs().max()) == 0.0
            continue
        x32, go32 = xd[lo:hi].float(), go[lo:hi].float()
        h32 = x32 @ w1[e].float().t() + b1[e].float()
        assert rel_err(h[lo:hi], h32) < t
        assert rel_err(a[lo:hi], torch.nn.functional.gelu(h32)) < t
        assert rel_err(out[lo:hi], torch.nn.functional.gelu(h32) @ w2[e].float() + b2[e].float()) < t
        hs = h[lo:hi].float()                      # the derivative the reference compiles (MOLE/cpp/gelu.cu:3-14)
        th = torch.tanh(c * (hs + 0.044715 * hs ** 3))
        dg = 0.5 * (1 + th) + 0.5 * hs * c * (1 - th * th) * (1 + 3 * 0.044715 * hs * hs)
        t32 = (go32 @ w2[e].float().t()) * dg
        assert rel_err(g_w2[e], a[lo:hi].float().t() @ go32) < t
        assert rel_err(g_w1[e], t32.t() @ x32) < t
        assert rel_err(gx[lo:hi], t32 @ w1[e].float()) < t
        assert rel_err(g_b1[e], t32.sum(0)) < t
        assert rel_err(g_b2[e], go32.sum(0)) < t


def test_ffn_fine_grained_full_size_against_fp32_products():
    """The fine-grained configuration at its real shape (256 experts of 2048 -> 1024 -> 2048 in bf16, top-8 of
    32768 tokens: 262144 kept rows, about a thousand per expert, more than 16 rounds of tiles per launch): three
    experts against fp32 torch products of the same rounded operands, forward and backward (exact GELU')."""
    from mole_amd import hip_ops as H, _lib as L
    S, E, k, M, Fd = 32768, 256, 8, 2048, 1024
    dev, dt = "cuda", torch.bfloat16
    gd = torch.Generator(device=dev).manual_seed(21)
    scores = torch.softmax(torch.randn(S, E, generator=gd, device=dev), -1)
    r = H.route(scores, k, 0.0)
    off = r.offsets.cpu()
    R = int(off[-1])
    assert R == S * k
    print(f"ffn fine-grained full size: loads {int(r.kept_rows.min())}..{int(r.kept_rows.max())}", flush=True)
    rnd = lambda *s, sc=1.0: (torch.randn(*s, generator=gd, device=dev) * sc).to(dt)
    xd, go = rnd(R, M), rnd(R, M, sc=0.02)
    w1, b1, w2, b2 = rnd(E, Fd, M, sc=0.02), rnd(E, Fd, sc=0.02), rnd(E, Fd, M, sc=0.02), rnd(E, M, sc=0.02)
    out, h, a = H.ffn_fwd(xd, r.offsets, r.kept_rows, w1, b1, w2, b2)
    g_w1, g_b1, g_w2, g_b2 = torch.empty_like(w1), torch.empty_like(b1), torch.empty_like(w2), torch.empty_like(b2)
    gx = H.ffn_bwd(go, xd, h, a, r.offsets, r.kept_rows, w1, w2, g_w1, g_b1, g_w2, g_b2, True, False, L.GELU_BWD_EXACT)
    torch.cuda.synchronize()
    t = tol(dt)
    for e in (0, 131, 255):
        lo, hi = int(off[e]), int(off[e + 1])
        x32, go32 = xd[lo:hi].float(), go[lo:hi].float()
        h32 = x32 @ w1[e].float().t() + b1[e].float()
        assert rel_err(h[lo:hi], h32) < t
        assert rel_err(out[lo:hi], torch.nn.functional.gelu(h32) @ w2[e].float() + b2[e].float()) < t
        hs = h[lo:hi].float()
        hs.requires_grad_(True)
        torch.nn.functional.gelu(hs).backward(go32 @ w2[e].float().t())
        t32 = hs.grad
        assert rel_err(g_w2[e], a[lo:hi].float().t() @ go32) < t
        assert rel_err(g_w1[e], t32.t() @ x32) < t
        assert rel_err(gx[lo:hi], t32 @ w1[e].float()) < t
        assert rel_err(g_b1[e], t32.sum(0)) < t
        assert rel_err(g_b2[e], go32.sum(0)) < t


def _bf16_grid(limit=8.0, min_exp=-14):
    """Every bf16 value v with 2^min_exp <= |v| <= limit, and zero."""
    bits = torch.arange(0, 1 << 15, dtype=torch.int32)
    v = (bits << 16).view(torch.float32)
    v = v[torch.isfinite(v) & (v <= limit) & (v >= 2.0 ** min_exp)]
    return torch.cat([torch.zeros(1), v, -v])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_activation_math_on_a_dense_grid(dtype):
    """The GELU of the forward epilogue and both GELU derivatives of the backward epilogue, pinned through the
    FFN entry points themselves on every bf16 value of magnitude 2^-14 .. 8 (about 4400 points): one-hot rows in
    w1 make h an exact copy of xd, one-hot rows in w2 make go . w2^T exactly 1, so a = gelu(h) and t = gelu'(h)
    rounded once to the buffer dtype.  bf16 results come from polynomial fits (stated absolute error 6e-5 for the
    GELU's erf part, 2e-4 for the derivatives); the bound is that error plus the rounding of the result (half a
    unit in the last place of its binade).  fp32 results come from the closed forms and are held to 2e-6."""
    from mole_amd import hip_ops as H, _lib as L
    grid = _bf16_grid()
    M, Fd = 64, 256
    rows = (grid.numel() + M - 1) // M
    vals = torch.zeros(rows * M)
    vals[:grid.numel()] = grid
    xd = vals.view(rows, M).to(dtype).cuda()
    w1 = torch.zeros(1, Fd, M)
    w1[0, torch.arange(Fd), torch.arange(Fd) % M] = 1.0          # h[r, f] = xd[r, f mod M]
    w2 = torch.zeros(1, Fd, M)
    w2[0, :, 0] = 1.0                                             # (go . w2^T)[r, f] = go[r, 0]
    b1, b2 = torch.zeros(1, Fd), torch.zeros(1, M)
    go = torch.zeros(rows, M)
    go[:, 0] = 1.0
    off = torch.tensor([0, rows], dtype=torch.int32).cuda()
    n = torch.tensor([rows], dtype=torch.int32).cuda()
    dev = lambda t: t.to(dtype).cuda()
    w1d, w2d = dev(w1), dev(w2)
    out, h, a = H.ffn_fwd(xd, off, n, w1d, dev(b1), w2d, dev(b2))
    h64 = xd.double().cpu().repeat(1, Fd // M)
    assert torch.equal(h.double().cpu(), h64)                     # the set-up: h is xd, exactly
    gelu64 = 0.5 * h64 * (1.0 + torch.erf(h64 / 2.0 ** 0.5))
    bits = 8 if dtype == torch.bfloat16 else 24          # significand bits of the buffer dtype

    def half_ulp(v, slack):
        """Half a unit in the last place of the binade that |v| + slack falls into (the result is rounded once)."""
        mag = torch.clamp(v.abs() + slack, min=2.0 ** -126)
        return torch.pow(2.0, torch.floor(torch.log2(mag)) - bits)

    poly = 6e-5 if dtype == torch.bfloat16 else 2e-6
    err = (a.double().cpu() - gelu64).abs()
    slack = poly * torch.clamp(h64.abs(), min=1.0)
    bound = slack + half_ulp(gelu64, slack)
    worst = float((err - half_ulp(gelu64, slack)).max())
    print(f"fused GELU {dtype}: worst error beyond rounding {worst:.2e}", flush=True)
    assert bool((err <= bound).all()), f"GELU off by {float((err / bound).max()):.2f}x its bound"
    for variant, fn, code in (("tanh", O.d_gelu_tanh, L.GELU_BWD_TANH), ("exact", O.d_gelu_exact, L.GELU_BWD_EXACT)):
        g_w1, g_b1, g_w2, g_b2 = (torch.empty_like(t) for t in (w1d, dev(b1), w2d, dev(b2)))
        t = torch.empty(rows, Fd, dtype=dtype, device="cuda")
        H.ffn_bwd_into(dev(go), xd, h, a, off, n, 1, rows, M, Fd, w1d, w2d, t, g_w1, g_b1, g_w2, g_b2, None, False, code)
        d64 = fn(h64)
        err = (t.double().cpu() - d64).abs()
        polyd = 2e-4 if dtype == torch.bfloat16 else 2e-6
        slack = torch.full_like(d64, polyd)
        bound = slack + half_ulp(d64, slack)
        worst = float((err - half_ulp(d64, slack)).max())
        print(f"fused GELU' ({variant}) {dtype}: worst error beyond rounding {worst:.2e}", flush=True)
        assert bool((err <= bound).all()), f"GELU' ({variant}) off by {float((err / bound).max()):.2f}x its bound"
