"""HIP dispatch / combine forward and backward against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import rel_err, tol, zipf_scores

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ragged", [True, False])
@pytest.mark.parametrize("S,E,k,cf,M", [(1, 2, 1, 1.0, 8), (300, 8, 2, 1.0, 64), (1000, 16, 1, 0.5, 520),
                                        (513, 4, 4, 0.0, 1024), (200, 32, 8, 0.0, 2048), (300, 64, 4, 0.0, 256),
                                        # top-k values between the kernels' compiled bounds (1, 2, 4, 8, 16), with drops
                                        (257, 8, 3, 0.5, 72), (129, 16, 5, 1.0, 264), (65, 32, 16, 0.0, 128),
                                        (40, 16, 16, 0.5, 1032), (90, 12, 7, 0.3, 2056)])
def test_permutes_match_oracle(S, E, k, cf, M, ragged, dtype):
    from mole_amd import hip_ops as H, _lib as L
    print(f"permute S={S} E={E} k={k} cf={cf} M={M} ragged={ragged} {dtype}", flush=True)
    g = torch.Generator().manual_seed(S + M)
    scores = zipf_scores(S, E, seed=S)
    c = O.extract_critical(scores.numpy(), k, cf)
    r = H.route(scores.cuda(), k, cf, True, 1, L.LAYOUT_RAGGED if ragged else L.LAYOUT_PADDED)
    total = int(c.offsets[-1]) if ragged else E * c.capacity
    x = torch.randn(S, M, generator=g).to(dtype)
    xf = x.float()
    # dispatch forward: a pure copy, exact in every dtype; padding rows zeroed like the reference's buffer
    xd = torch.full((max(total, 1), M), 7.0, dtype=dtype, device="cuda")
    H.dispatch_fwd(x.cuda(), r.row, total, out=xd)
    H.zero_pad_rows(xd, r.kept_rows, r.offsets)
    want = O.fast_encode(xf, c, ragged).reshape(total, M)
    assert torch.equal(xd[:total].float().cpu(), want)
    # combine forward
    o = torch.randn(max(total, 1), M, generator=g).to(dtype)
    y = H.combine_fwd(o.cuda(), r.row, r.gates)
    want_y = O.fast_decode(o[:total].float(), c, ragged)
    assert rel_err(y, want_y) < tol(dtype)
    # combine backward
    dy = torch.randn(S, M, generator=g).to(dtype)
    d_o = torch.full((max(total, 1), M), 3.0, dtype=dtype, device="cuda")
    d_o, dg = H.combine_bwd(dy.cuda(), o.cuda(), r.row, r.gates, d_o)
    H.zero_pad_rows(d_o, r.kept_rows, r.offsets)
    want_do, want_dg = O.fast_decode_bwd(dy.float(), o[:total].float(), c, ragged)
    assert rel_err(d_o[:total], want_do) < tol(dtype)
    assert rel_err(dg, want_dg) < (1e-5 if dtype == torch.float32 else 1e-4)   # fp32 sums of exact products
    # dispatch backward, alone and with the gate's input gradient folded in
    dxd = torch.randn(max(total, 1), M, generator=g).to(dtype)
    dx = H.dispatch_bwd(dxd.cuda(), r.row)
    want_dx = O.fast_encode_bwd(dxd[:total].float(), c, ragged)
    assert rel_err(dx, want_dx) < tol(dtype)
    dlog = torch.randn(S, E, generator=g) * 0.1
    wg = torch.randn(E, M, generator=g)
    dx2 = H.dispatch_bwd(dxd.cuda(), r.row, dlog.cuda(), wg.cuda())
    assert rel_err(dx2, want_dx + dlog @ wg) < tol(dtype)


def test_permute_full_size_properties():
    """c5-sized round trip: combine(dispatch(x)) with unit gates = k*x, and <dispatch(x), D> = <x, dispatch_bwd(D)>."""
    from mole_amd import hip_ops as H
    S, E, k, M = 32768, 256, 8, 2048
    print("permute full size c5", flush=True)
    scores = zipf_scores(S, E, seed=2).cuda()
    r = H.route(scores, k, 0.0, normalize_gate=False)
    x = torch.randn(S, M, device="cuda", generator=torch.Generator(device="cuda").manual_seed(4)).bfloat16()
    xd = H.dispatch_fwd(x, r.row, S * k)
    y = H.combine_fwd(xd, r.row, torch.ones_like(r.gates))
    assert torch.equal(y.float(), (x.float() * k).bfloat16().float())
    # adjointness on small integers: every sum of k = 8 values stays exactly representable in bf16, so the two
    # inner products must agree to the last bit
    gen = torch.Generator(device="cuda").manual_seed(5)
    xi = torch.randint(-3, 4, (S, M), device="cuda", generator=gen).bfloat16()
    d = torch.randint(-2, 3, (S * k, M), device="cuda", generator=gen).bfloat16()
    xdi = H.dispatch_fwd(xi, r.row, S * k)
    lhs = (xdi.double() * d.double()).sum()
    dx = H.dispatch_bwd(d, r.row)
    rhs = (xi.double() * dx.double()).sum()
    assert float(lhs) == float(rhs)


@pytest.mark.parametrize("S,E,k,M,cf", [(100, 16, 1, 256, 1.0), (1000, 3, 2, 512, 0.0), (777, 32, 4, 1280, 0.5),
                                        (16384, 16, 1, 1024, 1.25), (33, 20, 2, 256, 0.0),
                                        (500, 24, 2, 384, 1.0), (64, 8, 1, 128, 1.0)])
def test_dispatch_bwd_with_gate_bf16_wide_rows(S, E, k, M, cf):
    """The fused dispatch backward for bf16 rows of whole 256-column groups (the matrix-core variant): gather-sum
    of the kept rows plus dlogits @ Wg, against the oracle's gather and an fp32 product of the bf16-rounded
    operands (the kernel rounds dlogits and Wg to bf16, which the 2e-2 bf16 tolerance covers either way)."""
    from mole_amd import hip_ops as H
    print(f"dispatch_bwd+gate S={S} E={E} k={k} M={M} cf={cf}", flush=True)
    g = torch.Generator().manual_seed(S + M)
    scores = zipf_scores(S, E, seed=S)
    c = O.extract_critical(scores.numpy(), k, cf)
    r = H.route(scores.cuda(), k, cf)
    total = int(c.offsets[-1])
    dxd = torch.randn(max(total, 1), M, generator=g).bfloat16()
    dlog = torch.randn(S, E, generator=g) * 0.1
    wg = torch.randn(E, M, generator=g)
    got = H.dispatch_bwd(dxd.cuda(), r.row, dlog.cuda(), wg.cuda())
    want = O.fast_encode_bwd(dxd[:total].float(), c, True) + dlog @ wg
    assert got.shape == (S, M)
    assert rel_err(got, want) < tol(torch.bfloat16)
    tight = O.fast_encode_bwd(dxd[:total].float(), c, True) + dlog.bfloat16().float() @ wg.bfloat16().float()
    assert rel_err(got, tight) < 6e-3          # what is left is the output's own rounding to bf16


def test_kernel_timing_counts_launches_and_leaves_results_alone():
    """The optional per-kernel timing (events attached to the launches): counts one launch per call and id,
    reports a positive duration, and the timed launches give the same bits as the untimed ones."""
    from mole_amd import hip_ops as H, _lib as L
    S, E, k, M = 700, 8, 2, 256
    print("kernel timing", flush=True)
    scores = zipf_scores(S, E, seed=3).cuda()
    x = torch.randn(S, M, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()

    def run():
        r = H.route(scores, k, 1.0)
        xd = H.dispatch_fwd(x, r.row, S * k)
        total = int(r.offsets[-1])                    # rows past the kept ones are never written
        return xd[:total], H.combine_fwd(xd, r.row, r.gates), r.row

    plain = [t.clone() for t in run()]
    L.kernel_timing_read()                                              # forget whatever an earlier test left
    L.kernel_timing_enable(True)
    try:
        timed = [[t.clone() for t in run()] for _ in range(3)]
        stats = L.kernel_timing_read()
    finally:
        L.kernel_timing_enable(False)
    for name in ("route", "dispatch_fwd", "combine_fwd"):
        count, ms = stats[name]
        assert count == 3 and 0.0 < ms < 50.0, (name, count, ms)
    assert stats["combine_bwd"][0] == 0
    for rep in timed:
        assert all(torch.equal(a, b) for a, b in zip(rep, plain))
    assert all(c == 0 for c, _ in L.kernel_timing_read().values())      # a read forgets what it returned


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,M,E,k,cf,normalize,aux", [(300, 64, 8, 2, 1.0, True, True), (1000, 128, 16, 1, 1.25, True, False),
                                                      (513, 64, 100, 4, 0.0, False, True), (257, 256, 256, 8, 0.0, True, True),
                                                      (64, 64, 3, 3, 0.5, True, False)])
def test_combine_bwd_with_the_gate_backward_in_its_tail(S, M, E, k, cf, normalize, aux, dtype):
    """mole_combine_bwd_gate against mole_combine_bwd followed by mole_gate_bwd on the same inputs: the same d_o bit
    for bit, the same d(logits) to rounding (the two sum a token's k terms over lanes in different patterns)."""
    from mole_amd import hip_ops as H
    from tests.util import zipf_scores
    print(f"combine_bwd_gate S={S} M={M} E={E} k={k} cf={cf} {dtype}", flush=True)
    g = torch.Generator().manual_seed(S + E)
    scores = zipf_scores(S, E, seed=S).cuda()
    r = H.route(scores, k, cf, normalize)
    rows = max(int(r.offsets[-1]), 1)
    o = torch.randn(rows, M, generator=g).to(dtype).cuda()
    dy = torch.randn(S, M, generator=g).to(dtype).cuda()
    kw = dict(counts0=r.counts[0], d_l_aux=torch.tensor([0.7], device="cuda")) if aux else {}
    d_o1, dgates = H.combine_bwd(dy, o, r.row, r.gates)
    want = H.gate_bwd(dgates, scores, r.idx, normalize, True, **kw)
    d_o2, got = H.combine_bwd_gate(dy, o, r.row, r.gates, scores, r.idx, normalize, True, **kw)
    torch.cuda.synchronize()
    kept = (r.row >= 0).any(dim=0)
    assert bool(kept.any())
    written = torch.zeros(rows, dtype=torch.bool, device="cuda")
    written[r.row[r.row >= 0].long()] = True
    assert torch.equal(d_o1[written], d_o2[written])
    assert rel_err(got, want) < 1e-5
    want_s = H.gate_bwd(dgates, scores, r.idx, normalize, False, **kw)
    _, got_s = H.combine_bwd_gate(dy, o, r.row, r.gates, scores, r.idx, normalize, False, **kw)
    assert rel_err(got_s, want_s) < 1e-5
