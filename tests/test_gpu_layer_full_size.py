"""The whole layer (gate, routing, dispatch, grouped FFN, combine and all their gradients) at the full sizes of the
bf16 configurations - Switch-style top-1 with capacity drop, Zipf-imbalanced top-2, fine-grained top-8 - against an
fp32 restatement of the same layer written with torch autograd on the GPU (the CPU oracle would take minutes at these
sizes; at small sizes tests/test_gpu_layer.py compares the same module with the oracle itself).  The restatement
takes the routing decisions (expert indices, dropped pairs) from the layer's own route, which is compared with the
oracle bit for bit elsewhere, and recomputes everything that is floating point from the bf16-rounded operands:
scores, normalised gates, both Linear layers with erf-GELU forward and the tanh-form derivative backward, the
gate-weighted sum and every gradient."""
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O
from tests.util import BF16_TOL, rel_err_dev

pytestmark = pytest.mark.gpu


class _GeluErfFwdTanhBwd(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h):
        ctx.save_for_backward(h)
        return F.gelu(h)

    @staticmethod
    def backward(ctx, g):
        (h,) = ctx.saved_tensors
        return g * O.d_gelu_tanh(h)


CONFIGS = {
    # name: S, M, E, k, F, capacity factor, Zipf gate bias
    "c2": (16384, 1024, 16, 1, 4096, 1.25, False),
    "c2_cf1": (16384, 1024, 16, 1, 4096, 1.0, False),     # the same layer at capacity 1024: the fuller experts overflow
    "c3": (8192, 2048, 64, 2, 8192, 0.0, True),
    "c5": (32768, 2048, 256, 8, 1024, 0.0, False),
}


@pytest.mark.parametrize("name", ["c2", "c2_cf1", "c3", "c5"])
def test_layer_full_size_against_fp32_restatement(name):
    from mole_amd.moe.layer import MOLEModule
    S, M, E, k, Fd, cf, zipf = CONFIGS[name]
    print(f"layer full size {name}", flush=True)
    MOLEModule.reset_instances()
    g = torch.Generator(device="cuda").manual_seed(3)
    bias = None
    if zipf:
        ranks = torch.randperm(E, generator=torch.Generator().manual_seed(3)).float() + 1.0
        bias = torch.log(ranks ** -1.2)
    m = MOLEModule(0, E, M, Fd, -1, k, 4, {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", 1, False, False,
                   dtype=torch.bfloat16, gate_logit_bias=bias)
    with torch.no_grad():
        scale = 1.0 / M ** 0.5 if name == "c5" else 0.02          # c5: gate logits of unit variance
        m.gate[0].linear.weight.copy_(torch.randn(E, M, device="cuda", generator=g) * scale)
        for p in (m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU):
            p.all_tensors.copy_((torch.randn(p.all_tensors.shape, device="cuda", generator=g) * 0.02).bfloat16())
    x = torch.randn(S, M, device="cuda", generator=g).bfloat16()
    dy = (torch.randn(S, M, device="cuda", generator=g) * 1e-2).bfloat16()
    xin = x.clone().requires_grad_(True)
    y = m(xin, capacity_factor=cf)
    y.backward(dy)
    torch.cuda.synchronize()
    r = m.last_route
    loads = r.kept_rows.cpu()
    print(f"layer full size {name}: kept rows {int(loads.sum())} of {S * k}, loads {int(loads.min())}..{int(loads.max())}", flush=True)
    if zipf:
        assert int(loads.max()) > 20 * max(int(loads.min()), 1)
    if cf > 0:
        assert int(loads.max()) <= k * int(cf * ((S + E - 1) // E))
    if name == "c2_cf1":
        assert int(loads.sum()) < S * k                          # pairs were dropped, their tokens output zeros
        dropped = (r.row < 0).all(dim=0)
        assert int(dropped.sum()) > 0 and float(y[dropped].float().abs().max()) == 0.0

    # ---- the restatement -------------------------------------------------------------------------
    idx, keep = r.idx.long(), r.row >= 0
    xf = x.float().requires_grad_(True)
    wgf = m.gate[0].linear.weight.detach().bfloat16().float().requires_grad_(True)     # the gate multiplies bf16 operands
    logits = xf @ wgf.t()
    if bias is not None:
        logits = logits + bias.cuda()
    scores = torch.softmax(logits, dim=-1)
    graw = scores.gather(1, idx.t()).t()
    gates = graw / torch.clamp(graw.sum(0, keepdim=True), min=O.FP32_EPS) if k > 1 else graw
    # the layer's own gates, computed from its own scores, agree to rounding
    assert rel_err_dev(r.gates, gates.detach()) < 1e-3
    y_ref = torch.zeros(S, M, device="cuda")
    leaves = []
    for e in range(E):
        w1, b1, w2, b2 = (p.all_tensors[e].float().requires_grad_(True)
                          for p in (m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU))
        leaves.append((w1, b1, w2, b2))
        sel = (idx == e) & keep                                   # [k, S]: kept pairs routed to this expert
        for j in range(k):
            tok = sel[j].nonzero().flatten()
            if tok.numel() == 0:
                continue
            o = _GeluErfFwdTanhBwd.apply(xf[tok] @ w1.t() + b1) @ w2 + b2
            y_ref = y_ref.index_add(0, tok, gates[j, tok].unsqueeze(1) * o)
    assert rel_err_dev(y, y_ref.detach()) < BF16_TOL
    y_ref.backward(dy.float())
    assert rel_err_dev(xin.grad, xf.grad) < BF16_TOL
    assert rel_err_dev(m.gate[0].linear.weight.grad, wgf.grad) < BF16_TOL
    worst = [0.0] * 4
    stores = (m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU)
    for e in range(E):
        for p in range(4):
            want = leaves[e][p].grad
            got = stores[p].grad_tensors[e]
            if want is None:                                      # an expert without rows: zero gradient
                assert float(got.float().abs().max()) == 0.0
                continue
            err = rel_err_dev(got, want)
            worst[p] = max(worst[p], err)
            assert err < BF16_TOL, f"{name}: expert {e} ({int(loads[e])} rows), parameter kind {p}: {err}"
    print(f"layer full size {name}: worst relative errors of g_w1, g_b1, g_w2, g_b2: {[round(w, 5) for w in worst]}", flush=True)
    MOLEModule.reset_instances()
