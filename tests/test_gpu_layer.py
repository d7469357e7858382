"""The MoE layer module end to end (forward + backward) against the CPU oracle's layer, for
GPU-resident and host-offloaded experts, in both execution shapes of MOLEModule."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import expert_rel_err, rel_err, row_rel_err, tol

pytestmark = pytest.mark.gpu


def _build(S, M, E, k, Fd, dtype, d_experts=0, pool=0, ebatch=4, seed=0, acc_step=1, adv_adam=False, **kw):
    from mole_amd.moe.layer import MOLEModule
    MOLEModule.reset_instances()
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(S, M, generator=g)
    wg = torch.randn(E, M, generator=g) * 0.02
    w1, b1 = torch.randn(E, Fd, M, generator=g) * 0.02, torch.randn(E, Fd, generator=g) * 0.02
    w2, b2 = torch.randn(E, Fd, M, generator=g) * 0.02, torch.randn(E, M, generator=g) * 0.02
    m = MOLEModule(d_experts, E - d_experts, M, Fd, pool if d_experts else -1, k, ebatch,
                   {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", acc_step, adv_adam, d_experts > 0, dtype=dtype, **kw)
    s = E - d_experts
    with torch.no_grad():
        m.gate[0].linear.weight.copy_(wg)
        for gp, cp, t in ((m.FC1_W_GPU, m.FC1_W_CPU, w1), (m.FC1_B_GPU, m.FC1_B_CPU, b1), (m.FC2_W_GPU, m.FC2_W_CPU, w2),
                          (m.FC2_B_GPU, m.FC2_B_CPU, b2)):
            if s:
                gp.all_tensors.copy_(t[:s])
            if d_experts:
                cp.all_tensors.copy_(t[s:])
    # the oracle sees the values the GPU sees: rounded to the parameter dtype
    rd = lambda t: t.to(dtype).float()
    ref = dict(x=rd(x), wg=(rd(wg) if dtype != torch.float32 else wg), w1=rd(w1), b1=rd(b1), w2=rd(w2), b2=rd(b2))
    return m, x.to(dtype).cuda(), ref


def _grads(m, E):
    s = m.s_experts
    out = []
    for gp, cp in ((m.FC1_W_GPU, m.FC1_W_CPU), (m.FC1_B_GPU, m.FC1_B_CPU), (m.FC2_W_GPU, m.FC2_W_CPU), (m.FC2_B_GPU, m.FC2_B_CPU)):
        parts = []
        if s:
            parts.append(gp.grad_tensors.float().cpu())
        if m.d_experts:
            parts.append(cp.all_tensors.grad_.float())
        out.append(torch.cat(parts))
    return out


def _run_and_compare(m, x, ref, k, cf, dtype, gelu_bwd="tanh", normalize=True, aux_w=0.0):
    """aux_w: weight of the load-balancing loss in the loss (loss = mean(y^2) + aux_w * l_aux)."""
    from mole_amd import core
    from mole_amd.utils import Ugate
    x = x.clone().requires_grad_(True)
    y = m(x, capacity_factor=cf)
    dy = (2.0 * y.detach().float() / y.numel()).to(dtype)       # d/dy of mean(y^2): the MSE-vs-zero loss
    if aux_w:
        assert m.l_aux.requires_grad
        torch.autograd.backward([y, m.l_aux], [dy, torch.tensor(aux_w, device=y.device)])
    else:
        y.backward(dy)
    torch.cuda.synchronize()
    core.synchronize_tran()                # gradients of offloaded experts are on their way to the host
    t = tol(dtype)
    # gate scores: GPU vs oracle within tolerance; then the oracle re-routes on the GPU's own scores so that
    # every routing decision is compared on identical inputs
    scores_gpu = Ugate.gate_scores(x.detach(), m.gate[0].linear.weight, m.gate[0].logit_bias).cpu()
    bias = m.gate[0].logit_bias.cpu() if m.gate[0].logit_bias is not None else None
    assert rel_err(scores_gpu, O.gate_scores(ref["x"], ref["wg"], bias)) < (1e-5 if dtype == torch.float32 else 2e-2)
    res = O.moe_layer(ref["x"], ref["wg"], ref["w1"], ref["b1"], ref["w2"], ref["b2"], k, cf, dy=dy.float().cpu(),
                      logit_bias=bias, normalize_gate=normalize, gelu_bwd=gelu_bwd, scores_override=scores_gpu,
                      d_l_aux=aux_w)
    assert rel_err(y, res.y) < t
    assert rel_err(x.grad, res.dx) < t
    assert rel_err(m.gate[0].linear.weight.grad, res.dwg) < t
    # the four expert gradients, every expert against its own largest element (an expert with few rows has small
    # gradients: one maximum over all experts would let it be wrong by any factor)
    for name, got, want in zip(("g_w1", "g_b1", "g_w2", "g_b2"), _grads(m, ref["w1"].shape[0]),
                               (res.g_w1, res.g_b1, res.g_w2, res.g_b2)):
        err = expert_rel_err(got, want)
        assert err < t, f"{name}: worst expert off by {err:.2e}"
        res.extras[name + "_gpu"] = got
    assert abs(float(m.l_aux.detach()) - res.crit.l_aux) < 1e-4 * max(1.0, res.crit.l_aux)
    res.extras["y_gpu"], res.extras["dx_gpu"] = y.detach(), x.grad
    return res


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("reference_layout", [False, True])
@pytest.mark.parametrize("S,M,E,k,Fd,cf", [(300, 64, 4, 2, 128, 1.0), (1000, 128, 8, 1, 256, 1.25), (513, 64, 16, 4, 128, 0.0)])
def test_layer_static_experts(S, M, E, k, Fd, cf, reference_layout, dtype):
    print(f"layer static S={S} M={M} E={E} k={k} F={Fd} cf={cf} ref_layout={reference_layout} {dtype}", flush=True)
    m, x, ref = _build(S, M, E, k, Fd, dtype, reference_layout=reference_layout)
    _run_and_compare(m, x, ref, k, cf, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("reference_layout", [False, True])
def test_layer_l_aux_carries_a_gradient(reference_layout, dtype):
    """loss = mean(y^2) + w * l_aux: the load-balancing term reaches the gate weight and the input through the
    scores (d l_aux / d scores[i,e] = E/S^2 counts0[e]), in both execution shapes of the module; the oracle's
    version of that term is pinned against autograd in tests/test_oracle_ffn.py."""
    print(f"layer l_aux gradient ref_layout={reference_layout} {dtype}", flush=True)
    m, x, ref = _build(500, 64, 8, 2, 128, dtype, reference_layout=reference_layout, seed=4)
    res0 = _run_and_compare(m, x, ref, 2, 1.0, dtype)
    m.gate[0].linear.weight.grad = None
    res1 = _run_and_compare(m, x, ref, 2, 1.0, dtype, aux_w=25.0)
    assert rel_err(res1.dwg, res0.dwg) > 0.05           # the term is not lost in the comparison's tolerance


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("activated_only", [True, False])
@pytest.mark.parametrize("d_experts,pool,ebatch,prefetch_n", [(8, 8, 4, 0), (6, 3, 2, 0), (8, 5, 2, 3), (4, 2, 4, 2),
                                                              (6, 5, 2, 5), (6, 4, 3, 4)])
def test_layer_offloaded_experts(d_experts, pool, ebatch, prefetch_n, activated_only, dtype):
    """Some or all experts live in pinned host memory and stream through a pool smaller than the layer.  The last
    two cases prefetch as many experts as the pool holds, so that a chunk which still contains prefetched
    experts reaches the end of the pool (the chunk is cut there, not wrapped onto slot 0)."""
    print(f"layer offload d={d_experts} pool={pool} ebatch={ebatch} prefetch={prefetch_n} act_only={activated_only} {dtype}", flush=True)
    E, k = 8, 2
    m, x, ref = _build(400, 64, E, k, 128, dtype, d_experts=d_experts, pool=pool, ebatch=ebatch,
                       activated_only=activated_only)
    if prefetch_n:
        m.set_prefetch(prefetch_n, prefetch_n)
        m.prefetch_fwd(prefetch_n)             # what the scheduler does before the first layer
        x2 = x.clone().requires_grad_(True)
        y = m(x2, capacity_factor=0.0, prefetch=True)   # last layer: triggers its own backward prefetch
        y.backward(torch.ones_like(y) * 1e-3)
        m.MOLECore.step = 0
        for gp in (m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU):
            if m.s_experts:
                gp.grad_tensors.zero_()
        m.gate[0].linear.weight.grad = None
        m.prefetch_fwd(prefetch_n)
        assert m.MOLECore.fwd_base == prefetch_n
    _run_and_compare(m, x, ref, k, 0.0, dtype)
    from mole_amd import core
    um = core.get_UniMem()
    assert um.virtual_offset() == 0 and um.view_pool_size() == pool


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("unified", [False, True])
def test_layer_activated_only_skips_experts_without_rows(unified, dtype):
    """Twelve tokens, top-1, eight offloaded experts: several experts get no row.  Only the activated ones are
    copied (the pool's byte counter says so exactly, forward and backward), the results equal the oracle's, the
    host gradients of the others read zero - also when they held a gradient from an earlier step - and a run
    with activated_only=False (every expert copied and launched, as the reference does) gives the same bits."""
    from mole_amd import core
    print(f"layer activated-only unified={unified} {dtype}", flush=True)
    S, M, E, k, Fd = 12, 64, 8, 1, 128
    kw = dict(device_s_experts=E) if unified else {}
    es = 4 if dtype == torch.float32 else 2
    expert_bytes = (2 * Fd * M + Fd + M) * es

    def run(activated_only, x_override=None):
        m, x, ref = _build(S, M, E, k, Fd, dtype, d_experts=E, pool=4, ebatch=2, seed=8, activated_only=activated_only, **kw)
        if x_override is not None:
            x = x_override
        um = core.get_UniMem()
        # an earlier step in which every expert was active leaves gradients behind in the host arrays
        big = torch.randn(4 * S * E, M, generator=torch.Generator().manual_seed(1)).to(dtype).cuda().requires_grad_(True)
        yb = m(big, capacity_factor=0.0)
        yb.backward(torch.ones_like(yb) * 1e-2)
        torch.cuda.synchronize(); core.synchronize_tran()
        assert all(float(m.FC1_W_CPU.all_tensors.grad_[e].abs().max()) > 0 for e in range(E))
        um.copy_stats(); um.reuse_stats()
        m.gate[0].linear.weight.grad = None
        res = _run_and_compare(m, x, ref, k, 0.0, dtype)
        nbytes, _ = um.copy_stats()
        nbytes += um.reuse_stats()          # what a backward pass found still in place from its forward pass
        return m, res, nbytes, _grads(m, E)

    m, res, nbytes, grads = run(True)
    active = [e for e in range(E) if res.crit.kept_rows[e] > 0]
    assert 0 < len(active) < E
    assert nbytes == 2 * len(active) * expert_bytes          # forward + backward, activated experts only
    for e in range(E):
        if e not in active:
            assert all(float(g[e].abs().max()) == 0.0 for g in grads)
    if unified:
        from mole_amd.utils.Uparam import UnifiedCPUTensor
        pool_t = UnifiedCPUTensor.get_cpu_experts()[0]
        assert pool_t.is_pinned() and pool_t.numel() == E * (2 * Fd * M + Fd + M)
        assert m.FC1_W_CPU.all_tensors.data_ptr() == pool_t.data_ptr()
        assert m.FC1_B_CPU.all_tensors.data_ptr() == pool_t.data_ptr() + E * Fd * M * es
    m2, res2, nbytes2, grads2 = run(False)
    assert nbytes2 == 2 * E * expert_bytes
    for a, b in zip(grads, grads2):
        assert torch.equal(a, b)


def test_pool_guards_and_reserve():
    """The process-wide pool refuses a second layer whose experts have another shape (it would read the slots at the
    wrong strides), and pool_prefetch hands out the reserved slots as tensors (core.cpp:1425)."""
    from mole_amd import core
    from mole_amd.moe.layer import MOLEModule
    m, x, ref = _build(100, 64, 4, 2, 128, torch.float32, d_experts=4, pool=4, ebatch=2)
    dist = {"local_rank": 0, "world_size": 1, "rank": 0}
    with pytest.raises(RuntimeError, match="cannot share"):
        MOLEModule(2, 0, 64, 256, 4, 2, 2, dist, "gelu", 1, False, True, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="slots"):
        core.create_UniMem(0, 9, torch.float32, [[128, 64], [128], [128, 64], [64]])
    MOLEModule._instance = MOLEModule._instance[:1]
    slots = core.pool_prefetch(0, 3)
    assert [tuple(t.shape) for t in slots] == [(3, 128, 64), (3, 128), (3, 128, 64), (3, 64)]
    um = core.get_UniMem()
    assert um.view_pool_size() == 1 and um.virtual_offset() == 3
    assert slots[0].data_ptr() == um.slot_tensor(0, 0, 3)
    slots[0].fill_(1.5)
    assert core.fetch_top_prefetched_batch(0) == 3 and um.view_pool_size() == 4
    assert core.get_stream_cdata(0, 1) == um.tran_stream_handle() != core.get_stream_cdata(0, 2)
    assert core.get_stream_cdata(0, 4) == um.tranback_stream_handle()
    from mole_amd.utils.Ustream import ExpertStreamCtx
    ExpertStreamCtx(device="cuda:0")
    assert ExpertStreamCtx.tran_back_stream().cuda_stream == um.tranback_stream_handle()
    assert ExpertStreamCtx.tran_stream().cuda_stream == um.tran_stream_handle()
    MOLEModule.reset_instances()


def test_layer_config1_exact():
    """Configuration 1 of the benchmark set as specified: 4096 x 512 fp32, 8 experts, top-2, F = 2048, N(0, 0.02) weights,
    MSE against zero, seed 0; with the reference's default capacity factor and without dropping.  Besides the
    max-norm tolerance, every row of y and dx is held to it relative to the row's own largest element."""
    for cf in (1.0, 0.0):
        print(f"layer config1 cf={cf}", flush=True)
        m, x, ref = _build(4096, 512, 8, 2, 2048, torch.float32, seed=0)
        res = _run_and_compare(m, x, ref, 2, cf, torch.float32)
        ry, rdx = row_rel_err(res.extras["y_gpu"], res.y), row_rel_err(res.extras["dx_gpu"], res.dx)
        print(f"layer config1 cf={cf}: per-row relative error y {ry:.2e}, dx {rdx:.2e}", flush=True)
        assert ry < 1e-5 and rdx < 1e-5
        # the two weight gradients row by row: row (e, f) of g_w1 and of g_w2 against its own largest element
        rw1 = row_rel_err(res.extras["g_w1_gpu"], res.g_w1)
        rw2 = row_rel_err(res.extras["g_w2_gpu"], res.g_w2)
        print(f"layer config1 cf={cf}: per-row relative error g_w1 {rw1:.2e}, g_w2 {rw2:.2e}", flush=True)
        assert rw1 < 1e-5 and rw2 < 1e-5


def _near_tie_report(scores64, idx_gpu, idx_cpu, k, bound):
    """Tokens whose chosen expert sets differ between the GPU and the oracle, each checked to be a genuine near
    tie: the scores (fp64 reference) of the experts the two sides disagree about lie within `bound` (relative)."""
    diff = (idx_gpu != idx_cpu).any(axis=0).nonzero()[0]
    for i in diff:
        a, b = idx_gpu[:, i], idx_cpu[:, i]
        # the experts at the choice positions where the two sides differ: another expert chosen, or the same experts
        # in another order
        involved = sorted(set(a[a != b].tolist()) | set(b[a != b].tolist()))
        vals = scores64[i, involved]
        assert float(vals.max() - vals.min()) <= bound * float(vals.max()), \
            f"token {i}: GPU chose {a.tolist()}, oracle {b.tolist()}, scores {scores64[i, sorted(set(a.tolist()) | set(b.tolist()))]}"
    return len(diff)


@pytest.mark.parametrize("name,S,M,E,k,cf,dtype", [("c1", 4096, 512, 8, 2, 1.0, torch.float32),
                                                   ("c2", 16384, 1024, 16, 1, 1.25, torch.bfloat16),
                                                   ("c3", 8192, 2048, 64, 2, 0.0, torch.bfloat16),
                                                   ("c5", 32768, 2048, 256, 8, 0.0, torch.bfloat16)])
def test_routing_from_tokens_matches_oracle(name, S, M, E, k, cf, dtype):
    """Routing end to end from x (gate product, softmax, top-k, locations, capacity, permutation) against the
    oracle run on the same seeded x and Wg with no help from the GPU's scores.  The two gates sum their products
    in different orders (and the bf16 gate multiplies bf16-rounded operands exactly into fp32), so scores differ
    in the last bits; an index may differ only where the competing scores are that close, and such tokens
    are counted.  With none, every routing output must be equal bit for bit."""
    from mole_amd import hip_ops as H
    from mole_amd.utils import Ugate
    print(f"routing from tokens {name}", flush=True)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(S, M, generator=g)
    # c5 is specified with N(0,1) gate logits (the two-kernel gate of 256 experts, top-8: near ties are likeliest
    # there), c3 with a Zipf(1.2) per-expert logit bias over a random ranking of the experts
    wg = torch.randn(E, M, generator=g) * (1.0 / M ** 0.5 if name == "c5" else 0.02)
    bias = torch.log((torch.randperm(E, generator=g).float() + 1.0) ** -1.2) if name == "c3" else None
    xr = x.to(dtype)
    wr = wg if dtype == torch.float32 else wg.bfloat16().float()      # the bf16 gate kernel rounds Wg
    scores_gpu = Ugate.gate_scores(xr.cuda(), wg.cuda(), None if bias is None else bias.cuda())
    r = H.route(scores_gpu, k, cf)
    scores_cpu = O.gate_scores(xr.float(), wr, bias)
    c = O.extract_critical(scores_cpu.numpy(), k, cf)
    idx_gpu, idx_cpu = r.idx.cpu().numpy(), np.stack(c.indices_s)
    logits64 = xr.double() @ wr.double().t()
    scores64 = torch.softmax(logits64 if bias is None else logits64 + bias.double(), dim=-1).numpy()
    # a few ulp of fp32 relative to the score.  An absolute difference d between two sums for the same logit is a
    # relative difference d of the score; c5's logits have unit variance and 2048 terms, so its two summation
    # orders differ by a few 1e-7 absolute where the other configurations' (logits of variance 0.02^2 M) stay below 1e-7
    flips = _near_tie_report(scores64, idx_gpu, idx_cpu, k, bound=(32 if name == "c5" else 8) * 1.2e-7)
    print(f"routing from tokens {name}: {flips} of {S} tokens routed differently (near ties)", flush=True)
    # with k choices out of E there are k orderings per token that a last-bit difference can turn: at top-8 of 256
    # a handful of the 32768 tokens is expected, at top-1 and top-2 none or one
    assert flips <= (2 if k <= 2 else 24)
    if flips:
        # the oracle once more, with the GPU's scores for exactly the near-tie tokens and its own for all others:
        # everything downstream of those few decisions must then agree as well
        diff = (idx_gpu != idx_cpu).any(axis=0).nonzero()[0]
        mixed = scores_cpu.numpy().copy()
        mixed[diff] = scores_gpu.cpu().numpy()[diff]
        c = O.extract_critical(mixed, k, cf)
        idx_cpu = np.stack(c.indices_s)
    np.testing.assert_array_equal(idx_gpu, idx_cpu)
    np.testing.assert_array_equal(r.counts.cpu().numpy(), c.counts)
    np.testing.assert_array_equal(r.loc.cpu().numpy(), np.stack(c.locations_s))
    np.testing.assert_array_equal(r.row.cpu().numpy(), c.rows(True))
    np.testing.assert_array_equal(r.kept_rows.cpu().numpy(), c.kept_rows)
    assert int(r.capacity.cpu()) == c.capacity
    assert rel_err(r.gates.cpu(), torch.from_numpy(np.stack(c.gates_s))) < 1e-5


def test_layer_gelu_exact_switch_and_gate_bias():
    m, x, ref = _build(600, 64, 8, 2, 128, torch.float32, gelu_bwd="exact",
                       gate_logit_bias=torch.log(torch.arange(1, 9, dtype=torch.float32) ** -1.2))
    res = _run_and_compare(m, x, ref, 2, 0.0, torch.float32, gelu_bwd="exact")
    loads = res.crit.counts.sum(0)
    assert loads.max() > 3 * max(loads.min(), 1)       # the Zipf bias really skews the load


def test_layer_config2_downsized_bf16_drops_overflow():
    print("layer config2 downsized", flush=True)
    m, x, ref = _build(2048, 256, 16, 1, 512, torch.bfloat16, seed=2)
    res = _run_and_compare(m, x, ref, 1, 1.25, torch.bfloat16)
    assert res.crit.capacity == 1 * int(1.25 * 128)


def test_unimem_bookkeeping_matches_model():
    """The pool's prefetch stack (C ABI) against the oracle's integer model, plus byte-exact slot contents."""
    from mole_amd import core
    from mole_amd.moe.layer import MOLEModule
    MOLEModule.reset_instances()
    F, M, pool = 16, 8, 6
    um = core.create_UniMem(0, pool, torch.float32, [[F, M], [F], [F, M], [M]])
    model = O.UniMemModel(pool)
    host = [torch.randn(10, F, M).pin_memory(), torch.randn(10, F).pin_memory(), torch.randn(10, F, M).pin_memory(),
            torch.randn(10, M).pin_memory()]
    for (layer, base, n) in [(0, 0, 2), (0, 2, 1), (1, 0, 2)]:
        um.prefetch(layer, host, base, n)
        model.prefetch(layer, n)
        assert um.view_pool_size() == model.view_pool_size and um.virtual_offset() == model.virtual_offset
    with pytest.raises(RuntimeError):
        um.prefetch(2, host, 0, 5)                 # does not fit the free slots
    assert um.fetch_top(0) == model.fetch_top(0) == 0
    assert um.fetch_top(1) == model.fetch_top(1) == 2
    p = um.fetch(host, 0, 0, 3, 2)                 # experts 0..2 of layer 1: 2 prefetched, 1 fetched now
    um.sync_tran()
    lo, _ = model.fetch_batch(0, 3)
    from mole_amd import _lib as L
    assert p[0] == um.slot_tensor(0, lo, 3)
    # read the slots back with the library's own row-copy kernel (identity permutation)
    dev = torch.empty(3 * F, M, device="cuda")
    ident = torch.arange(3 * F, dtype=torch.int32, device="cuda").view(1, -1)
    L.check(L.lib().mole_dispatch_fwd(L.ptr(p[0]), L.MOLE_F32, L.ptr(ident), 3 * F, M, 1, L.ptr(dev), L.stream()), "copy")
    torch.cuda.synchronize()
    assert torch.equal(dev.cpu().view(3, F, M), host[0][0:3])
    assert um.fetch_top(0) == model.fetch_top(0) == 3
    nbytes, ms = um.copy_stats()
    assert nbytes > 0 and ms >= 0.0
    MOLEModule.reset_instances()


def test_fast_assign_prefetch_matches_oracle():
    from mole_amd import core
    rng = np.random.default_rng(1)
    for _ in range(200):
        n = int(rng.integers(1, 8)); P = int(rng.integers(1, 12))
        Fv = [int(v) for v in rng.integers(0, 12, n)]; Ev = [int(v) for v in rng.integers(0, 9, n)]
        assert core.fast_assign_prefetch(P, Fv, Ev) == tuple(O.fast_assign_prefetch(P, Fv, Ev))


def test_layer_degenerate_inputs():
    """No tokens at all; fewer tokens than experts; every pair beyond the capacity dropped but one per expert."""
    from mole_amd.moe.layer import MOLEModule
    print("layer degenerate", flush=True)
    for dtype in (torch.float32, torch.bfloat16):
        m, x, ref = _build(0, 64, 4, 2, 128, dtype)
        xe = torch.zeros(0, 64, dtype=dtype, device="cuda", requires_grad=True)
        y = m(xe, capacity_factor=1.0)
        assert y.shape == (0, 64)
        y.sum().backward()
        assert xe.grad.shape == (0, 64)
        # 3 tokens, 8 experts, top-2: most experts receive nothing
        m, x, ref = _build(3, 64, 8, 2, 128, dtype, seed=5)
        _run_and_compare(m, x, ref, 2, 0.0, dtype)
        # capacity 1 row per expert and choice: nearly everything is dropped, dropped tokens output zeros
        m, x, ref = _build(200, 64, 4, 1, 128, dtype, seed=6)
        res = _run_and_compare(m, x, ref, 1, 0.02, dtype)
        assert res.crit.capacity == 1 and int(res.crit.kept_rows.sum()) <= 4
        # a capacity of zero drops everything: zeros out, zero gradients, no error
        m, x, ref = _build(50, 64, 4, 2, 128, dtype, seed=7)
        res = _run_and_compare(m, x, ref, 2, 0.001, dtype)
        assert res.crit.capacity == 0 and float(res.y.abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gradient_accumulation_over_micro_steps(dtype):
    """acc_step = 3 with two GPU-resident and four offloaded experts: after three backward passes of the same
    batch the gradient buffers hold g + g + g, summed in the parameter dtype in that order (static experts
    accumulate in the weight-gradient epilogue, core.cpp:457-514; offloaded ones into their pinned host arrays,
    core.cpp:77-103) - the first pass overwrites whatever the buffers held (lazy zero)."""
    from mole_amd import core
    S, M, E, k, Fd, d = 300, 64, 6, 2, 128, 4
    print(f"gradient accumulation {dtype}", flush=True)

    def step(m, x):
        xin = x.clone().requires_grad_(True)
        y = m(xin, capacity_factor=0.0)
        y.backward((2.0 * y.detach().float() / y.numel()).to(dtype) * 50.0)
        torch.cuda.synchronize()

    m0, x, _ = _build(S, M, E, k, Fd, dtype, d_experts=d, pool=4, ebatch=2, seed=3)
    step(m0, x)
    core.synchronize_tran()
    single = [g.clone() for g in _grads(m0, E)]
    assert all(float(g.abs().max()) > 0 for g in single)

    m1, x1, _ = _build(S, M, E, k, Fd, dtype, d_experts=d, pool=4, ebatch=2, seed=3, acc_step=3)
    for cp in (m1.FC1_W_CPU, m1.FC1_B_CPU, m1.FC2_W_CPU, m1.FC2_B_CPU):
        cp.all_tensors.grad_.fill_(7.0)          # stale contents that the first micro-step must overwrite
    for _ in range(3):
        step(m1, x1)
    core.synchronize_tran()
    s = E - d
    for name, g1, g3 in zip(("g_w1", "g_b1", "g_w2", "g_b2"), single, _grads(m1, E)):
        g = g1.to(dtype)
        want = ((g + g) + g).float()
        # offloaded experts: one rounding per addition, exactly reproducible
        assert torch.equal(g3[s:], want[s:]), f"{name} of the offloaded experts"
        # GPU-resident experts accumulate inside the product's epilogue (fp32 sum, rounded once per pass)
        assert rel_err(g3[:s], 3.0 * g1[:s]) < (1e-6 if dtype == torch.float32 else 1e-2), f"{name} of the resident experts"


def test_layer_state_round_trip():
    """get_layer_state / set_layer_state (the reference's checkpoint payload, layer.py:350-427): a second layer
    loaded from the first one's state computes the same output and holds the same gradients."""
    S, M, E, k, Fd, dtype = 300, 64, 6, 2, 128, torch.float32
    m1, x, _ = _build(S, M, E, k, Fd, dtype, d_experts=4, pool=4, ebatch=2, seed=1)
    xin = x.clone().requires_grad_(True)
    y1 = m1(xin, capacity_factor=1.0)
    y1.backward(torch.ones_like(y1) * 1e-2)
    torch.cuda.synchronize()
    state = m1.get_layer_state(True)
    assert len(state["experts"]) == E and len(state["grad"]) == E + 2
    assert all(t.device.type == "cpu" for ex in state["experts"] for t in ex)
    y1 = y1.detach().clone()
    # MOLEModule keeps one slot pool per process: the first layer goes away before the second is built
    m2, _, _ = _build(S, M, E, k, Fd, dtype, d_experts=4, pool=4, ebatch=2, seed=2)
    y_other = m2(x, capacity_factor=1.0).detach()
    assert not torch.allclose(y_other, y1)
    m2.set_layer_state(state, True)
    y2 = m2(x, capacity_factor=1.0).detach()
    assert torch.equal(y2, y1)
    back = m2.get_layer_state(True)
    for a, b in zip(state["experts"] + state["grad"][:E], back["experts"] + back["grad"][:E]):
        assert all(torch.equal(u, v) for u, v in zip(a, b))
    assert torch.equal(state["grad"][E], back["grad"][E]) and back["grad"][E + 1] is None
    m2.unset_lazy_zero()
    assert m2.FC1_W_CPU.all_tensors.grad_.lazy_zero is False
    m2.set_hybrid_adam_count(3)
    assert m2.MOLECore.hybrid_adam_count == 3


def _stack(n_layers, S, M, E, k, Fd, dtype, pool, ebatch, seed, **kw):
    from mole_amd.moe.layer import MOLEModule
    MOLEModule.reset_instances()
    torch.manual_seed(seed)
    dist = {"local_rank": 0, "world_size": 1, "rank": 0}
    return [MOLEModule(E, 0, M, Fd, pool, k, ebatch, dist, "gelu", 1, False, True, dtype=dtype, **kw) for _ in range(n_layers)]


def _run_stack(layers, x, prefetch):
    from mole_amd.utils.Uscheduler import UniScheduler
    xin = x.clone().requires_grad_(True)
    if prefetch:
        UniScheduler.prefetch_fwd()
    h = xin
    for m in layers:
        h = m(h, capacity_factor=0.0, prefetch=prefetch)
    h.backward(torch.ones_like(h) * 1e-2)
    torch.cuda.synchronize()
    from mole_amd import core
    core.synchronize_tran()
    grads = [t.grad_.clone() for m in layers for t in m.d_experts_param()]
    return h.detach().clone(), xin.grad.clone(), grads


@pytest.mark.parametrize("global_prefetch", [False, True])
def test_stack_with_planned_prefetch_matches_plain_run(global_prefetch):
    """Four offloaded layers share a pool smaller than two layers; the scheduler plans local and cross-layer
    prefetches from (made-up) layer times.  Prefetching moves copies, never results: output, input gradient and
    expert gradients equal the run without any prefetch bit for bit, and the prefetch stack ends empty."""
    from mole_amd import core
    from mole_amd.utils.Uscheduler import UniScheduler
    S, M, E, k, Fd, dtype = 200, 64, 4, 2, 128, torch.float32
    x = torch.randn(S, M, generator=torch.Generator().manual_seed(3)).cuda()
    layers = _stack(4, S, M, E, k, Fd, dtype, pool=6, ebatch=2, seed=11)
    want = _run_stack(layers, x, prefetch=False)
    layers = _stack(4, S, M, E, k, Fd, dtype, pool=6, ebatch=2, seed=11)
    plan = UniScheduler.set_prefetch_scheme(fwd_stat=[3.0, 1.0, 6.0, 2.0], bwd_stat=[2.0, 5.0, 0.0, 4.0], ftime=1.0,
                                            global_prefetch=global_prefetch)
    print("plan", plan, flush=True)
    assert any(p["local_fwd"] or p["global_fwd"] for p in plan)
    if global_prefetch:
        assert any(p["global_fwd"] or p["global_bwd"] for p in plan)
    for rep in range(2):                      # a second step starts from the state the first one left
        got = _run_stack(layers, x, prefetch=True)
        um = core.get_UniMem()
        assert um.virtual_offset() == 0 and um.view_pool_size() == 6
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        for a, b in zip(got[2], want[2]):
            assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_resident_experts_halve_the_traffic_and_follow_weight_updates(dtype):
    """Three offloaded layers and a pool with a slot for every expert: each layer keeps its own stretch of slots,
    the backward pass finds the experts where the forward pass left them (half the host-to-device bytes of a
    step), and the results equal, bit for bit, those of a stack that fetches for every pass.  Host weights changed
    between two passes are picked up: a pass never trusts what an earlier pass left behind."""
    from mole_amd import core
    S, M, E, k, Fd = 150, 64, 4, 2, 128
    es = 4 if dtype == torch.float32 else 2
    expert_bytes = (2 * Fd * M + Fd + M) * es
    x = torch.randn(S, M, generator=torch.Generator().manual_seed(5)).to(dtype).cuda()
    print(f"resident experts {dtype}", flush=True)
    layers = _stack(3, S, M, E, k, Fd, dtype, pool=12, ebatch=3, seed=21, resident=False)
    want = _run_stack(layers, x, prefetch=False)
    layers = _stack(3, S, M, E, k, Fd, dtype, pool=12, ebatch=3, seed=21)
    assert [m.MOLECore._home_base() for m in layers] == [0, 4, 8]
    for m in layers:
        m.set_prefetch(E, E)
    um = core.get_UniMem()
    for rep in range(2):
        um.copy_stats(); um.reuse_stats()
        got = _run_stack(layers, x, prefetch=bool(rep))
        nbytes, _ = um.copy_stats()
        active = sum(int((m.last_route.kept_rows > 0).sum()) for m in layers)
        assert nbytes == active * expert_bytes
        # every request for an expert that is already in place counts: without prefetch that is the backward pass's
        # request alone, with prefetch the passes' own requests find what their prefetches brought as well
        reused = um.reuse_stats()
        assert reused == active * expert_bytes * (3 if rep else 1)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        for a, b in zip(got[2], want[2]):
            assert torch.equal(a, b)
    # new host weights between two forward passes without a backward pass in between
    y_before = layers[0](x, capacity_factor=0.0).detach().clone()
    layers[0].FC2_W_CPU.all_tensors.mul_(2.0)
    layers[0].FC2_B_CPU.all_tensors.mul_(2.0)
    y_after = layers[0](x, capacity_factor=0.0).detach()
    assert rel_err(y_after, 2.0 * y_before.float()) < (1e-5 if dtype == torch.float32 else 2e-2)
