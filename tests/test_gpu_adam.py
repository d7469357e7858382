"""The fused Adam kernel against the CPU oracle, and the in-pipeline update of offloaded experts
(parameters, moments and gradients travelling between pinned host memory and the GPU) against the
oracle applied to the gradients of a plain backward pass."""
import pytest
import torch

from oracle import moe_oracle as O
from tests.test_gpu_layer import _build
from tests.util import rel_err

pytestmark = pytest.mark.gpu

HYPER = dict(beta1=0.9, beta2=0.999, lr=1e-2, eps=1e-8)


@pytest.mark.parametrize("adamW", [False, True])
@pytest.mark.parametrize("n", [1, 5, 1027, 8 * 256 * 3, (1 << 20) + 3])
def test_adam_kernel_fp32(n, adamW):
    from mole_amd import hip_ops as H
    print(f"adam fp32 n={n} adamW={adamW}", flush=True)
    g_ = torch.Generator().manual_seed(n)
    p, g = torch.randn(n, generator=g_), torch.randn(n, generator=g_)
    m, v = torch.randn(n, generator=g_) * 0.1, torch.rand(n, generator=g_) * 0.1
    pe, me, ve = O.adam_step(p, m, v, g, HYPER["beta1"], HYPER["beta2"], 6, HYPER["lr"], 0.1, HYPER["eps"], adamW)
    pd, gd, md, vd = p.cuda(), g.cuda(), m.cuda(), v.cuda()
    out = torch.empty_like(pd)
    H.adam_step(pd, gd, md, vd, HYPER["beta1"], HYPER["beta2"], 7, HYPER["lr"], 0.1, HYPER["eps"], adamW, p_out=out)
    torch.cuda.synchronize()
    assert torch.equal(pd.cpu(), p), "p must stay untouched when p_out is a separate buffer"
    # fp32 elementwise arithmetic in the same order: a few ulp at most
    assert torch.allclose(out.cpu(), pe, rtol=2e-6, atol=1e-7)
    assert torch.allclose(md.cpu(), me, rtol=2e-6, atol=1e-9)
    assert torch.allclose(vd.cpu(), ve, rtol=2e-6, atol=1e-9)
    # in place: same result
    md2, vd2 = m.cuda(), v.cuda()
    H.adam_step(pd, gd, md2, vd2, HYPER["beta1"], HYPER["beta2"], 7, HYPER["lr"], 0.1, HYPER["eps"], adamW)
    torch.cuda.synchronize()
    assert torch.equal(pd, out) and torch.equal(md2, md) and torch.equal(vd2, vd)


@pytest.mark.parametrize("adamW", [False, True])
@pytest.mark.parametrize("n", [3, 8 * 256 + 5, (1 << 19) + 9])
def test_adam_kernel_bf16(n, adamW):
    from mole_amd import hip_ops as H
    print(f"adam bf16 n={n} adamW={adamW}", flush=True)
    g_ = torch.Generator().manual_seed(n)
    p, g = torch.randn(n, generator=g_).bfloat16(), (torch.randn(n, generator=g_) * 0.5).bfloat16()
    m, v = torch.randn(n, generator=g_) * 0.1, torch.rand(n, generator=g_) * 0.1
    pe, me, ve = O.adam_step(p.float(), m, v, g.float(), 0.9, 0.99, 0, 1e-2, 0.05, 1e-8, adamW)
    pd, gd, md, vd = p.cuda(), g.cuda(), m.cuda(), v.cuda()
    H.adam_step(pd, gd, md, vd, 0.9, 0.99, 1, 1e-2, 0.05, 1e-8, adamW)
    torch.cuda.synchronize()
    assert torch.allclose(md.cpu(), me, rtol=2e-6, atol=1e-9)
    assert torch.allclose(vd.cpu(), ve, rtol=2e-6, atol=1e-9)
    # the fp32 result rounded to bf16: equal except where a last-bit difference in fp32 flips the rounding
    expect = pe.bfloat16()
    got = pd.cpu()
    assert (got != expect).float().mean().item() < 1e-3
    assert torch.allclose(got.float(), pe, rtol=2 ** -8, atol=1e-6)


def test_adam_rejects_bad_arguments():
    from mole_amd import hip_ops as H
    p = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError, match="t=0"):
        H.adam_step(p, p.clone(), p.clone(), p.clone(), 0.9, 0.999, 0, 1e-3, 0.0, 1e-8, False)
    with pytest.raises(RuntimeError, match="below 1"):
        H.adam_step(p, p.clone(), p.clone(), p.clone(), 1.0, 0.999, 1, 1e-3, 0.0, 1e-8, False)
    with pytest.raises(RuntimeError, match="fp32"):
        H.adam_step(p, p.clone(), p.clone().bfloat16(), p.clone(), 0.9, 0.999, 1, 1e-3, 0.0, 1e-8, False)


def _cpu_params(m):
    return [cp.all_tensors for cp in (m.FC1_W_CPU, m.FC1_B_CPU, m.FC2_W_CPU, m.FC2_B_CPU)]


def _step(m, x, dtype):
    x = x.clone().requires_grad_(True)
    y = m(x, capacity_factor=0.0)
    y.backward((2.0 * y.detach().float() / y.numel()).to(dtype) * 100.0)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("adamW,hybrid,acc_step", [(False, -1, 1), (True, -1, 1), (False, 3, 1), (True, -1, 2), (False, 4, 2)])
def test_pipeline_adam_offloaded_experts(adamW, hybrid, acc_step, dtype):
    """6 offloaded experts through a 3-slot pool, two per batch: after the backward pass their host
    parameters and moments hold the Adam step of the pass's gradients."""
    print(f"pipeline adam adamW={adamW} hybrid={hybrid} acc_step={acc_step} {dtype}", flush=True)
    from mole_amd import core
    S, M, E, k, Fd, d = 400, 64, 8, 2, 128, 6
    # gradients of one plain backward pass
    m0, x, _ = _build(S, M, E, k, Fd, dtype, d_experts=d, pool=3, ebatch=2)
    _step(m0, x, dtype)
    core.synchronize_tran()
    grads = [t.grad_.clone().float() for t in _cpu_params(m0)]
    p_start = [t.clone() for t in _cpu_params(m0)]

    m1, x1, _ = _build(S, M, E, k, Fd, dtype, d_experts=d, pool=3, ebatch=2, acc_step=acc_step, adv_adam=True)
    g_ = torch.Generator().manual_seed(11)
    for t in _cpu_params(m1):
        assert t.momentum is not None and t.momentum.dtype == torch.float32
        t.momentum.copy_(torch.randn(t.shape, generator=g_) * 1e-3)
        t.variance.copy_(torch.rand(t.shape, generator=g_) * 1e-5)
    m_start = [t.momentum.clone() for t in _cpu_params(m1)]
    v_start = [t.variance.clone() for t in _cpu_params(m1)]
    lam = 0.1
    m1.MOLECore.set_adam(0.9, 0.999, 3, 1e-2, lam, 1e-8, adamW, hybrid)
    for _ in range(acc_step):                 # the update happens in the last micro-step
        _step(m1, x1, dtype)
    core.synchronize_tran()
    n_gpu = d if hybrid == -1 else hybrid
    for i, t in enumerate(_cpu_params(m1)):
        g_total = grads[i] * acc_step
        if dtype == torch.bfloat16 and acc_step > 1:
            g_total = (grads[i].bfloat16() + grads[i].bfloat16()).float()     # the sum is formed in bf16 on the GPU
        pe, me, ve = O.adam_step(p_start[i].float()[:n_gpu], m_start[i][:n_gpu], v_start[i][:n_gpu], g_total[:n_gpu],
                                 0.9, 0.999, 3, 1e-2, lam, 1e-8, adamW)
        assert torch.allclose(t.momentum[:n_gpu], me, rtol=1e-4, atol=1e-7), f"momentum of parameter {i}"
        assert torch.allclose(t.variance[:n_gpu], ve, rtol=1e-4, atol=1e-9), f"variance of parameter {i}"
        assert rel_err(t[:n_gpu].float(), pe) < (1e-5 if dtype == torch.float32 else 4e-3), f"parameter {i}"
        assert not torch.equal(t[:n_gpu], p_start[i][:n_gpu])
        # experts past the GPU-updated prefix: untouched parameters and moments, gradients on the host
        assert torch.equal(t[n_gpu:], p_start[i][n_gpu:])
        assert torch.equal(t.momentum[n_gpu:], m_start[i][n_gpu:])
        if n_gpu < d:
            assert rel_err(t.grad_[n_gpu:].float(), g_total[n_gpu:]) < (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S", [400, 5])
@pytest.mark.parametrize("adamW,hybrid,acc_step", [(False, -1, 1), (False, 3, 1), (True, -1, 2), (False, 4, 2)])
def test_pipeline_adam_with_home_slots_equals_the_stack_run(adamW, hybrid, acc_step, S, dtype):
    """A pool with a slot for every offloaded expert (each expert keeps a slot of its own from the forward to the
    backward pass, the update reads the parameters there) against a pool of 3 slots recycled through the prefetch
    stack: host parameters, moments and gradients are equal bit for bit.  hybrid = 3 cuts a chunk of two experts in
    the middle; with 5 tokens most experts get no row (their gradient is zero, the optimizer still moves them)."""
    print(f"pipeline adam home slots adamW={adamW} hybrid={hybrid} acc_step={acc_step} S={S} {dtype}", flush=True)
    from mole_amd import core
    M, E, k, Fd, d = 64, 8, 2, 128, 6

    def run(pool):
        m, x, _ = _build(S, M, E, k, Fd, dtype, d_experts=d, pool=pool, ebatch=2, acc_step=acc_step, adv_adam=True)
        assert (m.MOLECore._home_base() is not None) == (pool >= d)
        g_ = torch.Generator().manual_seed(11)
        for t in _cpu_params(m):
            t.momentum.copy_(torch.randn(t.shape, generator=g_) * 1e-3)
            t.variance.copy_(torch.rand(t.shape, generator=g_) * 1e-5)
            t.grad_.fill_(3.0)               # stale contents: the first micro-step overwrites them
        m.MOLECore.set_adam(0.9, 0.999, 3, 1e-2, 0.1, 1e-8, adamW, hybrid)
        for _ in range(acc_step):
            _step(m, x, dtype)
        core.synchronize_tran()
        out = []
        if S == 5:
            # experts without rows: their gradient is exactly zero, so the update is the Adam step of a zero
            # gradient from the moments set above (the weight-gradient kernel writes zeros for an expert without rows)
            idle = [e for e in range(d) if int(m.last_route.kept_rows[E - d + e]) == 0 and (hybrid == -1 or e < hybrid)]
            assert idle
            p0 = _cpu_params_initial(S, M, E, k, Fd, dtype, d, keep=m)
            g_ = torch.Generator().manual_seed(11)
            for t, p_init in zip(_cpu_params(m), p0):
                m_init = torch.randn(t.shape, generator=g_) * 1e-3
                v_init = torch.rand(t.shape, generator=g_) * 1e-5
                pe, me, ve = O.adam_step(p_init.float()[idle], m_init[idle], v_init[idle], torch.zeros_like(m_init[idle]),
                                         0.9, 0.999, 3, 1e-2, 0.1, 1e-8, adamW)
                assert torch.allclose(t.momentum[idle], me, rtol=1e-5, atol=1e-9)
                assert torch.allclose(t.variance[idle], ve, rtol=1e-5, atol=1e-12)
                assert rel_err(t[idle].float(), pe) < (1e-5 if dtype == torch.float32 else 4e-3)
        for t in _cpu_params(m):
            out += [t.clone(), t.momentum.clone(), t.variance.clone(), t.grad_.clone()]
        return out

    want = run(3)
    got = run(d)
    names = [f"{p} {w}" for p in ("w1", "b1", "w2", "b2") for w in ("parameter", "momentum", "variance", "gradient")]
    n_gpu = d if hybrid == -1 else hybrid
    for name, a, b in zip(names, got, want):
        if name.endswith("gradient"):
            # experts updated on the GPU keep whatever their host gradient array held (the update consumed the
            # gradient on the device); those past the prefix hold the step's gradient
            a, b = a[n_gpu:], b[n_gpu:]
        assert torch.equal(a, b), name


def _cpu_params_initial(S, M, E, k, Fd, dtype, d, keep):
    """the offloaded parameters as _build sets them for this seed (drawn again on the host; `keep` is the live
    layer, whose pool must not be torn down)"""
    g = torch.Generator().manual_seed(0)
    torch.randn(S, M, generator=g); torch.randn(E, M, generator=g)
    w1, b1 = torch.randn(E, Fd, M, generator=g) * 0.02, torch.randn(E, Fd, generator=g) * 0.02
    w2, b2 = torch.randn(E, Fd, M, generator=g) * 0.02, torch.randn(E, M, generator=g) * 0.02
    return [t[E - d:].to(dtype) for t in (w1, b1, w2, b2)]
