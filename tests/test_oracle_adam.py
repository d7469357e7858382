"""Pins oracle.adam_step (restating MOLE/cpp/define.hpp:543-579) against independent implementations:
torch.optim.Adam / AdamW over several steps in fp64, and hand-computed first-step values."""
import math

import numpy as np

import pytest
import torch

from oracle import moe_oracle as O


@pytest.mark.parametrize("adamW", [False, True])
@pytest.mark.parametrize("lam", [0.0, 0.1])
def test_adam_matches_torch_optim(adamW, lam):
    torch.manual_seed(3)
    beta1, beta2, lr, eps = 0.9, 0.999, 1e-2, 1e-8
    p0 = torch.randn(257, dtype=torch.float64)
    grads = [torch.randn(257, dtype=torch.float64) for _ in range(5)]
    # library optimizer
    q = torch.nn.Parameter(p0.clone())
    opt = (torch.optim.AdamW if adamW else torch.optim.Adam)([q], lr=lr, betas=(beta1, beta2), eps=eps, weight_decay=lam)
    # oracle
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step, g in enumerate(grads):
        q.grad = g.clone()
        opt.step()
        p, m, v = O.adam_step(p, m, v, g, beta1, beta2, step, lr, lam, eps, adamW, scalar=np.float64)
        assert torch.allclose(p, q.detach(), rtol=1e-12, atol=1e-12), f"step {step}"
    st = opt.state[q]
    assert torch.allclose(m, st["exp_avg"], rtol=1e-12, atol=0)
    assert torch.allclose(v, st["exp_avg_sq"], rtol=1e-12, atol=0)


def test_adam_first_step_closed_form():
    # zero moments, t = 1: m = (1-b1) g, v = (1-b2) g^2, so mt = g, vt = g^2 and p' = p - lr g / (|g| + eps)
    p = torch.tensor([1.0, -2.0, 0.5], dtype=torch.float64)
    g = torch.tensor([0.25, -4.0, 0.0], dtype=torch.float64)
    z = torch.zeros_like(p)
    pn, mn, vn = O.adam_step(p, z, z, g, 0.9, 0.999, 0, 0.1, 0.0, 1e-8, False, scalar=np.float64)
    assert torch.allclose(mn, 0.1 * g, rtol=1e-13, atol=0) and torch.allclose(vn, 0.001 * g * g, rtol=1e-13, atol=0)
    expect = p - 0.1 * g / (g.abs() + 1e-8)
    assert torch.allclose(pn, expect, rtol=1e-12, atol=0)
    # weight decay, plain Adam: the gradient becomes g + lam p; AdamW: p shrinks by (1 - lam lr) first
    pn2, mn2, _ = O.adam_step(p, z, z, g, 0.9, 0.999, 0, 0.1, 0.5, 1e-8, False, scalar=np.float64)
    g2 = g + 0.5 * p
    assert torch.allclose(mn2, 0.1 * g2, rtol=1e-13, atol=0)
    assert torch.allclose(pn2, p - 0.1 * g2 / (g2.abs() + 1e-8), rtol=1e-12, atol=0)
    pn3, _, _ = O.adam_step(p, z, z, g, 0.9, 0.999, 0, 0.1, 0.5, 1e-8, True, scalar=np.float64)
    assert torch.allclose(pn3, p * (1 - 0.05) - 0.1 * g / (g.abs() + 1e-8), rtol=1e-12, atol=0)


def test_adam_uses_stored_counter_plus_one():
    # the bias corrections use t = stored counter + 1 (define.hpp:547)
    p = torch.ones(4, dtype=torch.float64)
    g = torch.full((4,), 2.0, dtype=torch.float64)
    m = torch.full((4,), 0.3, dtype=torch.float64)
    v = torch.full((4,), 0.7, dtype=torch.float64)
    pn, mn, vn = O.adam_step(p, m, v, g, 0.9, 0.99, 9, 0.01, 0.0, 1e-8, False, scalar=np.float64)
    m1 = 0.9 * 0.3 + 0.1 * 2.0
    v1 = 0.99 * 0.7 + 0.01 * 4.0
    expect = 1.0 - 0.01 * (m1 / (1 - 0.9 ** 10)) / (math.sqrt(v1 / (1 - 0.99 ** 10)) + 1e-8)
    assert abs(pn[0].item() - expect) < 1e-14


def test_adam_single_precision_constants():
    """The default follows the reference's C++ floats: 1 - beta2 is formed in single precision, which moves the
    second-moment weight by about 1e-5 relative to the double-precision constant; everything else stays within
    single-precision rounding of the textbook update."""
    assert float(np.float32(1) - np.float32(0.999)) == pytest.approx(0.00099998713, rel=1e-6)
    torch.manual_seed(0)
    p, g = torch.randn(64, dtype=torch.float64), torch.randn(64, dtype=torch.float64)
    m, v = torch.randn(64, dtype=torch.float64) * 0.1, torch.rand(64, dtype=torch.float64) * 0.1
    a = O.adam_step(p, m, v, g, 0.9, 0.999, 4, 1e-2, 0.1, 1e-8, False)
    b = O.adam_step(p, m, v, g, 0.9, 0.999, 4, 1e-2, 0.1, 1e-8, False, scalar=np.float64)
    for x, y in zip(a, b):
        assert torch.allclose(x, y, rtol=2e-5, atol=1e-9)
    # the v update uses exactly the single-precision weight
    w = float(np.float32(1) - np.float32(0.999))
    g1 = g + float(np.float32(0.1)) * p
    assert torch.allclose(a[2], float(np.float32(0.999)) * v + w * g1 * g1, rtol=1e-14, atol=0)
