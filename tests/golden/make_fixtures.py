#!/usr/bin/env python3
"""Writes the golden fixtures of the MoE-layer path: small seeded inputs with the outputs the CPU
oracle gives for them.  Run from the repository root:  python tests/golden/make_fixtures.py

The reference holds no golden vectors, known-answer tests or fixtures for this path (its tests/
directory has none and tutel, which owns routing and dispatch, is absent), so these vectors come
from the oracle, after tests/test_oracle_*.py have pinned it against brute force, closed forms and
torch autograd.  They freeze the oracle's answers: a later edit of the oracle or of the HIP path
that changes a routing decision or a gradient shows up against data that does not move with it.

  routing_cases.npz   scores -> idx, loc, gates, counts, kept_rows, offsets, capacity, row (both layouts), l_aux
                      for hand-made tie / overflow / degenerate cases and seeded Zipf-skewed cases
  layer_small.npz     one fp32 layer (S 96, M 32, E 4, top-2, F 64, capacity factor 1.0, both GELU backward
                      variants): inputs, y, dx, dwg and the four expert gradients
  MOLE_states_tiny.pt a checkpoint file in the layout UniScheduler.save_states writes in the reference
                      (MOLE/utils/Uscheduler.py:67-75, MOLE/moe/layer.py:397-427): [model_state, optim_state],
                      model_state = one {"gate", "experts", "grad"} dict per layer, here the one layer of
                      layer_small.npz with the oracle's gradients, laid out by hand from those arrays
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def routing_cases():
    g = torch.Generator().manual_seed(1234)
    cases = {}

    def zipf(S, E):
        logits = torch.randn(S, E, generator=g)
        logits += torch.log(torch.arange(1, E + 1, dtype=torch.float32) ** -1.2)[torch.randperm(E, generator=g)]
        return torch.softmax(logits, dim=-1)

    # hand-made: every score equal (pure tie-breaking), duplicated columns, one hot expert that overflows
    cases["all_equal"] = (torch.full((37, 8), 0.125), 3, 1.0, True, 1)
    s = zipf(64, 8); s[:, 7] = s[:, 0]; s[::3, 1] = s[::3, 2]
    cases["dup_columns"] = (s, 4, 0.0, True, 1)
    s = torch.full((50, 4), 0.1); s[:, 2] = 0.7
    cases["one_hot_expert_overflow"] = (s, 1, 1.25, True, 1)
    cases["single_token_single_expert"] = (torch.ones(1, 1), 1, 1.0, True, 1)
    cases["zipf_top2_cf1"] = (zipf(200, 8), 2, 1.0, True, 1)
    cases["zipf_top1_cf125"] = (zipf(333, 16), 1, 1.25, True, 1)
    cases["zipf_top8_nodrop"] = (zipf(150, 32), 8, 0.0, True, 1)
    cases["zipf_negcf_unnormalised_aligned"] = (zipf(257, 8), 2, -0.5, False, 8)
    out = {"names": np.array(sorted(cases))}
    for name, (scores, k, cf, normalize, align) in cases.items():
        c = O.extract_critical(scores.numpy(), k, cf, normalize, align)
        out[f"{name}/scores"] = scores.numpy()
        out[f"{name}/params"] = np.array([k, cf, int(normalize), align], dtype=np.float64)
        out[f"{name}/idx"] = np.stack(c.indices_s)
        out[f"{name}/loc"] = np.stack(c.locations_s)
        out[f"{name}/gates"] = np.stack(c.gates_s)
        out[f"{name}/counts"] = c.counts
        out[f"{name}/kept_rows"] = c.kept_rows
        out[f"{name}/offsets"] = c.offsets
        out[f"{name}/capacity"] = np.array(c.capacity, dtype=np.int32)
        out[f"{name}/row_ragged"] = c.rows(True)
        out[f"{name}/row_padded"] = c.rows(False)
        out[f"{name}/l_aux"] = np.array(c.l_aux, dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "routing_cases.npz"), **out)


def layer_small():
    g = torch.Generator().manual_seed(7)
    S, M, E, k, F = 96, 32, 4, 2, 64
    x = torch.randn(S, M, generator=g)
    wg = torch.randn(E, M, generator=g) * 0.3
    w1, b1 = torch.randn(E, F, M, generator=g) * 0.2, torch.randn(E, F, generator=g) * 0.2
    w2, b2 = torch.randn(E, F, M, generator=g) * 0.2, torch.randn(E, M, generator=g) * 0.2
    dy = torch.randn(S, M, generator=g)
    out = dict(x=x, wg=wg, w1=w1, b1=b1, w2=w2, b2=b2, dy=dy, params=np.array([k, 1.0]))
    for variant in ("tanh", "exact"):
        r = O.moe_layer(x, wg, w1, b1, w2, b2, k, 1.0, dy=dy, gelu_bwd=variant)
        if variant == "tanh":
            out.update(scores=r.scores, y=r.y, row=r.crit.rows(True), capacity=np.array(r.crit.capacity))
        for n in ("dx", "dwg", "g_w1", "g_b1", "g_w2", "g_b2"):
            out[f"{variant}/{n}"] = getattr(r, n)
    out = {k_: (v.numpy() if isinstance(v, torch.Tensor) else v) for k_, v in out.items()}
    np.savez_compressed(os.path.join(HERE, "layer_small.npz"), **out)


def states_tiny():
    z = np.load(os.path.join(HERE, "layer_small.npz"))
    t = lambda name: torch.from_numpy(z[name]).clone()
    E = z["w1"].shape[0]
    experts = [[t("w1")[e], t("b1")[e], t("w2")[e], t("b2")[e]] for e in range(E)]
    grads = [[t("tanh/g_w1")[e], t("tanh/g_b1")[e], t("tanh/g_w2")[e], t("tanh/g_b2")[e]] for e in range(E)]
    grads += [t("tanh/dwg"), None]                  # the gate's weight gradient, then its (absent) bias gradient
    layer = {"gate": [t("wg"), None], "experts": experts, "grad": grads}
    optim_state = [None, None]                      # [expert_state, gate_state] of an optimizer that has not stepped
    torch.save([[layer], optim_state], os.path.join(HERE, "MOLE_states_tiny.pt"))


if __name__ == "__main__":
    routing_cases()
    layer_small()
    states_tiny()
    for f in ("routing_cases.npz", "layer_small.npz", "MOLE_states_tiny.pt"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
