"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the oracle reproduces the committed vectors, and the hand-derivable cases among them equal what
the routing rules give on paper.  GPU: the HIP path, through the C ABI, reproduces the same vectors."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.util import rel_err

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INT_KEYS = ("idx", "loc", "counts", "kept_rows", "offsets", "capacity", "row_ragged", "row_padded")


def _routing():
    z = np.load(os.path.join(GOLD, "routing_cases.npz"))
    for name in z["names"]:
        name = str(name)
        k, cf, normalize, align = z[f"{name}/params"]
        yield name, z, int(k), float(cf), bool(normalize), int(align)


def test_oracle_reproduces_routing_fixtures():
    n = 0
    for name, z, k, cf, normalize, align in _routing():
        c = O.extract_critical(z[f"{name}/scores"], k, cf, normalize, align)
        got = dict(idx=np.stack(c.indices_s), loc=np.stack(c.locations_s), counts=c.counts, kept_rows=c.kept_rows,
                   offsets=c.offsets, capacity=np.array(c.capacity), row_ragged=c.rows(True), row_padded=c.rows(False))
        for key in INT_KEYS:
            np.testing.assert_array_equal(got[key], z[f"{name}/{key}"], err_msg=f"{name}/{key}")
        np.testing.assert_array_equal(np.stack(c.gates_s), z[f"{name}/gates"])
        assert abs(c.l_aux - float(z[f"{name}/l_aux"])) < 1e-6
        n += 1
    assert n == 8


def test_routing_fixtures_hand_derived_cases():
    z = np.load(os.path.join(GOLD, "routing_cases.npz"))
    # 37 tokens, 8 experts, every score 1/8, top-3, cf 1.0: ties go to experts 0,1,2 in that order; choice j only
    # ever names expert j, so a token's location is its own index; ceil(37/8) = 5 -> C = 3*5 = 15.
    i = np.arange(37)
    np.testing.assert_array_equal(z["all_equal/idx"], np.stack([np.full(37, j) for j in range(3)]))
    np.testing.assert_array_equal(z["all_equal/loc"], np.stack([i, i, i]))
    assert int(z["all_equal/capacity"]) == 15
    np.testing.assert_array_equal(z["all_equal/kept_rows"], [15, 15, 15, 0, 0, 0, 0, 0])
    np.testing.assert_array_equal(z["all_equal/offsets"], [0, 15, 30, 45, 45, 45, 45, 45, 45])
    np.testing.assert_array_equal(z["all_equal/row_ragged"], np.stack([np.where(i < 15, 15 * j + i, -1) for j in range(3)]))
    np.testing.assert_allclose(z["all_equal/gates"], 1.0 / 3.0, rtol=1e-6)
    # 50 tokens all preferring expert 2 of 4, top-1, cf 1.25: ceil(50/4) = 13, C = int(16.25) = 16; the first 16
    # tokens are kept, the rest dropped; a top-1 gate is the raw score.
    i = np.arange(50)
    name = "one_hot_expert_overflow"
    np.testing.assert_array_equal(z[f"{name}/idx"], np.full((1, 50), 2))
    np.testing.assert_array_equal(z[f"{name}/loc"], i[None])
    assert int(z[f"{name}/capacity"]) == 16
    np.testing.assert_array_equal(z[f"{name}/kept_rows"], [0, 0, 16, 0])
    np.testing.assert_array_equal(z[f"{name}/offsets"], [0, 0, 0, 16, 16])
    np.testing.assert_array_equal(z[f"{name}/row_ragged"], np.where(i < 16, i, -1)[None])
    np.testing.assert_array_equal(z[f"{name}/row_padded"], np.where(i < 16, 2 * 16 + i, -1)[None])
    np.testing.assert_array_equal(z[f"{name}/gates"], np.full((1, 50), np.float32(0.7)))
    name = "single_token_single_expert"
    assert z[f"{name}/row_ragged"].tolist() == [[0]] and int(z[f"{name}/capacity"]) == 1


def _layer():
    z = np.load(os.path.join(GOLD, "layer_small.npz"))
    t = {k: torch.from_numpy(z[k]) for k in ("x", "wg", "w1", "b1", "w2", "b2", "dy")}
    return z, t, int(z["params"][0]), float(z["params"][1])


def test_oracle_reproduces_layer_fixture():
    z, t, k, cf = _layer()
    for variant in ("tanh", "exact"):
        r = O.moe_layer(t["x"], t["wg"], t["w1"], t["b1"], t["w2"], t["b2"], k, cf, dy=t["dy"], gelu_bwd=variant)
        np.testing.assert_array_equal(r.crit.rows(True), z["row"])
        assert rel_err(r.y, torch.from_numpy(z["y"])) < 1e-6
        for n in ("dx", "dwg", "g_w1", "g_b1", "g_w2", "g_b2"):
            assert rel_err(getattr(r, n), torch.from_numpy(z[f"{variant}/{n}"])) < 1e-6, (variant, n)


@pytest.mark.gpu
def test_hip_route_reproduces_routing_fixtures():
    from mole_amd import hip_ops as H, _lib as L
    for name, z, k, cf, normalize, align in _routing():
        print(f"golden route {name}", flush=True)
        scores = torch.from_numpy(z[f"{name}/scores"]).cuda()
        for layout, key in ((L.LAYOUT_RAGGED, "row_ragged"), (L.LAYOUT_PADDED, "row_padded")):
            r = H.route(scores, k, cf, normalize, align, layout)
            np.testing.assert_array_equal(r.idx.cpu().numpy(), z[f"{name}/idx"])
            np.testing.assert_array_equal(r.loc.cpu().numpy(), z[f"{name}/loc"])
            np.testing.assert_array_equal(r.counts.cpu().numpy(), z[f"{name}/counts"])
            np.testing.assert_array_equal(r.kept_rows.cpu().numpy(), z[f"{name}/kept_rows"])
            assert int(r.capacity.cpu()) == int(z[f"{name}/capacity"])
            np.testing.assert_array_equal(r.row.cpu().numpy(), z[f"{name}/{key}"])
            np.testing.assert_array_equal(r.gates.cpu().numpy(), z[f"{name}/gates"])
            if layout == L.LAYOUT_RAGGED:
                np.testing.assert_array_equal(r.offsets.cpu().numpy(), z[f"{name}/offsets"])
            assert abs(float(r.l_aux.cpu()) - float(z[f"{name}/l_aux"])) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["tanh", "exact"])
def test_hip_layer_reproduces_layer_fixture(variant):
    from mole_amd.moe.layer import MOLEModule
    print(f"golden layer {variant}", flush=True)
    z, t, k, cf = _layer()
    E, F, M = t["w1"].shape
    MOLEModule.reset_instances()
    m = MOLEModule(0, E, M, F, -1, k, 4, {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", 1, False, False,
                   dtype=torch.float32, gelu_bwd=variant)
    with torch.no_grad():
        m.gate[0].linear.weight.copy_(t["wg"])
        for p, n in ((m.FC1_W_GPU, "w1"), (m.FC1_B_GPU, "b1"), (m.FC2_W_GPU, "w2"), (m.FC2_B_GPU, "b2")):
            p.all_tensors.copy_(t[n])
    x = t["x"].cuda().requires_grad_(True)
    y = m(x, capacity_factor=cf)
    y.backward(t["dy"].cuda())
    np.testing.assert_array_equal(m.last_route.row.cpu().numpy(), z["row"])
    assert rel_err(y, torch.from_numpy(z["y"])) < 1e-5
    assert rel_err(x.grad, torch.from_numpy(z[f"{variant}/dx"])) < 1e-5
    assert rel_err(m.gate[0].linear.weight.grad, torch.from_numpy(z[f"{variant}/dwg"])) < 1e-5
    for p, n in ((m.FC1_W_GPU, "g_w1"), (m.FC1_B_GPU, "g_b1"), (m.FC2_W_GPU, "g_w2"), (m.FC2_B_GPU, "g_b2")):
        assert rel_err(p.grad_tensors, torch.from_numpy(z[f"{variant}/{n}"])) < 1e-5, n


def test_checkpoint_fixture_has_the_reference_file_layout():
    """tests/golden/MOLE_states_tiny.pt: [model_state, optim_state] as UniScheduler.save_states writes it
    (MOLE/utils/Uscheduler.py:67-75), one {"gate", "experts", "grad"} dict per layer (MOLE/moe/layer.py:397-427),
    readable by a loader that executes nothing from the file, and holding the arrays of layer_small.npz."""
    all_state = torch.load(os.path.join(GOLD, "MOLE_states_tiny.pt"), map_location="cpu", weights_only=True)
    z = np.load(os.path.join(GOLD, "layer_small.npz"))
    assert isinstance(all_state, list) and len(all_state) == 2
    model_state, optim_state = all_state
    assert optim_state == [None, None] and len(model_state) == 1
    st = model_state[0]
    assert sorted(st) == ["experts", "gate", "grad"]
    E = z["w1"].shape[0]
    assert len(st["gate"]) == 2 and st["gate"][1] is None and np.array_equal(st["gate"][0].numpy(), z["wg"])
    assert len(st["experts"]) == E and len(st["grad"]) == E + 2 and st["grad"][E + 1] is None
    for e in range(E):
        for t, name in zip(st["experts"][e], ("w1", "b1", "w2", "b2")):
            assert np.array_equal(t.numpy(), z[name][e])
        for t, name in zip(st["grad"][e], ("g_w1", "g_b1", "g_w2", "g_b2")):
            assert np.array_equal(t.numpy(), z[f"tanh/{name}"][e])
    assert np.array_equal(st["grad"][E].numpy(), z["tanh/dwg"])
