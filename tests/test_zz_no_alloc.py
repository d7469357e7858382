"""mole_route_static, the routing entry point that allocates nothing (its scratch is a static device array inside
the library), against mole_route with a caller-provided workspace: every output bit for bit, on consecutive calls
that share the array - the second on a smaller input, so that anything the first call left behind would show -
and the size limit's error."""
import ctypes

import numpy as np
import pytest
import torch

from tests.util import zipf_scores

pytestmark = pytest.mark.gpu

OUTS = ("idx", "loc", "gates", "row", "counts", "kept", "offsets", "cap", "l_aux")


def _buffers(S, E, k):
    i32 = dict(dtype=torch.int32, device="cuda")
    f32 = dict(dtype=torch.float32, device="cuda")
    return dict(idx=torch.full((k, S), -7, **i32), loc=torch.full((k, S), -7, **i32), gates=torch.full((k, S), -7.0, **f32),
                row=torch.full((k, S), -7, **i32), counts=torch.full((k, E), -7, **i32), kept=torch.full((E,), -7, **i32),
                offsets=torch.full((E + 1,), -7, **i32), cap=torch.full((1,), -7, **i32), l_aux=torch.full((1,), -7.0, **f32))


def _route(static, scores, k, cf, layout):
    from mole_amd import _lib as L
    S, E = scores.shape
    b = _buffers(S, E, k)
    args = [L.ptr(scores), S, E, k, float(cf), 1, 1, layout] + [L.ptr(b[n]) for n in OUTS]
    if static:
        rc = L.lib().mole_route_static(*args, L.stream())
    else:
        nbytes = L.lib().mole_route_workspace_bytes(S, E, k)
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        rc = L.lib().mole_route(*args, L.ptr(ws), nbytes, L.stream())
    L.check(rc, "mole_route_static" if static else "mole_route")
    torch.cuda.synchronize()
    return {n: t.cpu().numpy() for n, t in b.items()}


def test_route_static_matches_route_on_consecutive_calls():
    from mole_amd import _lib as L
    assert L.lib().mole_route_static_max_bytes() == 8 << 20
    # a large call first, then smaller ones on the same scratch, then a large one again
    cases = [(32768, 256, 8, 0.0), (3000, 100, 4, -0.5), (16384, 16, 1, 1.25), (257, 8, 2, 0.5), (1, 1, 1, 1.0),
             (8192, 64, 2, 0.0), (4096, 8, 2, 1.0)]
    for n, (S, E, k, cf) in enumerate(cases):
        print(f"route_static S={S} E={E} k={k} cf={cf}", flush=True)
        assert L.lib().mole_route_workspace_bytes(S, E, k) <= 8 << 20
        scores = zipf_scores(S, E, seed=n, ties=(n % 2 == 1)).cuda()
        for layout in (L.LAYOUT_RAGGED, L.LAYOUT_PADDED):
            got = _route(True, scores, k, cf, layout)
            want = _route(False, scores, k, cf, layout)
            for name in OUTS:
                np.testing.assert_array_equal(got[name], want[name], err_msg=f"{name} of case {n}")


def test_route_static_allocates_nothing():
    """Device memory in use is the same before and after calls of the entry point (outputs allocated beforehand)."""
    from mole_amd import _lib as L
    S, E, k = 4096, 64, 2
    scores = zipf_scores(S, E, seed=3).cuda()
    b = _buffers(S, E, k)
    args = [L.ptr(scores), S, E, k, 0.0, 1, 1, L.LAYOUT_RAGGED] + [L.ptr(b[n]) for n in OUTS]
    L.check(L.lib().mole_route_static(*args, L.stream()), "mole_route_static")      # first call on the device: set-up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for _ in range(3):
        L.check(L.lib().mole_route_static(*args, L.stream()), "mole_route_static")
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and torch.cuda.memory_reserved() == reserved0


def test_route_static_rejects_what_does_not_fit():
    from mole_amd import _lib as L
    S, E, k = 200000, 512, 8
    assert L.lib().mole_route_workspace_bytes(S, E, k) > 8 << 20
    rc = L.lib().mole_route_static(None, S, E, k, 0.0, 1, 1, 1, *([None] * 9), None)
    assert rc == -2
    assert "mole_route_static" in L.last_error() and "scratch" in L.last_error()
