"""CPU-side checks of the boundary: the shared library loads, exports every symbol include/mole_hip.h
declares, rejects bad arguments without touching a GPU, and the host-only planner matches the oracle."""
import os
import re

import numpy as np
import pytest

from oracle import moe_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mole_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mole_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from mole_amd import _lib as L
    lib = L.lib()
    declared = _declared()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in mole_hip.h but not exported"
    assert sorted(L.EXPORTS) == declared
    assert lib.mole_version() >= 100


def test_argument_validation_needs_no_gpu():
    from mole_amd import _lib as L
    lib = L.lib()
    assert lib.mole_route(None, 10, 0, 1, 1.0, 1, 1, 1, None, None, None, None, None, None, None, None, None, None, 0, None) == -1
    assert "E" in L.last_error()
    assert lib.mole_dispatch_fwd(None, 1, None, 8, 12, 2, None, None) == -1      # M not a multiple of 8 for bf16
    assert lib.mole_ffn_fwd(None, 7, None, None, 1, 0, 8, 8, None, None, None, None, None, None, None, None) == -1
    assert lib.mole_route_workspace_bytes(16384, 16, 1) > 0


def test_fast_assign_prefetch_host_planner():
    from mole_amd import core
    rng = np.random.default_rng(0)
    for _ in range(300):
        n = int(rng.integers(1, 8)); P = int(rng.integers(1, 12))
        Fv = [int(v) for v in rng.integers(0, 12, n)]; Ev = [int(v) for v in rng.integers(0, 9, n)]
        gp, lp = core.fast_assign_prefetch(P, Fv, Ev)
        want_gp, want_lp = O.fast_assign_prefetch(P, Fv, Ev)
        assert gp == want_gp and lp == want_lp


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "mole_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("the oracle", ""), f"{f} mentions the oracle package"
