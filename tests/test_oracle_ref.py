"""The reference's own `_fast_assign_prefetch` (MOLE/cpp/core.cpp:1301-1345), compiled by oracle/build_ref.py into
oracle/_ref/libmole_ref.so, against the oracle's restatement of it and against the library's host-side
`mole_fast_assign_prefetch`: exhaustively on small inputs and on random larger ones."""
import ctypes
import itertools
import os

import numpy as np
import pytest

from oracle import moe_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libmole_ref.so")


def _ref():
    if not os.path.exists(REF_LIB):
        from oracle import build_ref
        if build_ref.build() is None:
            pytest.skip("oracle/_ref/libmole_ref.so is not built and the reference is not here to build it from")
    lib = ctypes.CDLL(REF_LIB)
    lib.ref_fast_assign_prefetch.restype = ctypes.c_int

    def call(P, Fv, Ev):
        n = len(Ev)
        arr = lambda v: (ctypes.c_int * max(len(v), 1))(*v)
        lp = (ctypes.c_int * max(n, 1))()
        cap = 4 * n * n + 4
        gp = (ctypes.c_int * (3 * cap))()
        m = lib.ref_fast_assign_prefetch(P, arr(Fv), arr(Ev), n, lp, gp, cap)
        assert m >= 0
        scheme = [[] for _ in range(n)]
        for t in range(m):
            scheme[gp[3 * t]].append([gp[3 * t + 1], gp[3 * t + 2]])
        return scheme, [lp[i] for i in range(n)]
    return call


def test_oracle_planner_equals_the_compiled_reference_function():
    ref = _ref()
    cases = 0
    for n in (1, 2, 3):                                   # every input with small entries
        for P in range(0, 6):
            for Fv in itertools.product(range(0, 5), repeat=n):
                for Ev in itertools.product(range(0, 4), repeat=n):
                    gp, lp = ref(P, list(Fv), list(Ev))
                    ogp, olp = O.fast_assign_prefetch(P, list(Fv), list(Ev))
                    assert (gp, lp) == ([list(map(list, g)) for g in ogp], list(olp)), (P, Fv, Ev)
                    cases += 1
    rng = np.random.default_rng(0)
    for _ in range(3000):                                 # deeper stacks, pools up to a node's worth of slots
        n = int(rng.integers(1, 14)); P = int(rng.integers(0, 100))
        Fv = [int(v) for v in rng.integers(0, 80, n)]; Ev = [int(v) for v in rng.integers(0, 40, n)]
        gp, lp = ref(P, Fv, Ev)
        ogp, olp = O.fast_assign_prefetch(P, Fv, Ev)
        assert (gp, lp) == ([list(map(list, g)) for g in ogp], list(olp)), (P, Fv, Ev)
        cases += 1
    assert cases > 50000


def test_library_planner_equals_the_compiled_reference_function():
    from mole_amd import core
    ref = _ref()
    rng = np.random.default_rng(1)
    for _ in range(2000):
        n = int(rng.integers(1, 14)); P = int(rng.integers(0, 100))
        Fv = [int(v) for v in rng.integers(0, 80, n)]; Ev = [int(v) for v in rng.integers(0, 40, n)]
        gp, lp = ref(P, Fv, Ev)
        got_gp, got_lp = core.fast_assign_prefetch(P, Fv, Ev)
        assert ([list(map(list, g)) for g in got_gp], list(got_lp)) == (gp, lp), (P, Fv, Ev)
