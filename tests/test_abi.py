"""CPU-side checks of the boundary: the shared library loads, exports every symbol include/mole_hip.h
declares, rejects bad arguments without touching a GPU, and the host-only planner matches the oracle."""
import os
import re

import numpy as np
import pytest

from oracle import moe_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    """every function declared in include/*.h: the boundary (mole_hip.h) and the measurement aids (mole_hip_probe.h)"""
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if header.endswith(".h"):
            text = open(os.path.join(ROOT, "include", header)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b(mole_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_boundary_header_holds_no_measurement_aids():
    text = open(os.path.join(ROOT, "include", "mole_hip.h")).read()
    assert "mole_probe" not in text


def test_library_exports_every_declared_symbol():
    from mole_amd import _lib as L
    lib = L.lib()
    declared = _declared()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in mole_hip.h but not exported"
    assert sorted(L.EXPORTS) == declared
    assert lib.mole_version() >= 100


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 (no C++ types, no torch types), and a C program
    that calls an entry point links against the shared library and runs without a GPU."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc here")
    inc = os.path.join(ROOT, "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c",
                    os.path.join(inc, "mole_hip.h")], check=True)
    src = tmp_path / "caller.c"
    src.write_text('#include <stdio.h>\n#include "mole_hip.h"\n'
                   'int main(void) {\n'
                   '    /* bad arguments are refused on the host, with a message, before anything touches a GPU */\n'
                   '    int rc = mole_dispatch_fwd(NULL, MOLE_BF16, NULL, 8, 12, 2, NULL, NULL);\n'
                   '    printf("%d %d %s\\n", mole_version(), rc, mole_last_error_string());\n'
                   '    return rc == -1 ? 0 : 1;\n}\n')
    from mole_amd import _lib as L
    libdir = os.path.dirname(L.LIB_PATH)
    exe = tmp_path / "caller"
    subprocess.run([gcc, "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-l:" + os.path.basename(L.LIB_PATH),
                    "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 2)
    assert int(out[0]) >= 100 and int(out[1]) == -1 and "M" in out[2]


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


def test_every_entry_point_rejects_bad_arguments_on_the_host():
    """Shape, dtype, alignment and null checks come before any launch: each call below returns a negative library
    code and leaves a message that names the entry point, on a machine without a GPU."""
    import ctypes
    from mole_amd import _lib as L
    lib = L.lib()
    P = ctypes.c_void_p
    bad16 = P(8)        # a non-null, misaligned "pointer" that is never dereferenced
    ok = P(4096)
    cases = [
        ("mole_softmax_fwd", lambda: lib.mole_softmax_fwd(None, None, 10, 0, None, None)),
        ("mole_gate_fwd", lambda: lib.mole_gate_fwd(ok, L.MOLE_F32, ok, None, 10, 64, 128, ok, None)),      # fp32: E <= 32
        ("mole_gate_fwd", lambda: lib.mole_gate_fwd(bad16, L.MOLE_F32, ok, None, 10, 8, 128, ok, None)),    # fp32: alignment
        ("mole_gate_fwd", lambda: lib.mole_gate_fwd(ok, L.MOLE_BF16, ok, None, 10, 8, 100, ok, None)),
        ("mole_softmax_bwd", lambda: lib.mole_softmax_bwd(ok, ok, 10, 0, ok, None)),
        ("mole_gate_bwd", lambda: lib.mole_gate_bwd(ok, ok, ok, 10, 4, 5, 1, 1, None, None, ok, None)),
        ("mole_gate_bwd", lambda: lib.mole_gate_bwd(ok, ok, ok, 10, 4, 2, 1, 1, ok, None, ok, None)),      # counts0 without d_l_aux
        ("mole_gate_wgrad", lambda: lib.mole_gate_wgrad(ok, ok, L.MOLE_F32, 10, 64, 128, ok, ok, 1 << 30, None)),
        ("mole_gate_wgrad", lambda: lib.mole_gate_wgrad(ok, ok, L.MOLE_BF16, 10, 8, 128, ok, ok, 16, None)),
        ("mole_route", lambda: lib.mole_route(ok, 10, 4, 5, 1.0, 1, 1, 1, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, 1 << 20, None)),
        ("mole_route", lambda: lib.mole_route(ok, 10, 4, 2, 1.0, 1, 1, 1, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, 8, None)),
        ("mole_dispatch_fwd", lambda: lib.mole_dispatch_fwd(bad16, L.MOLE_F32, ok, 8, 16, 2, ok, None)),
        ("mole_dispatch_bwd", lambda: lib.mole_dispatch_bwd(ok, L.MOLE_F32, ok, 8, 16, 2, ok, None, 4, None, ok, None)),
        ("mole_combine_fwd", lambda: lib.mole_combine_fwd(ok, L.MOLE_BF16, ok, ok, 8, 12, 2, ok, None)),
        ("mole_combine_bwd", lambda: lib.mole_combine_bwd(None, ok, L.MOLE_F32, ok, ok, 8, 16, 2, ok, ok, None)),
        ("mole_zero_pad_rows", lambda: lib.mole_zero_pad_rows(ok, 9, ok, ok, 4, 16, None)),
        ("mole_ffn_fwd", lambda: lib.mole_ffn_fwd(ok, L.MOLE_BF16, ok, ok, 2, 16, 12, 16, ok, ok, ok, ok, ok, ok, ok, None)),
        ("mole_ffn_fwd", lambda: lib.mole_ffn_fwd(bad16, L.MOLE_F32, ok, ok, 2, 16, 16, 16, ok, ok, ok, ok, ok, ok, ok, None)),
        ("mole_ffn_bwd", lambda: lib.mole_ffn_bwd(ok, ok, ok, ok, 5, ok, ok, 2, 16, 16, 16, ok, ok, ok, ok, ok, ok, ok, ok, 0, 0, None)),
        ("mole_gemm_nt", lambda: lib.mole_gemm_nt(ok, ok, 4, 16, 16, 16, ok, None)),
        ("mole_gemm_nn", lambda: lib.mole_gemm_nn(ok, ok, 4, 16, 16, 16, ok, None)),
        ("mole_gemm_tn", lambda: lib.mole_gemm_tn(ok, ok, L.MOLE_F32, 16, 6, 16, ok, None)),                  # Mo % 4
        ("mole_adam_step", lambda: lib.mole_adam_step(ok, ok, ok, ok, ok, 64, L.MOLE_F32, 0.9, 0.999, 0, 1e-3, 0.0, 1e-8, 0, None)),
        ("mole_adam_step", lambda: lib.mole_adam_step(ok, bad16, ok, ok, ok, 64, L.MOLE_BF16, 0.9, 0.999, 1, 1e-3, 0.0, 1e-8, 0, None)),
        ("mole_adam_step", lambda: lib.mole_adam_step(ok, ok, ok, ok, ok, 64, L.MOLE_F32, 1.0, 0.999, 1, 1e-3, 0.0, 1e-8, 0, None)),
        ("mole_unimem_prefetch", lambda: lib.mole_unimem_prefetch(None, 0, None, 0, 1)),
        ("mole_unimem_fetch", lambda: lib.mole_unimem_fetch(None, None, 0, 0, 1, 0, None)),
        ("mole_unimem_prefetch_ids", lambda: lib.mole_unimem_prefetch_ids(None, 0, None, None, 1, 0)),
        ("mole_unimem_fetch_ids", lambda: lib.mole_unimem_fetch_ids(None, None, 0, None, 1, 0, 0, None)),
        ("mole_unimem_wait_slots", lambda: lib.mole_unimem_wait_slots(None, 0, 1, None)),
        ("mole_unimem_reserve", lambda: lib.mole_unimem_reserve(None, 0, 1, None)),
        ("mole_unimem_store_grads_ids", lambda: lib.mole_unimem_store_grads_ids(None, None, None, None, 1, None)),
        ("mole_unimem_zero_grads_ids", lambda: lib.mole_unimem_zero_grads_ids(None, None, None, 1)),
        ("mole_unimem_store_grads", lambda: lib.mole_unimem_store_grads(None, None, None, 0, 1, None)),
        ("mole_unimem_load_state", lambda: lib.mole_unimem_load_state(None, None, None, None, 1, 0, None)),
        ("mole_unimem_store_state", lambda: lib.mole_unimem_store_state(None, None, None, None, 1, None)),
        ("mole_unimem_sync_tran", lambda: lib.mole_unimem_sync_tran(None)),
        ("mole_fast_assign_prefetch", lambda: lib.mole_fast_assign_prefetch(4, None, None, 3, None, None, 0, None)),
    ]
    for name, call in cases:
        rc = call()
        assert rc < 0, f"{name}: expected a library error code, got {rc}"
        msg = L.last_error()
        assert name in msg, f"{name}: message does not name the entry point: {msg!r}"
