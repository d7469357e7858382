"""Builds oracle/_ref/libmole_ref.so: the reference's own `_fast_assign_prefetch` compiled from where it lies.

Test infrastructure, like everything under oracle/: only tests/, __graft_entry__ and bench.py's cpu_baseline leg may
use it, and only as the checker.

The reference's C++ cannot be built as a whole here (MOLE/cpp/core.cpp needs CUDA, cuBLAS, NCCL, ATen and pybind11
headers), but one function of the path is plain standard C++: `_fast_assign_prefetch` (MOLE/cpp/core.cpp:1301-1345,
<vector> / <tuple> / std::min only), the greedy cross-layer prefetch assignment behind
`core.fast_assign_prefetch`.  This recipe reads that function's text out of the reference file at build time, puts
the three standard headers in front of it and a C wrapper behind it, and hands the translation unit to g++ on its
standard input: nothing of the reference is copied into the repository or left on disk, only the shared library is
written, into oracle/_ref/ (git-ignored).  The oracle's Python restatement and the library's
`mole_fast_assign_prefetch` are then checked against it (tests/test_oracle_ref.py).

    python -m oracle.build_ref          (needs /root/reference; a no-op with a message when it is absent)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REF_FILE = os.environ.get("MOLE_REFERENCE_CORE", "/root/reference/MOLE/cpp/core.cpp")
OUT_DIR = os.path.join(HERE, "_ref")
LIB = os.path.join(OUT_DIR, "libmole_ref.so")
SIGNATURE = "_fast_assign_prefetch(int P, std::vector<int> F, std::vector<int> E)"

PREAMBLE = "#include <algorithm>\n#include <tuple>\n#include <vector>\n"
# flat C interface: F, E [n] in; lp_out [n]; gp_out: up to gp_cap triples (layer, later_layer, count) in the order the
# reference appends them; returns the number of triples, or -1 when gp_cap is too small
WRAPPER = r'''
extern "C" int ref_fast_assign_prefetch(int P, const int *F, const int *E, int n, int *lp_out, int *gp_out, int gp_cap) {
    std::vector<int> Fv(F, F + n), Ev(E, E + n);
    auto res = _fast_assign_prefetch(P, Fv, Ev);
    const auto &gp = std::get<0>(res);
    const auto &lp = std::get<1>(res);
    for (int i = 0; i < n; ++i) lp_out[i] = lp[i];
    int m = 0;
    for (int i = 0; i < n; ++i)
        for (const auto &pair : gp[i]) {
            if (m >= gp_cap) return -1;
            gp_out[3 * m] = i; gp_out[3 * m + 1] = pair[0]; gp_out[3 * m + 2] = pair[1];
            ++m;
        }
    return m;
}
'''


def _function_text(path: str) -> str:
    """The function's definition, from the line of its signature to the brace that closes its body."""
    lines = open(path, encoding="utf-8", errors="replace").read().splitlines()
    start = next((i for i, l in enumerate(lines) if SIGNATURE in l), None)
    if start is None:
        raise RuntimeError(f"{path}: no definition of _fast_assign_prefetch found")
    depth, seen_open, out = 0, False, []
    for l in lines[start:]:
        out.append(l)
        depth += l.count("{") - l.count("}")
        seen_open = seen_open or "{" in l
        if seen_open and depth == 0:
            return "\n".join(out) + "\n"
    raise RuntimeError(f"{path}: unbalanced braces after the signature of _fast_assign_prefetch")


def build(verbose: bool = False):
    """Returns the library's path, or None when the reference is not there (the GPU box: the prebuilt file travels)."""
    if not os.path.exists(REF_FILE):
        if verbose:
            print(f"oracle/_ref: {REF_FILE} not present, nothing built", file=sys.stderr)
        return LIB if os.path.exists(LIB) else None
    os.makedirs(OUT_DIR, exist_ok=True)
    unit = PREAMBLE + _function_text(REF_FILE) + WRAPPER
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-x", "c++", "-", "-o", LIB]
    r = subprocess.run(cmd, input=unit, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("g++ failed on the reference's _fast_assign_prefetch:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
