"""Builds MOLE/cpp/libmole_hip.so (gfx950 only) with hipcc, from the sources beside it: the native extension sits
where the reference keeps its own (MOLE/cpp).  `python -m mole_amd.build`."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CPP = os.path.join(ROOT, "MOLE", "cpp")
LIB = os.path.join(CPP, "libmole_hip.so")
SOURCES = ["error.cpp", "route.hip", "permute.hip", "ffn_gemm.hip", "gemm256.hip", "gemm_f32.hip", "adam.hip", "unimem.hip", "probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
         # keep the compiler from forming packed-fp32 VALU ops
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument",
         "-I" + os.path.join(ROOT, "include"), "-I" + CPP]
# MOLE_TUNING=1 in the environment of the build adds the tile shapes, launch orders and K-loop ablations that were
# measured against the defaults (selected at run time by MOLE_TMB, MOLE_MFAST, ...: see MOLE/cpp/gemm256.hip)
if os.environ.get("MOLE_TUNING"):
    FLAGS.append("-DMOLE_TUNING")


def _compile(src: str) -> str:
    obj = os.path.join(CPP, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CPP, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                     if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{msgs}")
    if msgs:
        print(msgs, file=sys.stderr)
    return obj


def build(verbose: bool = False) -> str:
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CPP, s))]
    missing = sorted(set(SOURCES) - set(srcs))
    if missing:
        raise RuntimeError(f"missing sources: {missing}")
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
