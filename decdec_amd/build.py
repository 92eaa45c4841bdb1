"""Builds libdecdec_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc.

Usage: ``python -m decdec_amd.build`` or ``decdec_amd.build.build_library()``.
hipcc cross-compiles for gfx950 without a GPU.  The translation units are compiled in parallel and
linked into ``decdec_amd/libdecdec_hip.so``.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "obj")
LIB_PATH = os.path.join(HERE, "libdecdec_hip.so")
SOURCES = ["k_dec.hip", "k_anyprec.hip", "k_lutgemm.hip", "k_sqllm.hip", "k_decode.hip", "capi.hip"]
ARCH = "gfx950"

# -packed-fp32-ops switches the packed-FP32 VALU forms off for the device pass (the host pass
# prints a harmless "not a recognized feature" note); -munsafe-fp-atomics selects the hardware
# float / packed-half atomic instructions instead of compare-and-swap loops.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}")
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l).strip()
    if out:
        print(out, file=sys.stderr)
    return obj


def build_library(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
