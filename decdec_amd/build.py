"""Builds libdecdec_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc.

Usage: ``python -m decdec_amd.build`` or ``decdec_amd.build.build_library()``.
hipcc cross-compiles for gfx950 without a GPU.  The translation units are compiled in parallel and
linked into ``decdec_amd/libdecdec_hip.so``.
"""
from __future__ import annotations

import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "obj")
LIB_PATH = os.path.join(HERE, "libdecdec_hip.so")
RESOURCES_PATH = os.path.join(OBJ_DIR, "kernel_resources.json")
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


_REMARK = re.compile(r"remark:\s+(Function Name|TotalSGPRs|VGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]):\s*(\S+)")


def _compile(src: str):
    """Compiles one translation unit; returns (object path, {kernel: {"sgprs", "vgprs", "scratch", "occupancy"}})
    from the compiler's kernel-resource-usage remarks."""
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}")
    kernels, cur, rest, skip = {}, None, [], 0
    keys = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "ScratchSize [bytes/lane]": "scratch", "Occupancy [waves/SIMD]": "occupancy"}
    for line in proc.stdout.splitlines():
        if "kernel-resource-usage" in line:
            m = _REMARK.search(line)
            if m and m.group(1) == "Function Name":
                cur = kernels.setdefault(m.group(2), {})
                skip = 2                                   # the remark is followed by the source line and a caret
            elif m and cur is not None:
                cur[keys[m.group(1)]] = int(m.group(2))
            continue
        if skip:
            skip -= 1
            continue
        if "is not a recognized feature for this target" not in line and "remarks generated" not in line:
            rest.append(line)
    out = "\n".join(rest).strip()
    if out:
        print(out, file=sys.stderr)
    return obj, kernels


def check_resources(kernels: dict) -> list:
    """The register budgets the launch logic relies on; returns the violations as strings.
    * a fused kernel instance chosen to let two 1024-thread workgroups share a compute unit (template flag
      `true`, mangled `Lb1E`) must reach 8 waves per SIMD without spilling;
    * the 16-bit 3-bit any-precision, SqueezeLLM and DEC kernels of the decode path must not use scratch at all
      (a kernel with scratch pays for its set-up at every wave launch)."""
    bad = []
    for name, r in kernels.items():
        two = "Lb1E" in name and "dec_" in name
        fp32 = "kernelILi0E" in name
        if two and not fp32 and "lutgemm" not in name and (r.get("occupancy", 0) < 8 or r.get("scratch", 0) != 0):
            bad.append(f"{name}: budgeted instance has occupancy {r.get('occupancy')} / scratch {r.get('scratch')}")
        hot = (("anyprec_kernelILi1ELi3E" in name or "anyprec_kernelILi2ELi3E" in name) and "dec_" not in name) or \
              "sqllm_kernelILi1E" in name or "dec_kernelILi1E" in name or "dec_kernelILi2E" in name or \
              "dec_anyprec_kernelILi1ELi3E" in name
        if hot and r.get("scratch", 0) != 0:
            bad.append(f"{name}: uses {r.get('scratch')} bytes of scratch per lane")
    return bad


def build_library(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    kernels = {}
    for _, k in results:
        kernels.update(k)
    with open(RESOURCES_PATH, "w") as f:
        json.dump(kernels, f, indent=1, sort_keys=True)
    for msg in check_resources(kernels):
        print(f"register budget: {msg}", file=sys.stderr)
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
