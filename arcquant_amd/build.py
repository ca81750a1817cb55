"""Builds libarcq_hip.so (gfx950) in-tree with hipcc.

    python -m arcquant_amd.build            # build if stale
    python -m arcquant_amd.build --force    # rebuild even if up to date
    python -m arcquant_amd.build --experiments   # with the measured-and-not-taken kernel variants (ARCQ_GEMM_KERNEL)

hipcc cross-compiles for gfx950 without a GPU present.  The built libraries live next to the
sources (arcquant_amd/csrc/) so that they travel with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_SOURCES = ["arcq_common.hip", "arcq_quantize.hip", "arcq_gemm.hip", "arcq_kvcache.hip", "arcq_moe.hip"]
HIP_LIB = os.path.join(CSRC, "libarcq_hip.so")
# measurement only (plain copy kernels for bench.py and the counter calibration): its own library, so that the
# product library holds operators only
PROBE_LIB = os.path.join(CSRC, "libarcq_probe.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                              # one rounding per written operation
    "-fhip-fp32-correctly-rounded-divide-sqrt",       # x / s and sqrt are IEEE (the default, stated)
    "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build_hip(force: bool = False, verbose: bool = False, experiments: bool = False) -> str:
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    deps = srcs + [os.path.join(CSRC, h) for h in ("arcq_math.h", "arcq_internal.h", "arcq_swiglu.h")] + [
        os.path.join(HERE, "..", "include", "arcq.h")]
    if force or _stale(HIP_LIB, deps):
        # --experiments: also the kernel variants that were measured and not taken (reached only through
        # ARCQ_GEMM_KERNEL; the counter summaries under profiles/ that name one were made with such a build)
        cmd = [_hipcc(), *HIPCC_FLAGS, *(["-DARCQ_EXPERIMENTS"] if experiments else []), "-o", HIP_LIB, *srcs]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return HIP_LIB


def build_probe(force: bool = False, verbose: bool = False) -> str:
    src = os.path.join(CSRC, "arcq_probe.hip")
    if force or _stale(PROBE_LIB, [src, os.path.join(HERE, "..", "include", "arcq_probe.h")]):
        cmd = [_hipcc(), *HIPCC_FLAGS, "-o", PROBE_LIB, src]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return PROBE_LIB


def build_all(force: bool = False, verbose: bool = False, experiments: bool = False):
    return (build_hip(force or experiments, verbose, experiments), build_probe(force, verbose))


if __name__ == "__main__":
    print(build_all(force="--force" in sys.argv, verbose=True, experiments="--experiments" in sys.argv))
