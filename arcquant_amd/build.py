"""Builds libarcq_hip.so (gfx950) in-tree with hipcc.

    python -m arcquant_amd.build            # build if stale
    python -m arcquant_amd.build --force    # rebuild even if up to date
    python -m arcquant_amd.build --experiments   # with the measured-and-not-taken kernel variants (ARCQ_GEMM_KERNEL)
    python -m arcquant_amd.build --phases KERNEL # instruction counts between the ARCQ_PHASE markers of one kernel

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


def phase_listing(kernel: str, source: str = "arcq_quantize.hip") -> str:
    """Static instruction counts of one kernel, cut at its ARCQ_PHASE markers and at every label, in the order of
    the compiler's assembly (the device pass alone, -S, with -DARCQ_PHASE_MARKERS: the markers are comments, the
    code is the normal build's).  `kernel` is a substring of the mangled name.  Which pieces run how often per row
    follows from the branches, which the listing shows with their targets."""
    import re
    import tempfile
    flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        subprocess.check_call([_hipcc(), *flags, "-DARCQ_PHASE_MARKERS", "--cuda-device-only", "-S", "-o", out,
                               os.path.join(CSRC, source)], stderr=subprocess.DEVNULL)
        text = open(out).read()
    m = re.search(r"^(\S*%s\S*):" % re.escape(kernel), text, re.M)
    if not m:
        raise SystemExit(f"no kernel matching {kernel!r} in {source}")
    body = text[m.end():text.index(".Lfunc_end", m.end())].split("\n")
    classes = ("valu", "salu", "lds", "vmem")
    rows, phase, label, cur, notes = [], "entry", "", dict.fromkeys(classes, 0), []

    def flush():
        if any(cur.values()) or notes:
            rows.append((label, phase, dict(cur), " ".join(notes)))
        for c in classes:
            cur[c] = 0
        notes.clear()

    for line in body:
        mark = re.search(r"; ARCQ_PHASE (.*)", line)
        lab = re.match(r"(\.LBB\w+):", line)
        if mark or lab:
            flush()
            if mark:
                phase = mark.group(1).strip()
            else:
                label = lab.group(1)
            continue
        w = line.split()
        if not line.startswith("\t") or not w or w[0][0] in ".;":
            continue
        op = w[0]
        cur["valu" if op.startswith("v_") else "salu" if op.startswith("s_") else "lds" if op.startswith("ds_") else "vmem"] += 1
        if op.startswith(("s_cbranch", "s_branch")):
            notes.append(f"{op[2:]}->{w[1]}")
    flush()
    lines = [f"{m.group(1)}", f"{'label':10s} {'phase':42s} {'VALU':>5s} {'SALU':>5s} {'LDS':>4s} {'VMEM':>5s}  branches"]
    for lab, ph, c, n in rows:
        lines.append(f"{lab:10s} {ph:42s} {c['valu']:5d} {c['salu']:5d} {c['lds']:4d} {c['vmem']:5d}  {n}")
    return "\n".join(lines)


if __name__ == "__main__":
    if "--phases" in sys.argv:
        print(phase_listing(sys.argv[sys.argv.index("--phases") + 1]))
        sys.exit(0)
    print(build_all(force="--force" in sys.argv, verbose=True, experiments="--experiments" in sys.argv))
