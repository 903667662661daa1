"""Builds libfast_route_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m fast_route_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfast_route_hip.so")
SOURCES = ["fr_error.hip", "gating.hip", "routing.hip", "quant.hip", "moe_gemm.hip", "fused_moe.hip", "probe.hip"] + [
    "moe_gemm_inst_%s_%s.hip" % (t, e) for t in ("bf16", "f16", "fp8") for e in ("silu", "plain", "down")]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # compiler-generated packed fp32 arithmetic is kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), out))
    return out


MEASUREMENT_LIB = os.path.join(HERE, "libfast_route_hip_measure.so")


def build(verbose: bool = False) -> str:
    """Compiles every source and links the shared library; returns its path.
    FR_HIPCC_FLAGS in the environment adds compiler flags (the measurement switches of
    csrc/moe_gemm_persistent.h, e.g. FR_HIPCC_FLAGS="-DFR_ABL_NOLOAD": kernels whose RESULTS ARE WRONG,
    only their timings mean something).  Such a build never replaces the library tests and callers load:
    it goes to libfast_route_hip_measure.so (objects under build_measure/), which _native loads only when
    FR_NATIVE_LIB names it."""
    hipcc = _hipcc()
    extra = os.environ.get("FR_HIPCC_FLAGS", "").split()
    objdir = os.path.join(HERE, "build_measure" if extra else "build")
    lib = MEASUREMENT_LIB if extra else LIB
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def one(pair):
        src, obj = pair
        return _run([hipcc, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(os.cpu_count() or 8, 16, len(SOURCES))) as pool:
        for out in pool.map(one, zip(SOURCES, objs)):
            if verbose and out.strip():
                print(out)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs])
    return lib


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
