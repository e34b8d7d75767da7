"""Builds librgs_gfx950.so from the HIP sources in csrc/ with hipcc, in-tree.

Usage: ``python -m retinags_amd.build`` (add ``--force`` to rebuild everything).
There is no GPU requirement: hipcc cross-compiles for gfx950.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librgs_gfx950.so")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # packed fp32 math is kept off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # float atomics in LDS and global memory map to the hardware add instructions
    "-munsafe-fp-atomics",
]

# Files whose floating-point results feed bit-exact integer stages or per-pixel
# thresholds are built without fused multiply-add contraction.
SOURCES = {
    "api.hip": [],
    "preprocess.hip": ["-ffp-contract=off"],
    "binning.hip": [],
    "blend.hip": ["-ffp-contract=off"],
    "composite.hip": [],
    "sharing.hip": ["-ffp-contract=off"],
    "training.hip": [],
}

HEADERS = ["rgs_device.h", "rgs_kernels.h", "strip_filing.h", "tile_order.h", os.path.join("..", "..", "include", "rgs.h")]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = True) -> str:
    hipcc = _hipcc()
    hdrs = [os.path.join(CSRC, h) for h in HEADERS]
    objs, jobs = [], []
    for src, extra in SOURCES.items():
        s = os.path.join(CSRC, src)
        o = os.path.join(CSRC, src.replace(".hip", ".o"))
        objs.append(o)
        if force or _stale(o, [s] + hdrs):
            jobs.append([hipcc] + COMMON + extra + ["-c", s, "-o", o])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass of hipcc reports that it does not know the packed-fp32 feature; harmless
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed:\n{' '.join(cmd)}\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)

    with ThreadPoolExecutor(max_workers=min(4, max(1, len(jobs)))) as ex:
        list(ex.map(run, jobs))
    if force or jobs or _stale(LIB, objs):
        run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print(LIB)
