"""Builds ``poker2_amd/libp2hip.so`` for gfx950 with one ``hipcc`` call."""
from __future__ import annotations

import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libp2hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",          # keep a*b+c as two roundings, like the eager ops replaced
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; libp2hip.so cannot be built")


SWEEP_TIMER_LIB_PATH = os.path.join(PKG_DIR, "libp2hip_sweep_timers.so")


def build_library(verbose: bool = False, sweep_timers: bool = False) -> str:
    """The library; with ``sweep_timers`` a second one, beside it, whose iteration kernel also adds up the
    clock ticks each workgroup spends in each of its sweeps (a tuning build: ``poker2_amd.bench_sweeps``
    reads them; the product never loads it)."""
    out = SWEEP_TIMER_LIB_PATH if sweep_timers else LIB_PATH
    extra = ["-DP2_ITER_PROFILE"] if sweep_timers else []
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra, "-o", out, os.path.join(CSRC, "p2hip.hip")]
    res = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(" ".join(cmd))
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {res.returncode}")
    return out


if __name__ == "__main__":
    import sys
    print(build_library(verbose=True, sweep_timers="--sweep-timers" in sys.argv[1:]))
