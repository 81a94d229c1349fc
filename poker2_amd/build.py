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


def build_library(verbose: bool = False) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIB_PATH, os.path.join(CSRC, "p2hip.hip")]
    res = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(" ".join(cmd))
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {res.returncode}")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
