"""Compile the HIP sources into ``kernel_amd/libmoe_a2a.so`` for gfx950.

hipcc cross-compiles without a GPU.  Run as ``python -m kernel_amd.build``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "libmoe_a2a.so")
SOURCES = [os.path.join(PKG_DIR, "csrc", "moe_a2a.hip")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",  # multiply and add of the weighted sum must stay separate roundings
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no packed-f32 instructions
    "-shared",
    "-fPIC",
    "-I" + os.path.join(ROOT, "include"),
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


BENCH_LIB_PATH = os.path.join(PKG_DIR, "libmoe_a2a_bench.so")
BENCH_SOURCES = [os.path.join(PKG_DIR, "csrc", "bench_loop.cpp")]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("build failed:\n" + proc.stdout + proc.stderr)


def build_library(verbose: bool = False) -> str:
    """The product library, then the small host-loop helper bench.py uses (links against it)."""
    _run([hipcc_path(), *HIPCC_FLAGS, *SOURCES, "-o", LIB_PATH], verbose)
    _run(["g++", "-O2", "-shared", "-fPIC", "-I" + os.path.join(ROOT, "include"), *BENCH_SOURCES, "-o",
          BENCH_LIB_PATH, "-L" + PKG_DIR, "-lmoe_a2a", "-Wl,-rpath,$ORIGIN"], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    sys.exit(0)
