"""Compiles the HIP sampler library for gfx950 into executorch_amd/libet_sampler.so.

``python -m executorch_amd.build`` (or ``__graft_entry__.build()``) runs one hipcc command;
hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libet_sampler.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fvisibility=hidden",
    "-ffp-contract=off",  # the reference rounds after every multiply and add; never fuse them
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the sampler library cannot be built")
    return exe


def build_library(verbose: bool = True, extra_flags: list[str] | None = None, out: str = LIB) -> str:
    cmd = [hipcc(), *HIPCC_FLAGS, *(extra_flags or []), os.path.join(CSRC, "et_sampler.hip"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build_library()
    print("built", LIB)
    sys.exit(0)
