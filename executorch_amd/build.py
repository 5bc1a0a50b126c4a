"""Compiles the HIP sampler library for gfx950 into executorch_amd/libet_sampler.so.

``python -m executorch_amd.build`` (or ``__graft_entry__.build()``) runs one hipcc command;
hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import json
import os
import re
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


RESOURCES = os.path.join(HERE, "kernel_resources.json")

# hipcc's host pass does not know the device feature that the packed-fp32 switch names and says so
# once per pass; the device pass honours it (tests/test_build_hygiene.py looks for the packed
# instructions in the library's device code).
_HOST_PASS_NOISE = "is not a recognized feature for this target"


def build_library(verbose: bool = True, extra_flags: list[str] | None = None, out: str = LIB) -> str:
    """One hipcc command.  Also records what every kernel needs (registers, private memory, LDS) in
    kernel_resources.json next to the library: private memory in a hot kernel is a regression that
    no test of results would notice."""
    cmd = [hipcc(), *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", *(extra_flags or []),
           os.path.join(CSRC, "et_sampler.hip"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    kernels: dict[str, dict[str, int]] = {}
    name = None
    keep, pending = True, []
    for line in proc.stderr.splitlines():
        m = re.search(r"remark: +Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            keep, pending = False, []
            continue
        m = re.search(r"remark: +(VGPRs|AGPRs|TotalSGPRs|ScratchSize \[bytes/lane\]|LDS Size \[bytes/block\]|"
                      r"Occupancy \[waves/SIMD\]|SGPRs Spill|VGPRs Spill): (\d+)", line)
        if m and name:
            kernels[name][m.group(1).split(" [")[0]] = int(m.group(2))
            keep, pending = False, []
            continue
        # the rest goes to stderr diagnostic by diagnostic: a remark's or the host pass's own lines
        # (header, include chain, quoted source line, caret) are dropped, warnings and errors kept
        if re.search(r": (remark|warning|error|note|fatal error):", line):
            keep = not ("remark:" in line or _HOST_PASS_NOISE in line)
            if keep:
                for held in pending:
                    print(held, file=sys.stderr)
            pending = []
        elif line.startswith("In file included from") or line.startswith("                 from"):
            pending.append(line)
            continue
        if keep:
            print(line, file=sys.stderr)
    if proc.returncode != 0:
        raise subprocess.CalledProcessError(proc.returncode, cmd)
    if out == LIB:
        with open(RESOURCES, "w") as f:
            json.dump(kernels, f, indent=1, sort_keys=True)
            f.write("\n")
    return out


if __name__ == "__main__":
    build_library()
    print("built", LIB)
    sys.exit(0)
