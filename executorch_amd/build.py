"""Compiles the HIP sampler library for gfx950 into executorch_amd/libet_sampler.so.

``python -m executorch_amd.build`` (or ``__graft_entry__.build()``) compiles the translation units
of csrc/ side by side and links them; hipcc cross-compiles, so no GPU is needed to build.
``--phase-clocks OUT.so`` builds a profiling variant (device clocks around the kernels' phases).
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


# Translation units of libet_sampler.so: the host side of the C ABI, and one file per element type
# and kernel family, compiled side by side.
LIB_UNITS = [
    "et_sampler.hip",
    "ets_rows_f32.hip", "ets_rows_f16.hip", "ets_rows_bf16.hip",
    "ets_split_f32.hip", "ets_split_f16.hip", "ets_split_bf16.hip",
    "ets_split_topk_f32.hip", "ets_split_topk_f16.hip", "ets_split_topk_bf16.hip",
]
# Test and measurement hooks (csrc/ets_test_hooks.h): a library of their own.
HOOKS_LIB = os.path.join(HERE, "libet_sampler_hooks.so")
HOOKS_UNITS = ["ets_test_hooks.hip"]
OBJ_DIR = os.path.join(HERE, "build")


def _filter_diagnostics(stderr: str, kernels: dict[str, dict[str, int]]) -> None:
    """Collects the resource remarks of one compile into `kernels`; prints everything else but the
    remarks and the host pass's note about the packed-fp32 switch."""
    name = None
    keep, pending = True, []
    for line in stderr.splitlines():
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


def _compile(unit: str, obj: str, extra_flags: list[str], verbose: bool) -> tuple[str, subprocess.CompletedProcess]:
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    cmd = [hipcc(), *flags, "-Rpass-analysis=kernel-resource-usage", *extra_flags, "-c", os.path.join(CSRC, unit), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    return unit, subprocess.run(cmd, stderr=subprocess.PIPE, text=True)


def build_library(verbose: bool = True, extra_flags: list[str] | None = None, out: str = LIB,
                  hooks_out: str | None = HOOKS_LIB, jobs: int | None = None) -> str:
    """Compiles every translation unit (side by side, `jobs` at a time) and links libet_sampler.so
    and, unless `hooks_out` is None, libet_sampler_hooks.so.  Also records what every kernel needs
    (registers, private memory, LDS) in kernel_resources.json next to the library: private memory in
    a hot kernel is a regression that no test of results would notice."""
    from concurrent.futures import ThreadPoolExecutor

    extra = list(extra_flags or [])
    tag = "" if out == LIB else "_" + re.sub(r"\W", "_", os.path.basename(out))
    os.makedirs(OBJ_DIR, exist_ok=True)
    units = LIB_UNITS + (HOOKS_UNITS if hooks_out else [])
    objs = {u: os.path.join(OBJ_DIR, os.path.splitext(u)[0] + tag + ".o") for u in units}
    jobs = jobs or min(len(units), os.cpu_count() or 4, 16)
    kernels: dict[str, dict[str, int]] = {}
    failed = None
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for unit, proc in pool.map(lambda u: _compile(u, objs[u], extra, verbose), units):
            _filter_diagnostics(proc.stderr, kernels)
            if proc.returncode != 0 and failed is None:
                failed = subprocess.CalledProcessError(proc.returncode, unit)
    if failed is not None:
        raise failed
    link_flags = ["--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden"]
    for target, members in ((out, LIB_UNITS), (hooks_out, HOOKS_UNITS)):
        if not target:
            continue
        cmd = [hipcc(), *link_flags, *[objs[u] for u in members], "-o", target]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    if out == LIB:
        with open(RESOURCES, "w") as f:
            json.dump(kernels, f, indent=1, sort_keys=True)
            f.write("\n")
    return out


if __name__ == "__main__":
    if len(sys.argv) == 3 and sys.argv[1] == "--phase-clocks":
        build_library(extra_flags=["-DETS_PHASE_CLOCKS=1"], out=os.path.abspath(sys.argv[2]), hooks_out=None)
        print("built", sys.argv[2])
        sys.exit(0)
    build_library()
    print("built", LIB, "and", HOOKS_LIB)
    sys.exit(0)
