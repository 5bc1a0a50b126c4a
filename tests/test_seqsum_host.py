"""Builds tests/host/seqsum_host_check.cpp with g++ and runs it: the integer-scan emulation of
a sequential fp32 sum (executorch_amd/csrc/ets_seqsum_math.h) against the plain loop."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_seqsum_math_on_host(tmp_path):
    exe = tmp_path / "seqsum_host_check"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT, "executorch_amd", "csrc"),
                           os.path.join(ROOT, "tests", "host", "seqsum_host_check.cpp"), "-o", str(exe)])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "0 mismatches" in out.stdout


def test_bounded_walks_and_run_walk_on_host(tmp_path):
    """next_event() (an ordered walk only looks ahead, so it ends whatever the flags) and the closed
    form for runs of equal addends against the plain fp32 loop."""
    exe = tmp_path / "bounded_walk_check"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT, "executorch_amd", "csrc"),
                           os.path.join(ROOT, "tests", "host", "bounded_walk_check.cpp"), "-o", str(exe)])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-2000:]
    assert " 0 mismatches" in out.stdout
