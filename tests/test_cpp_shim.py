"""Builds tests/cpp/test_sampler_shim.cpp (the reference's C++ sampler tests written against the
drop-in class in include/executorch_amd/sampler.h) with g++ against libet_sampler.so; runs it
where a GPU is present."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def build(tmp_path):
    exe = tmp_path / "test_sampler_shim"
    libdir = os.path.join(ROOT, "executorch_amd")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp", "test_sampler_shim.cpp"), "-o", str(exe),
                           "-L", libdir, "-l:libet_sampler.so", f"-Wl,-rpath,{libdir}"])
    return exe


def test_shim_compiles_and_links(tmp_path):
    assert build(tmp_path).exists()


@pytest.mark.gpu
def test_shim_passes_reference_tests(tmp_path):
    out = subprocess.run([str(build(tmp_path))], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all passed" in out.stdout
