"""Compile proof of the drop-in against the real ExecuTorch types: tests/cpp/compile_against_reference.cpp
includes executorch::aten::Tensor / Half / BFloat16 from the reference tree in place and compiles
include/executorch_amd/sampler.h with the body of TextDecoderRunner::logits_to_token
(text_decoder_runner.h:84-94).  Runs only where the reference is mounted (this container); it is
skipped on the GPU box, which has no /root/reference."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = os.environ.get("ET_REFERENCE_ROOT", "/root/reference")


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "runtime", "core")), reason="the reference tree is not mounted")
def test_drop_in_compiles_against_executorch_headers(tmp_path):
    inc = tmp_path / "inc"
    inc.mkdir()
    os.symlink(REFERENCE, inc / "executorch")  # gives the <executorch/...> include prefix
    obj = tmp_path / "compile_against_reference.o"
    cmd = ["g++", "-std=c++17", "-c", "-Wall", "-Wno-deprecated-declarations",
           "-I", str(inc), "-I", os.path.join(REFERENCE, "runtime", "core", "portable_type", "c10"),
           "-DC10_USING_CUSTOM_GENERATED_MACROS", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", "compile_against_reference.cpp"), "-o", str(obj)]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    assert obj.exists()
