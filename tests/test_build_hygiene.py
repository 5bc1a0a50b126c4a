"""What the built library looks like from the outside: no kernel of the hot path keeps data in
private memory (a regression that no comparison of results would notice: an array indexed by a lane's
own value, or a parameter block passed by reference, silently moves there), and the device code holds
none of the packed fp32 instructions the build switches off."""
import json
import os
import re
import shutil
import subprocess

import pytest

from executorch_amd import _capi, build

LLVM = "/opt/rocm/llvm/bin"


def resources():
    if not os.path.exists(build.RESOURCES) or os.path.getmtime(build.RESOURCES) + 5 < os.path.getmtime(_capi.LIB_PATH):
        pytest.skip("kernel_resources.json is written by `python -m executorch_amd.build`; this library was built elsewhere")
    with open(build.RESOURCES) as f:
        return json.load(f)


def test_hot_kernels_keep_nothing_in_private_memory():
    r = resources()
    seen = 0
    for name, v in r.items():
        if "split_pass1_kernel" in name or "split_pass2_kernel" in name or "argmax_partial_kernel" in name or \
                "gumbel_partial_kernel" in name or "logit_chain_kernel" in name:
            assert v["ScratchSize"] == 0 and v["VGPRs Spill"] == 0, (name, v)
            seen += 1
        if re.search(r"split_finish_kernelILi\d+ELb0E", name):  # (the instantiations with a workgroup per row)
            # callee-saved registers of the out-of-line draw functions only (stored when such a
            # function is entered and read back when it returns, never inside a loop)
            assert v["ScratchSize"] <= 96 and v["VGPRs Spill"] == 0, (name, v)
            seen += 1
        if re.search(r"split_finish_kernelILi\d+ELb1E", name):  # (a workgroup takes one row after the other)
            # The loop over the rows costs registers: these instantiations do spill (launches with
            # more rows than compute units only).  The bound keeps that from growing unnoticed.  (The
            # private memory includes the frames of the functions the kernel calls, the chain among them.)
            assert v["ScratchSize"] <= 448 and v["VGPRs Spill"] <= 64, (name, v)
            seen += 1
    assert seen >= 24


def test_pass2_and_finish_fit_one_workgroup_per_cu():
    # 1024 lanes = 4 waves per SIMD: at most 128 vector registers
    for name, v in resources().items():
        if "split_pass2_kernel" in name or "split_finish_kernel" in name or "sample_rows_kernel" in name:
            assert v["VGPRs"] <= 128 and v["Occupancy"] >= 4, (name, v)


def test_no_packed_fp32_instructions_in_the_device_code(tmp_path):
    bundler, objdump = os.path.join(LLVM, "clang-offload-bundler"), os.path.join(LLVM, "llvm-objdump")
    if not (os.path.exists(bundler) and os.path.exists(objdump) and shutil.which("objcopy")):
        pytest.skip("needs ROCm's clang-offload-bundler / llvm-objdump and objcopy")
    fat = tmp_path / "fatbin"
    subprocess.check_call(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", _capi.LIB_PATH, str(fat)])
    # one bundle per translation unit, one after the other in the section
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    data = fat.read_bytes()
    starts = [m.start() for m in re.finditer(re.escape(magic), data)]
    assert len(starts) >= len(build.LIB_UNITS)
    ends, packed = 0, []
    for k, at in enumerate(starts):
        piece = tmp_path / f"bundle{k}"
        piece.write_bytes(data[at:starts[k + 1] if k + 1 < len(starts) else len(data)])
        co = tmp_path / f"gfx950_{k}.co"
        subprocess.check_call([bundler, "--unbundle", "--type=o", f"--input={piece}", f"--output={co}",
                               "--targets=hipv4-amdgcn-amd-amdhsa--gfx950"])
        asm = subprocess.run([objdump, "-d", str(co)], stdout=subprocess.PIPE, text=True, check=True).stdout
        ends += asm.count("s_endpgm")
        packed += re.findall(r"\bv_pk_(?:add|mul|fma)_f32\b", asm)
    assert ends >= 40  # the kernels are in there
    assert not packed, f"{len(packed)} packed fp32 instructions in the device code"
