"""tests/cpp/decode_loop.cpp: a C++ decode loop over the C ABI with device-resident logits (model
step -> logit processors -> batched sampling -> token fed back through a device-resident history,
the shape of extension/llm/runner/text_token_generator.h:133-148).  Its token sequence must equal
the CPU oracle's over the same synthetic logits: the numpy restatement of the processors, then the
oracle sampler, row by row and step by step."""
import os
import subprocess

import numpy as np
import pytest

from executorch_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KIND = {W.DTYPE_FLOAT: "f32", W.DTYPE_HALF: "f16", W.DTYPE_BFLOAT16: "bf16"}


def build(tmp_path):
    exe = tmp_path / "decode_loop"
    libdir = os.path.join(ROOT, "executorch_amd")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include",
                           os.path.join(ROOT, "tests", "cpp", "decode_loop.cpp"), "-o", str(exe),
                           "-L", libdir, "-l:libet_sampler.so", "-L", "/opt/rocm/lib", "-lamdhip64",
                           f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"])
    return exe


def mix(z):
    z = (z + np.uint64(0x9E3779B97F4A7C15)).astype(np.uint64)
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)).astype(np.uint64)
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)).astype(np.uint64)
    return z ^ (z >> np.uint64(31))


def ring_matrix(seed, r, B, V):
    """The harness's logit (r, b, i), as fp32 (exactly representable in every element type)."""
    with np.errstate(over="ignore"):
        row_id = (np.uint64(r) * np.uint64(B) + np.arange(B, dtype=np.uint64))[:, None]
        z = np.uint64(seed) + row_id * np.uint64(V) + np.arange(V, dtype=np.uint64)[None, :]
        x = ((mix(z) >> np.uint64(56)).astype(np.int64) - 128).astype(np.float32) / np.float32(16.0)
        for b in range(B):
            for j in range(3):
                k = int(mix(np.array([np.uint64(seed) + np.uint64(0xABCDEF) + np.uint64(r * B + b) * np.uint64(3) + np.uint64(j)],
                                     dtype=np.uint64))[0] % np.uint64(V))
                x[b, k] += np.float32(6.0)
    return x


def test_decode_loop_compiles_and_links(tmp_path):
    assert build(tmp_path).exists()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,V,B,steps,temperature", [(W.DTYPE_BFLOAT16, 32064, 6, 12, 0.7), (W.DTYPE_FLOAT, 9000, 3, 8, 0.9),
                                                         (W.DTYPE_HALF, 16384, 4, 6, 0.0)])
def test_decode_loop_tokens_equal_the_oracle(oracle, tmp_path, dtype, V, B, steps, temperature):
    from oracle import logit_processor_oracle as P

    seed, ring, topp = 12345, 3, 0.9
    out = subprocess.run([str(build(tmp_path)), str(V), str(B), str(steps), str(dtype), str(temperature), str(topp), str(seed),
                          str(ring)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    got = np.array([[int(v) for v in line.split(":")[1].split()] for line in out.stdout.splitlines() if line.startswith("tokens")])
    assert got.shape == (steps, B)
    stats = [line for line in out.stdout.splitlines() if line.startswith("stats")][0].split()
    assert int(stats[2]) == steps and int(stats[4]) == steps * B and float(stats[6]) > 0.0
    # the oracle loop
    samplers = [oracle.Sampler(V, temperature, topp, seed + b, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE) for b in range(B)]
    history = np.zeros((B, steps), dtype=np.int32)
    lengths = np.zeros(B, dtype=np.int32)
    for t in range(steps):
        x = ring_matrix(seed, t % ring, B, V)
        P.repetition_penalty(x, 1.25, history, lengths, KIND[dtype])
        P.mask(x, np.arange(100, 116), KIND[dtype])
        stored = W.to_storage(x, dtype)
        for b in range(B):
            want = samplers[b].sample(stored[b].copy(), dtype)
            assert got[t, b] == want, (t, b, got[t, b], want)
            history[b, t] = want
        lengths[:] = t + 1
    print("decode loop:", " ".join(stats))
