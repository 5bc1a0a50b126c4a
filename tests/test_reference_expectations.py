"""The reference's own test expectations for the sampling path, restated here and run against
both the CPU oracle (always) and the HIP sampler through its C ABI (on the GPU box).

Sources (reference tree): extension/llm/sampler/test/test_sampler.cpp:19-154,
extension/llm/runner/test/test_text_decoder_runner.cpp:83-230,
extension/llm/runner/test/test_text_llm_runner.cpp:656-762.
"""
import numpy as np
import pytest
import torch

from executorch_amd import workloads as W

BACKENDS = ["oracle", pytest.param("hip", marks=pytest.mark.gpu)]


class OracleBackend:
    def __init__(self, oracle):
        self.O = oracle

    def sampler(self, vocab, temperature, topp, seed):
        return self.O.Sampler(vocab, temperature, topp, seed)

    def sample(self, s, row, dtype):
        return s.sample(row.copy(), dtype)  # the reference mutates its input; keep the caller's

    def sample_from_logits(self, s, arr, dtype):
        import ctypes as C

        a = np.ascontiguousarray(arr).copy()
        sizes = (C.c_int64 * a.ndim)(*a.shape)
        return self.O.lib().oracle_sample_from_logits(C.byref(s.s), a.ctypes.data, dtype, a.ndim, sizes,
                                                      self.O.MODE_NATIVE, self.O.TIE_LIBSTDCXX)

    def logits_to_token(self, arr, dtype, temperature=0.0):
        s = self.O.Sampler(arr.shape[-1], temperature, 0.9, 12345)
        return self.sample_from_logits(s, arr, dtype)


class HipBackend:
    def sampler(self, vocab, temperature, topp, seed):
        import executorch_amd as ea

        return ea.Sampler(vocab, temperature, topp, seed)

    def sample(self, s, row, dtype):
        return s.sample(row, dtype)

    def sample_from_logits(self, s, arr, dtype):
        import executorch_amd as ea

        return ea.sample_from_logits(arr, s, dtype)

    def logits_to_token(self, arr, dtype, temperature=0.0):
        import executorch_amd as ea

        return ea.logits_to_token(arr, temperature, dtype)


@pytest.fixture
def be(request, oracle):
    return OracleBackend(oracle) if request.param == "oracle" else HipBackend()


def pytest_generate_tests(metafunc):
    if "be" in metafunc.fixturenames:
        metafunc.parametrize("be", BACKENDS, indirect=True)


def store(a, dtype):
    return W.to_storage(np.asarray(a, dtype=np.float32), dtype)


# ---- test_sampler.cpp:19-43
@pytest.mark.parametrize("dtype", [W.DTYPE_FLOAT, W.DTYPE_HALF])
def test_argmax(be, dtype):
    g = torch.Generator().manual_seed(0)
    x = np.minimum(torch.rand(32000, generator=g).numpy(), np.float32(0.999))  # stays < 1 in fp16 too
    x[396] = 1.0
    s = be.sampler(32000, 0.0, 0.9, 0)
    assert be.sample(s, store(x, dtype), dtype) == 396


# ---- test_sampler.cpp:45-68
def test_topk_restricts_to_candidates(be):
    s = be.sampler(100, 1.0, 0.0, 42)
    s.set_topk(3)
    x = np.full(100, -10.0, dtype=np.float32)
    x[7], x[13], x[42] = 5.0, 4.5, 4.0
    for _ in range(50):
        assert be.sample(s, x, W.DTYPE_FLOAT) in (7, 13, 42)


# ---- test_sampler.cpp:70-92
def test_topk_disabled_by_zero(be):
    s = be.sampler(50, 1.0, 0.0, 7)
    s.set_topk(0)
    x = np.full(50, -10.0, dtype=np.float32)
    x[11] = 20.0
    hits = sum(be.sample(s, x, W.DTYPE_FLOAT) == 11 for _ in range(20))
    assert hits >= 18


# ---- test_sampler.cpp:94-113
def test_topk_fp16(be):
    s = be.sampler(50, 1.0, 0.0, 99)
    s.set_topk(2)
    x = np.full(50, -10.0, dtype=np.float32)
    x[3], x[8] = 5.0, 4.5
    for _ in range(30):
        assert be.sample(s, store(x, W.DTYPE_HALF), W.DTYPE_HALF) in (3, 8)


# ---- test_sampler.cpp:115-131
def test_topk_one_is_argmax(be):
    s = be.sampler(100, 1.0, 0.0, 123)
    s.set_topk(1)
    x = torch.rand(100, generator=torch.Generator().manual_seed(1)).numpy()
    x[57] = 100.0
    for _ in range(10):
        assert be.sample(s, x, W.DTYPE_FLOAT) == 57


# ---- test_sampler.cpp:133-154
def test_topk_takes_precedence_over_topp(be):
    s = be.sampler(100, 1.0, 0.99, 99)
    s.set_topk(2)
    x = np.full(100, -10.0, dtype=np.float32)
    x[3], x[8], x[19] = 5.0, 4.5, 4.0
    for _ in range(50):
        assert be.sample(s, x, W.DTYPE_FLOAT) in (3, 8)


# ---- test_text_decoder_runner.cpp:83-140
@pytest.mark.parametrize("dtype", [W.DTYPE_FLOAT, W.DTYPE_HALF, W.DTYPE_BFLOAT16])
def test_logits_to_token_rank2(be, dtype):
    x = store([[0.1, 0.2, 0.8, 0.4]], dtype)
    assert be.logits_to_token(x, dtype) == 2


def test_logits_to_token_rank3_uses_last_position(be):
    x = store([[[0.8, 0.1, 0.1, 0.1], [0.1, 0.2, 0.8, 0.4]]], W.DTYPE_FLOAT)
    assert be.logits_to_token(x, W.DTYPE_FLOAT) == 2


def test_logits_to_token_with_temperature_in_range(be):
    x = store([[0.1, 0.2, 0.8, 0.4]], W.DTYPE_FLOAT)
    assert 0 <= be.logits_to_token(x, W.DTYPE_FLOAT, 1.0) < 4


# ---- test_text_decoder_runner.cpp:156-230: one injected Sampler reused across calls
def test_injected_sampler_reuse_and_temperature_switch(be):
    s = be.sampler(4, 0.0, 0.9, 1)
    x = store([[0.1, 0.2, 0.8, 0.4]], W.DTYPE_FLOAT)
    for _ in range(3):
        s.set_temperature(0.0)
        assert be.sample_from_logits(s, x, W.DTYPE_FLOAT) == 2
    s.set_temperature(1.0)
    assert 0 <= be.sample_from_logits(s, x, W.DTYPE_FLOAT) < 4
    s.set_temperature(0.0)
    assert be.sample_from_logits(s, x, W.DTYPE_FLOAT) == 2
    x3 = store([[[0.9, 0.0, 0.0, 0.0], [0.1, 0.2, 0.8, 0.4]]], W.DTYPE_FLOAT)
    assert be.sample_from_logits(s, x3, W.DTYPE_FLOAT) == 2


# ---- test_text_llm_runner.cpp:656-762: greedy over {0.1,0.2,0.3,0.4}, then masked with -inf
def test_greedy_and_masks(be):
    s = be.sampler(4, 0.0, 0.9, 1)
    x = np.array([0.1, 0.2, 0.3, 0.4], dtype=np.float32)
    assert be.sample(s, x, W.DTYPE_FLOAT) == 3
    x[3] = -np.inf
    assert be.sample(s, x, W.DTYPE_FLOAT) == 2
    x[2] = -np.inf
    assert be.sample(s, x, W.DTYPE_FLOAT) == 1


# ---- sampler.h:48-53
def test_negative_temperature_is_reset_to_greedy(be):
    s = be.sampler(4, 1.0, 0.9, 1)
    s.set_temperature(-3.0)
    x = np.array([0.1, 0.2, 0.8, 0.4], dtype=np.float32)
    for _ in range(5):
        assert be.sample(s, x, W.DTYPE_FLOAT) == 2
