"""Edge inputs and error behaviour of the C ABI on the device."""
import ctypes as C

import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W
from util import to_device

pytestmark = pytest.mark.gpu


def oracle_tokens(oracle, x, dtype, temperature, topp, topk, seeds):
    return oracle.sample_rows(x, dtype, oracle.inv_temperature(temperature), topp, topk, seeds.copy(),
                              mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)[0]


def test_masked_rows(oracle, dev):
    V, B = 3000, 6
    rng = np.random.default_rng(1)
    f = rng.standard_normal((B, V)).astype(np.float32)
    f[0, ::2] = -np.inf
    f[1, 1:] = -np.inf          # a single live token
    f[2, :-1] = -np.inf         # only the last token
    f[3, 10:] = -np.inf
    seeds = (np.uint64(5) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
    for topp in (0.9, 1.0):
        s = ea.Sampler(V, 0.7, topp, 5, max_batch=B)
        got = s.sample_batch(torch.from_numpy(f).to(dev)).cpu().numpy()
        assert np.array_equal(got, oracle_tokens(oracle, f, W.DTYPE_FLOAT, 0.7, topp, 0, seeds))
        assert got[1] == 0 and got[2] == V - 1 and got[0] % 2 == 1 and got[3] < 10


def test_nan_and_all_masked_rows(oracle, dev):
    """Rows the reference turns into all-NaN probabilities: multinomial returns the last index;
    top-p keeps no candidate, which the reference leaves undefined and both sides report as -1;
    top-k falls back to its last entry in index order."""
    V = 500
    f = np.random.default_rng(2).standard_normal((3, V)).astype(np.float32)
    f[0, 7] = np.nan
    f[1, :] = -np.inf
    f[2, 3] = np.inf
    seeds = np.array([9, 10, 11], dtype=np.uint64)
    for topp, want in ((1.0, V - 1), (0.9, -1)):
        s = ea.Sampler(V, 1.0, topp, 9, max_batch=3)
        got = s.sample_batch(torch.from_numpy(f).to(dev)).cpu().numpy()
        assert list(got) == [want] * 3
        assert np.array_equal(got, oracle_tokens(oracle, f, W.DTYPE_FLOAT, 1.0, topp, 0, seeds))
        assert not np.array_equal(s.get_rng_states(), seeds)  # the coin is still drawn
    # top-k: all comparisons are false, every entry ties; in index order the walk falls back to entry topk - 1
    for topk in (1, 40, V - 1):
        s = ea.Sampler(V, 1.0, 0.9, 9, max_batch=3)
        s.set_topk(topk)
        got = s.sample_batch(torch.from_numpy(f).to(dev)).cpu().numpy()
        assert list(got) == [topk - 1] * 3
        assert np.array_equal(got, oracle_tokens(oracle, f, W.DTYPE_FLOAT, 1.0, 0.9, topk, seeds))


def test_seed_zero_and_negative_temperature(oracle, dev):
    V, B = 2048, 4
    f = np.random.default_rng(3).standard_normal((B, V)).astype(np.float32)
    s = ea.Sampler(V, 0.8, 0.9, 0, max_batch=B)
    s.set_rng_states(np.zeros(B, dtype=np.uint64))  # xorshift's fixed point: every coin is 0.0
    got = s.sample_batch(torch.from_numpy(f).to(dev)).cpu().numpy()
    assert np.array_equal(got, np.argmax(f, axis=1))  # coin 0 picks the head of the sorted nucleus
    assert np.array_equal(s.get_rng_states(), np.zeros(B, dtype=np.uint64))
    # the 4-argument constructor does not clamp: a negative temperature flips the ranking
    seeds = (np.uint64(21) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
    s = ea.Sampler(V, -0.5, 0.9, 21, max_batch=B)
    got = s.sample_batch(torch.from_numpy(f).to(dev)).cpu().numpy()
    assert np.array_equal(got, oracle_tokens(oracle, f, W.DTYPE_FLOAT, -0.5, 0.9, 0, seeds))


def test_vocab_of_one(dev):
    x = torch.tensor([[1.5], [2.5]], device=dev)
    assert list(ea.Sampler(1, 0.0, 0.9, 1, max_batch=2).sample_batch(x).cpu().numpy()) == [0, 0]
    assert list(ea.Sampler(1, 1.0, 1.0, 1, max_batch=2).sample_batch(x).cpu().numpy()) == [0, 0]


def test_rank3_adapter_and_dtypes(oracle):
    rng = np.random.default_rng(4)
    V = 777
    f = rng.standard_normal((1, 5, V)).astype(np.float32)
    for dtype, arr in ((W.DTYPE_FLOAT, f), (W.DTYPE_HALF, f.astype(np.float16)), (W.DTYPE_BFLOAT16, W.f32_to_bf16_bits(f))):
        s = ea.Sampler(V, 0.9, 0.9, 314)
        o = oracle.Sampler(V, 0.9, 0.9, 314, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
        for _ in range(3):
            assert ea.sample_from_logits(arr, s, dtype) == o.sample(np.ascontiguousarray(arr[0, -1]).copy(), dtype)
    t = torch.from_numpy(f).to(torch.bfloat16)
    assert ea.logits_to_token(t) == int(torch.argmax(t[0, -1].float()))


def test_errors_are_statuses_not_aborts(dev):
    L = _capi.lib()
    s = ea.Sampler(100, 1.0, 0.9, 1, max_batch=2)
    x = torch.zeros((3, 100), device=dev)
    with pytest.raises(ea.SamplerError) as e:
        s.sample_batch(x)  # batch 3 > max_batch 2
    assert e.value.code == _capi.INVALID_ARGUMENT and "max_batch" in str(e.value)
    with pytest.raises(ea.SamplerError) as e:
        s.sample_batch(torch.zeros((2, 100), device=dev, dtype=torch.float64))
    assert e.value.code == _capi.INVALID_ARGUMENT
    with pytest.raises(ea.SamplerError) as e:
        s.sample_batch(torch.zeros((2, 99), device=dev))
    assert e.value.code == _capi.INVALID_ARGUMENT
    tok = C.c_int32()
    assert L.ets_sampler_sample(s._h, None, _capi.DTYPE_FLOAT, C.byref(tok)) == _capi.INVALID_ARGUMENT
    assert L.ets_sampler_sample(s._h, x.cpu().numpy().ctypes.data, 7, C.byref(tok)) == _capi.INVALID_ARGUMENT  # Double
    assert b"dtype" in L.ets_sampler_last_error(s._h)
    sizes = (C.c_int64 * 2)(1, 64)
    assert L.ets_sample_from_logits(s._h, x.cpu().numpy().ctypes.data, _capi.DTYPE_FLOAT, 2, sizes, C.byref(tok)) == _capi.INVALID_ARGUMENT
    u16 = torch.zeros((2, 100), device=dev, dtype=torch.uint16)
    with pytest.raises(ea.SamplerError) as e:
        s.sample_batch(u16)
    assert e.value.code == _capi.NOT_SUPPORTED
    s.set_temperature(0.0)
    assert list(s.sample_batch(u16).cpu().numpy()) == [0, 0]  # greedy over quantised logits is supported
    assert L.ets_sampler_sample_batch(s._h, x.data_ptr(), _capi.DTYPE_FLOAT, 0, 100, x.data_ptr(), None) == _capi.OK
    h = C.c_void_p()
    assert L.ets_sampler_create(1 << 24, 1.0, 0.9, 1, 1, C.byref(h)) == _capi.NOT_SUPPORTED  # counts are kept in floats


def test_runs_on_a_side_stream(oracle, dev):
    w = W.WORKLOADS["cfg2"]
    rows = 8
    x = W.logits(w, 1, rows)
    dx = to_device(x, w.dtype, dev)
    s = ea.Sampler(w.vocab, w.temperature, w.topp, 55, max_batch=rows)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out = s.sample_batch(dx)
    side.synchronize()
    seeds = (np.uint64(55) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    assert np.array_equal(out.cpu().numpy(), oracle_tokens(oracle, x, w.dtype, w.temperature, w.topp, 0, seeds))
