"""Device-side logit processors through the C ABI (include/et_logit_processor.h): first the
reference's own test cases (extension/llm/sampler/test/test_logit_processor.cpp:109-223, same
names, same expected values), then chains against the CPU restatement, bit for bit, and the
chain followed by the sampler on one stream."""
import os
import sys

import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W
from executorch_amd.logit_processor import AddBiasProcessor, LogitChain, MaskTokenProcessor, MultiplyProcessor
from util import to_device

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
from oracle import logit_processor_oracle as lpo  # noqa: E402

pytestmark = pytest.mark.gpu


def test_single_processor_mutates_logits(dev):
    logits = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=dev)
    AddBiasProcessor(10.0).process(logits)
    assert logits.cpu().tolist() == [[11.0, 12.0, 13.0, 14.0]]


def test_processor_chain_applies_in_order(dev):
    logits = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=dev)
    for p in (MultiplyProcessor(2.0), AddBiasProcessor(1.0)):
        p.process(logits)
    assert logits.cpu().tolist() == [[3.0, 5.0, 7.0, 9.0]]  # (x*2)+1, not (x+1)*2
    again = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=dev)
    LogitChain().add_scale(2.0).add_bias(1.0).process(again)  # the same chain as one launch
    assert again.cpu().tolist() == [[3.0, 5.0, 7.0, 9.0]]


def test_mask_token_drives_argmax_away(dev):
    logits = torch.tensor([[0.1, 0.2, 0.99, 0.4]], device=dev)
    MaskTokenProcessor(2).process(logits)
    out = logits.cpu().numpy()
    assert out[0, 2] == -np.inf
    assert out[0, 0] == np.float32(0.1) and out[0, 1] == np.float32(0.2) and out[0, 3] == np.float32(0.4)
    assert ea.logits_to_token(logits.cpu(), 0.0) == 3


def test_mask_token_out_of_range_is_noop(dev):
    logits = torch.tensor([[1.0, 2.0, 3.0]], device=dev)
    MaskTokenProcessor(99).process(logits)
    MaskTokenProcessor(-1).process(logits)
    assert logits.cpu().tolist() == [[1.0, 2.0, 3.0]]


def test_respects_last_position_of_3d_tensor(dev):
    logits = torch.tensor([[[99.0, 99.0, 99.0, 99.0], [1.0, 2.0, 3.0, 4.0]]], device=dev)
    AddBiasProcessor(10.0).process(logits)
    assert logits.cpu().tolist() == [[[99.0] * 4, [11.0, 12.0, 13.0, 14.0]]]


def test_processor_rejects_unsupported_dtype_and_rank(dev):
    with pytest.raises(ea.SamplerError) as e:
        AddBiasProcessor(1.0).process(torch.zeros((1, 4), dtype=torch.int32, device=dev))
    assert e.value.code == _capi.INVALID_ARGUMENT
    with pytest.raises(ea.SamplerError) as e:
        LogitChain().add_bias(1.0).process(torch.zeros((1, 4), dtype=torch.int16, device=dev), dtype=_capi.DTYPE_UINT16)
    assert e.value.code == _capi.INVALID_ARGUMENT
    for shape in ((4,), (1, 1, 1, 4)):
        with pytest.raises(ea.SamplerError) as e:
            AddBiasProcessor(1.0).process(torch.zeros(shape, device=dev))
        assert e.value.code == _capi.INVALID_ARGUMENT


KINDS = {"f32": (W.DTYPE_FLOAT, torch.float32), "f16": (W.DTYPE_HALF, torch.float16), "bf16": (W.DTYPE_BFLOAT16, torch.bfloat16)}


def device_tensor(values, kind, dev):
    """fp32 values (already representable in `kind`) as a device tensor of that element type."""
    return torch.from_numpy(values).to(dev).to(KINDS[kind][1]).contiguous()


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(3, 50), (5, 8192), (4, 3, 20000), (2, 128256)])
def test_chains_match_the_restatement_bit_for_bit(dev, kind, shape):
    rng = np.random.default_rng([len(kind), *shape])
    vocab, batch = shape[-1], shape[0]
    x = lpo.storage_round((rng.standard_normal(shape) * 3.0).astype(np.float32), kind)
    x.reshape(-1)[rng.integers(0, x.size, 5)] = 0.0
    hist_len = 300
    history = rng.integers(-3, vocab + 3, size=(batch, hist_len)).astype(np.int32)
    history[:, 10:40] = history[:, 50:80]  # repeats inside a row's history
    lengths = rng.integers(0, hist_len + 1, size=batch).astype(np.int32)
    lengths[0] = hist_len
    banned = rng.integers(-2, vocab + 2, size=17).astype(np.int32)
    ids = rng.integers(-2, vocab + 2, size=33).astype(np.int32)
    bias = (rng.standard_normal(33) * 2).astype(np.float32)
    dup_ids = np.concatenate([ids[:9], ids[:9], [ids[0]]]).astype(np.int32)  # an id listed up to three times
    dup_bias = (rng.standard_normal(dup_ids.size) * 2).astype(np.float32)
    d_hist, d_len = torch.from_numpy(history).to(dev), torch.from_numpy(lengths).to(dev)

    recipes = {
        "lists": [("rep", 1.3), ("tb", ids, bias), ("mask", banned)],
        "rows": [("scale", 0.7), ("bias", -1.25), ("scale", 1.0 / 3.0)],
        "mixed": [("mask", banned), ("scale", -1.5), ("tb", dup_ids, dup_bias), ("rep", 0.8), ("bias", 0.1), ("tb", ids, bias),
                  ("rep", 1.7)],
    }
    for name, recipe in recipes.items():
        want = x.copy()
        chain = LogitChain()
        for op in recipe:
            if op[0] == "bias":
                chain.add_bias(op[1]); lpo.add_bias(want, op[1], kind)
            elif op[0] == "scale":
                chain.add_scale(op[1]); lpo.scale(want, op[1], kind)
            elif op[0] == "mask":
                chain.add_mask(op[1]); lpo.mask(want, op[1], kind)
            elif op[0] == "tb":
                chain.add_token_bias(op[1], op[2]); lpo.token_bias(want, op[1], op[2], kind)
            else:
                chain.add_repetition_penalty(op[1], d_hist, d_len); lpo.repetition_penalty(want, op[1], history, lengths, kind)
        assert len(chain) == len(recipe)
        t = device_tensor(x, kind, dev)
        chain.process(t)
        got = t.float().cpu().numpy()
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), (kind, shape, name, np.argwhere(~same)[:5], got[~same][:5], want[~same][:5])


def test_chain_then_sampler_on_one_stream(oracle, dev):
    """Mask + repetition penalty, then the sampler: the tokens are those of the reference sampler
    on logits processed by the restatement."""
    w = W.WORKLOADS["cfg2"]
    rows = 8
    x = W.logits(w, 3, rows)
    xf = W.to_f32(x, w.dtype)
    history = np.argsort(-xf, axis=1)[:, :6].astype(np.int32)  # the six most likely tokens of every row
    lengths = np.full(rows, 6, dtype=np.int32)
    banned = history[:, 0].copy()
    want_logits = xf.copy()
    lpo.repetition_penalty(want_logits, 1.8, history, lengths, "bf16")
    lpo.mask(want_logits, banned, "bf16")
    chain = LogitChain().add_repetition_penalty(1.8, torch.from_numpy(history).to(dev), torch.from_numpy(lengths).to(dev))
    chain.add_mask(banned)
    d = to_device(x, w.dtype, dev)
    s = ea.Sampler(w.vocab, w.temperature, w.topp, 99, max_batch=rows)
    chain.process(d)
    got = s.sample_batch(d).cpu().numpy()
    states = (np.uint64(99) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    want, _ = oracle.sample_rows(W.to_storage(want_logits, w.dtype), w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0,
                                 states, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
    assert np.array_equal(got, want)
    assert not np.isin(got, banned).any()


@pytest.mark.parametrize("dtype_name", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("ops", [
    (("scale", 1.3), ("bias", -0.75)),
    (("bias", 2.5),),
    (("mask", None), ("scale", 0.7), ("bias", 0.3), ("scale", 1.1)),
    (("scale", 1.3), ("mask", None), ("bias", 0.4)),
    (("scale", -0.5), ("bias", 1.0)),
    (("bias", 0.1), ("bias", 0.2), ("scale", 2.0), ("scale", 0.5), ("bias", -0.3), ("scale", 1.7)),
])
def test_chain_fused_into_the_sampler(dev, dtype_name, ops):
    """sample_batch_chain against chain.process followed by sample_batch on a second copy: the same
    tokens and coin states, whatever part of the chain the sampler applies while it reads the rows
    (trailing biases and factors; a mask or more than four of them run in place first)."""
    vocab, rows = 40000, 6
    rng = np.random.default_rng(17)
    x = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    hot = rng.integers(0, vocab, size=(rows, 12))
    np.put_along_axis(x, hot, np.take_along_axis(x, hot, 1) + 7.0, 1)
    x[1, vocab - 3:] = -np.inf   # entries that drop out
    x[2, 5] = np.inf if ops[0][0] != "scale" or ops[0][1] > 0 else -np.inf  # an infinite maximum: every probability NaN or one hot
    tdt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dtype_name]
    if dtype_name == "fp16":
        x = np.clip(x, -60000.0, 60000.0)
    base = torch.from_numpy(x).to(dev).to(tdt)
    banned = np.array([int(hot[0, 0]), 3, vocab - 1], dtype=np.int32)

    def chain():
        c = LogitChain()
        for kind, v in ops:
            if kind == "scale":
                c.add_scale(v)
            elif kind == "bias":
                c.add_bias(v)
            else:
                c.add_mask(banned)
        return c

    for topp in (0.9, 0.5):
        a, b = base.clone(), base.clone()
        s1 = ea.Sampler(vocab, 0.8, topp, 1234, max_batch=rows)
        s2 = ea.Sampler(vocab, 0.8, topp, 1234, max_batch=rows)
        c1, c2 = chain(), chain()
        c1.process(a)
        want = s1.sample_batch(a).cpu().numpy()
        got = s2.sample_batch_chain(b, c2).cpu().numpy()
        assert np.array_equal(got, want), (dtype_name, ops, topp, got, want)
        # a second call continues both coin streams alike
        a2, b2 = base.clone(), base.clone()
        c1.process(a2)
        assert np.array_equal(s2.sample_batch_chain(b2, c2).cpu().numpy(), s1.sample_batch(a2).cpu().numpy())


def test_chain_fused_falls_back_in_place(dev):
    """Rows that do not take the several-workgroups path (here: too short, and temperature 0) get
    the whole chain in place, then the sampler: the tensor then holds the processed logits."""
    vocab, rows = 3000, 4
    rng = np.random.default_rng(5)
    x = rng.standard_normal((rows, vocab)).astype(np.float32)
    for temperature in (0.7, 0.0):
        a, b = torch.from_numpy(x).to(dev), torch.from_numpy(x).to(dev)
        c1, c2 = LogitChain().add_scale(1.5).add_bias(0.25), LogitChain().add_scale(1.5).add_bias(0.25)
        s1 = ea.Sampler(vocab, temperature, 0.9, 7, max_batch=rows)
        s2 = ea.Sampler(vocab, temperature, 0.9, 7, max_batch=rows)
        c1.process(a)
        want = s1.sample_batch(a).cpu().numpy()
        got = s2.sample_batch_chain(b, c2).cpu().numpy()
        assert np.array_equal(got, want)
        assert torch.equal(a, b)


def test_randomised_chains_against_the_restatement():
    """A few hundred random chains over random tensors (tests/fuzz_logit_chain.py), every element
    compared bit for bit with the CPU restatement; stops at the first mismatch."""
    import fuzz_logit_chain

    res = fuzz_logit_chain.run(cases=300, seed=5, stop_after=1)
    assert res["failures"] == 0, res["first_failures"]
    assert res["cases"] == 300
