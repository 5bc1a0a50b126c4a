"""Golden vectors written from the compiled reference (tests/golden/make_golden.py) against the
CPU oracle (always) and the HIP sampler (on the GPU box, where the reference is absent)."""
import hashlib
import json
import os

import numpy as np
import pytest

from executorch_amd import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "sampler_golden.json")) as f:
    GOLD = json.load(f)


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).view(np.uint8).tobytes()).hexdigest()[:16]


WL = {c["workload"]: c for c in GOLD["workloads"]}
EX = {c["label"]: c for c in GOLD["explicit"]}


@pytest.mark.parametrize("name", sorted(WL))
def test_generated_inputs_have_not_drifted(name):
    c = WL[name]
    w = W.WORKLOADS[name]
    for st in range(min(c["steps"], 3)):
        assert sha(W.logits(w, st, c["rows"])) == c["input_sha"][st]


@pytest.mark.parametrize("name", sorted(WL))
def test_oracle_reproduces_reference_tokens(oracle, name):
    c = WL[name]
    w = W.WORKLOADS[name]
    rows = c["rows"]
    native = [oracle.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed + b, mode=oracle.MODE_NATIVE) for b in range(rows)]
    upcast = [oracle.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed + b, mode=oracle.MODE_UPCAST) for b in range(rows)]
    for st in range(c["steps"]):
        x = W.logits(w, st, rows)
        for b in range(rows):
            probs = np.empty(w.vocab, dtype=np.float32)
            assert upcast[b].sample(x[b].copy(), w.dtype, probs_out=probs) == c["upcast_tokens"][st][b]
            assert native[b].sample(x[b].copy(), w.dtype) == c["native_tokens"][st][b]
            if w.temperature != 0:
                am = int(np.argmax(W.to_f32(x[b], w.dtype)))
                got = [int(probs.view(np.uint32)[i]) for i in (0, 1, w.vocab - 1, am)]
                assert got == c["upcast_prob_words"][st][b]


@pytest.mark.parametrize("label", sorted(EX))
def test_oracle_reproduces_explicit_cases(oracle, label):
    c = EX[label]
    x = W.to_storage(np.array(c["logits"], dtype=np.float32), c["dtype"])
    for mode, key in ((oracle.MODE_NATIVE, "tokens"), (oracle.MODE_UPCAST, "upcast_tokens")):
        s = oracle.Sampler(len(c["logits"]), c["temperature"], c["topp"], c["seed"], mode=mode)
        if c["topk"]:
            s.set_topk(c["topk"])
        assert [s.sample(x.copy(), c["dtype"]) for _ in c[key]] == c[key]


# ---- the same vectors through the HIP sampler's C ABI ---------------------------------------------
def _probs(oracle, w, row):
    po = np.empty(w.vocab, dtype=np.float32)
    oracle.Sampler(w.vocab, w.temperature, w.topp, 1, mode=oracle.MODE_UPCAST).sample(row.copy(), w.dtype, probs_out=po)
    return po


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(WL))
def test_hip_reproduces_reference_tokens(oracle, dev, name):
    """Tokens of the compiled reference (fp32 arithmetic on the converted row).  The one licence
    to differ is the order std::sort left among exactly tied candidates: such a row must carry
    the same probability on both tokens and must match the oracle run with index-ordered ties."""
    import executorch_amd as ea
    from util import to_device

    c = WL[name]
    w = W.WORKLOADS[name]
    rows = c["rows"]
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)
    inv = oracle.inv_temperature(w.temperature)
    tied = 0
    for st in range(c["steps"]):
        x = W.logits(w, st, rows)
        assert sha(x) == c["input_sha"][st]
        states = s.get_rng_states(rows)
        got = s.sample_batch(to_device(x, w.dtype, dev)).cpu().numpy()
        want = np.array(c["upcast_tokens"][st])
        stable, _ = oracle.sample_rows(x, w.dtype, inv, w.topp, 0, states.copy(), mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
        assert np.array_equal(got, stable)
        for b in np.nonzero(got != want)[0]:
            p = _probs(oracle, w, x[b])
            assert p[got[b]] == p[want[b]], (name, st, b)
            tied += 1
    print(f"{name}: {tied}/{rows * c['steps']} rows tie-equivalent, rest identical to the reference")


@pytest.mark.gpu
@pytest.mark.parametrize("label", sorted(EX))
def test_hip_reproduces_explicit_cases(oracle, label):
    import executorch_amd as ea

    c = EX[label]
    x = W.to_storage(np.array(c["logits"], dtype=np.float32), c["dtype"])
    s = ea.Sampler(len(c["logits"]), c["temperature"], c["topp"], c["seed"])
    if c["topk"]:
        s.set_topk(c["topk"])
    got = [s.sample(x, c["dtype"]) for _ in c["upcast_tokens"]]
    if got != c["upcast_tokens"]:
        # only rows with exactly tied probabilities may differ (the reference's sort order)
        o = oracle.Sampler(len(c["logits"]), c["temperature"], c["topp"], c["seed"], mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
        if c["topk"]:
            o.set_topk(c["topk"])
        assert got == [o.sample(x.copy(), c["dtype"]) for _ in c["upcast_tokens"]]
        p = np.empty(len(c["logits"]), dtype=np.float32)
        o.sample(x.copy(), c["dtype"], probs_out=p)
        for a, b in zip(got, c["upcast_tokens"]):
            assert p[a] == p[b]
