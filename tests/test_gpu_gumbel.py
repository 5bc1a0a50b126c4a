"""The Gumbel-max mode through the C ABI against its CPU restatement
(examples/models/qwen3_5_moe/sampler.py:17-60).

Tolerance: the draw is an arg-max over fp32 values x_i + g_i whose two logarithms come from
different fp32 log implementations on the two sides (each within an ulp or two of the true value).
The returned index must therefore be the oracle's arg-max, or an index whose perturbed value (as the
oracle computes it) lies within 1e-5 * max(1, |value|) of the oracle's maximum."""
import os
import sys

import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
from oracle import gumbel_oracle as go  # noqa: E402

pytestmark = pytest.mark.gpu


def check(got, logits, temperature, noise, label):
    v = go.perturbed(logits, temperature, noise)
    want = np.argmax(v, axis=1)
    rows = np.arange(len(want))
    slack = 1e-5 * np.maximum(1.0, np.abs(v[rows, want]))
    ok = (got == want) | (v[rows, got] >= v[rows, want] - slack)
    assert ok.all(), (label, np.nonzero(~ok)[0][:5], got[~ok][:5], want[~ok][:5])
    return int((got != want).sum())


@pytest.mark.parametrize("vocab,rows", [(4, 3), (1000, 7), (32000, 4), (128256, 16)])
def test_given_noise_matches_the_restatement(dev, vocab, rows):
    rng = np.random.default_rng(vocab)
    x = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    u = rng.random((rows, vocab), dtype=np.float32)
    u[:, ::97] = 0.0  # the 1e-20 epsilons matter exactly here
    s = ea.Sampler(vocab, 1.0, 0.9, 5, max_batch=rows)
    dx, du = torch.from_numpy(x).to(dev), torch.from_numpy(u).to(dev)
    near = 0
    for t in (1.0, 0.6, 1e-9, np.linspace(0.5, 2.0, rows).astype(np.float32)):
        got = s.gumbel_max_batch(dx, t, noise=du).cpu().numpy()
        near += check(got, x, t if np.ndim(t) else [t] * rows, u, (vocab, rows, str(t)))
    assert near <= 1  # near-ties are rare
    before = s.get_rng_states()
    s.gumbel_max_batch(dx, 1.0, noise=du)
    assert np.array_equal(s.get_rng_states(), before)  # caller's noise: the coin streams do not move


def test_own_noise_and_half_precision_rows(dev):
    vocab, rows = 50257, 6
    rng = np.random.default_rng(3)
    xf = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    for dtype, tdt in ((W.DTYPE_FLOAT, torch.float32), (W.DTYPE_BFLOAT16, torch.bfloat16), (W.DTYPE_HALF, torch.float16)):
        x = W.to_f32(W.to_storage(xf, dtype), dtype)  # values representable in the storage type
        s = ea.Sampler(vocab, 1.0, 0.9, 700, max_batch=rows)
        states = s.get_rng_states().copy()
        dx = torch.from_numpy(x).to(dev).to(tdt)
        for step in range(2):
            u = np.stack([go.uniform_of(int(states[b]), np.arange(vocab)) for b in range(rows)])
            got = s.gumbel_max_batch(dx, 0.8).cpu().numpy()
            check(got, x, [0.8] * rows, u, (dtype, step))
            for b in range(rows):  # one xorshift64* step per call
                st = int(states[b])
                st ^= st >> 12
                st = (st ^ (st << 25)) & go.MASK
                st ^= st >> 27
                states[b] = st
            assert np.array_equal(s.get_rng_states(), states)


def test_total_variation_of_gumbel_draws(dev):
    p = np.array([0.5, 0.3, 0.15, 0.05])
    rows = 2000
    x = torch.log(torch.tensor(p, dtype=torch.float32)).repeat(rows, 1).to(dev)
    s = ea.Sampler(4, 1.0, 0.9, 31337, max_batch=rows)
    counts = np.zeros(4)
    for _ in range(10):
        counts += np.bincount(s.gumbel_max_batch(x, 1.0).cpu().numpy(), minlength=4)
    assert 0.5 * np.abs(counts / counts.sum() - p).sum() < 0.02


def test_gumbel_argument_errors(dev):
    s = ea.Sampler(64, 1.0, 0.9, 1, max_batch=4)
    x = torch.zeros((4, 64), device=dev)
    with pytest.raises(ea.SamplerError):
        s.gumbel_max_batch(x, [1.0, 2.0])  # neither one temperature nor one per row
    with pytest.raises(ea.SamplerError) as e:
        s.gumbel_max_batch(torch.zeros((4, 64), dtype=torch.int16, device=dev), 1.0, dtype=_capi.DTYPE_UINT16)
    assert e.value.code == _capi.INVALID_ARGUMENT
