"""The Gumbel-max restatement (oracle/gumbel_oracle.py) against what the mathematics fixes."""
import math
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
from oracle import gumbel_oracle as go  # noqa: E402


def test_constant_noise_is_the_argmax_of_the_logits():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 1000)).astype(np.float32)
    for u in (0.0, 0.25, 0.999):
        assert np.array_equal(go.sample(x, 0.7, np.full_like(x, u)), np.argmax(x, axis=1))


def test_gumbel_transform_values():
    for u in (0.5, 0.0, 1.0 - 2.0 ** -24, 2.0 ** -24, 0.1):
        want = -math.log(-math.log(float(np.float32(u)) + 1e-20) + 1e-20)
        got = float(go.gumbel_of(np.array([u], dtype=np.float32))[0])
        assert abs(got - want) <= 4e-6 * max(1.0, abs(want)), (u, got, want)


def test_temperature_is_clamped_and_may_differ_per_row():
    x = np.array([[1.0, 2.0, 3.0], [1.0, 2.0, 3.0]], dtype=np.float32)
    u = np.array([[0.9, 0.5, 0.1], [0.9, 0.5, 0.1]], dtype=np.float32)
    v = go.perturbed(x, [0.0, 2.0], u)
    g = go.gumbel_of(u[0])
    assert np.allclose(v[0], x[0] / np.float32(1e-6) + g) and np.allclose(v[1], x[1] / np.float32(2.0) + g)
    assert go.sample(x, [0.0, 2.0], u).tolist() == [2, 0]  # hot row: the noise decides; cold row: the logits


def test_own_generator_is_uniform_and_keyed():
    u = go.uniform_of(12345, np.arange(200000))
    assert u.dtype == np.float32 and u.min() >= 0.0 and u.max() < 1.0
    assert abs(float(u.mean()) - 0.5) < 0.005 and abs(float(u.var()) - 1.0 / 12.0) < 0.002
    assert not np.array_equal(u[:1000], go.uniform_of(12346, np.arange(1000)))
    # one known answer, computed by hand with Python integers
    z = (7 + 1 * 0x9E3779B97F4A7C15) & go.MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & go.MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & go.MASK
    z ^= z >> 31
    assert float(go.uniform_of(7, np.array([0]))[0]) == (z >> 40) / 16777216.0


def test_draws_follow_the_softmax():
    p = np.array([0.5, 0.3, 0.15, 0.05])
    x = np.tile(np.log(p).astype(np.float32), (20000, 1))
    u = np.stack([go.uniform_of(1000 + b, np.arange(4)) for b in range(20000)])
    counts = np.bincount(go.sample(x, 1.0, u), minlength=4)
    assert 0.5 * np.abs(counts / counts.sum() - p).sum() < 0.02
