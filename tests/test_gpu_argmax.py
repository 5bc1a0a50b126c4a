"""Greedy path (temperature 0) of the HIP sampler against the oracle: bit-exact token ids for
every dtype, with ties, signed zeros, NaN, -inf masks, strided rows and ragged sizes."""
import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import workloads as W
from util import to_device

pytestmark = pytest.mark.gpu

DTYPES = [W.DTYPE_FLOAT, W.DTYPE_HALF, W.DTYPE_BFLOAT16]


def oracle_argmax(oracle, x, dtype):
    out = []
    for row in x:
        s = oracle.Sampler(row.size, 0.0, 0.9, 1)
        out.append(s.sample(row.copy(), dtype))
    return np.array(out, dtype=np.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,B", [(1, 3), (2, 5), (63, 4), (4096, 7), (32000, 1), (128256, 64), (151936, 16), (262144, 8)])
def test_argmax_matches_oracle(oracle, dev, dtype, V, B):
    rng = np.random.default_rng([V, B, dtype])
    f = rng.standard_normal((B, V)).astype(np.float32)
    f[B // 2] = np.round(f[B // 2] * 2) / 2  # a row full of ties
    x = W.to_storage(f, dtype)
    s = ea.Sampler(V, 0.0, 0.9, 5, max_batch=B)
    before = s.get_rng_states()
    got = s.sample_batch(to_device(x, dtype, dev)).cpu().numpy()
    assert np.array_equal(got, oracle_argmax(oracle, x, dtype))
    assert np.array_equal(s.get_rng_states(), before)  # greedy consumes no coin


def test_argmax_special_values(oracle, dev):
    V = 5000
    rows = []
    r = np.full(V, -1.0, np.float32); r[100] = r[4000] = 3.0; rows.append(r)                    # tie: lowest index
    r = np.full(V, -0.0, np.float32); r[77] = 0.0; rows.append(r)                                # -0 == +0: index 0
    r = np.full(V, 1.0, np.float32); r[0] = np.nan; r[9] = 50.0; rows.append(r)                  # NaN in slot 0 wins
    r = np.full(V, 1.0, np.float32); r[5] = np.nan; r[4321] = 2.0; rows.append(r)                # NaN elsewhere never wins
    r = np.full(V, -np.inf, np.float32); r[4999] = -1e4; rows.append(r)                          # masks
    r = np.full(V, -np.inf, np.float32); rows.append(r)                                          # all masked: index 0
    r = np.full(V, np.nan, np.float32); rows.append(r)                                           # all NaN: index 0
    r = np.full(V, 1.0, np.float32); r[3] = np.inf; r[8] = np.inf; rows.append(r)                # +inf tie
    x = np.stack(rows)
    for dtype in DTYPES:
        xs = W.to_storage(x, dtype)
        s = ea.Sampler(V, 0.0, 0.9, 5, max_batch=len(rows))
        got = s.sample_batch(to_device(xs, dtype, dev)).cpu().numpy()
        assert np.array_equal(got, oracle_argmax(oracle, xs, dtype)), dtype
        assert list(got) == [100, 0, 0, 4321, 4999, 0, 0, 3]


def test_argmax_uint16(oracle, dev):
    rng = np.random.default_rng(3)
    x = rng.integers(0, 65536, (6, 70000)).astype(np.uint16)
    x[2, :] = 7
    x[3, 100] = x[3, 60000] = 65535
    s = ea.Sampler(70000, 0.0, 0.9, 5, max_batch=6)
    got = s.sample_batch(to_device(x, W.DTYPE_UINT16, dev)).cpu().numpy()
    assert np.array_equal(got, oracle_argmax(oracle, x, W.DTYPE_UINT16))
    assert got[2] == 0 and got[3] == 100


def test_argmax_strided_rows_and_host_pointer(oracle, dev):
    V, B, stride = 1000, 9, 1536
    rng = np.random.default_rng(4)
    f = rng.standard_normal((B, stride)).astype(np.float32)
    f[:, V:] = 1e9  # padding beyond vocab must be ignored
    big = torch.from_numpy(f).to(dev)
    s = ea.Sampler(V, 0.0, 0.9, 5, max_batch=B)
    got = s.sample_batch(big[:, :V]).cpu().numpy()
    assert np.array_equal(got, np.argmax(f[:, :V], axis=1))
    assert s.sample(f[4, :V].copy()) == int(np.argmax(f[4, :V]))
    assert s.sample(torch.from_numpy(f[5, :V].copy()).to(torch.bfloat16)) == int(
        np.argmax(torch.from_numpy(f[5, :V].copy()).to(torch.bfloat16).float().numpy()))
