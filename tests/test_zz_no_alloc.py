"""ets_sampler_sample_batch_static(): the entry point whose kernels work out of a fixed array in the
library's device image and which allocates nothing.  Its tokens and coin states must equal those of
ets_sampler_sample_batch() -- here on two calls in a row, the second with a smaller input -- and a
problem beyond the array's size must be refused."""
import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W
from util import to_device

pytestmark = pytest.mark.gpu


def rows_of(V, B, dtype, seed, peaked):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, V)).astype(np.float32) * (1.0 if peaked else 0.5)
    if peaked:
        for b in range(B):
            x[b, rng.choice(V, size=12, replace=False)] += 8.0
    return W.to_storage(x, dtype)


@pytest.mark.parametrize("dtype", [W.DTYPE_BFLOAT16, W.DTYPE_HALF, W.DTYPE_FLOAT])
@pytest.mark.parametrize("temperature,topp,topk", [(0.7, 0.9, 0), (0.0, 0.9, 0), (1.0, 1.0, 0), (0.8, 0.9, 7)])
def test_static_entry_matches_the_allocating_one(dev, dtype, temperature, topp, topk):
    V = 50264
    ref = ea.Sampler(V, temperature, topp, 4242, max_batch=8)
    sta = ea.Sampler(V, temperature, topp, 4242, max_batch=8)
    for smp in (ref, sta):
        smp.set_topk(topk)
    # two calls in a row, the second with fewer rows; peaked rows, then flat ones (long nucleus)
    for rows, seed, peaked in ((8, 1, True), (3, 2, False)):
        x = to_device(rows_of(V, rows, dtype, seed, peaked), dtype, dev)
        want = ref.sample_batch(x).cpu().numpy()
        out = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        got = sta.sample_batch_static(x, out=out).cpu().numpy()
        assert np.array_equal(got, want), (rows, got, want)
        assert np.array_equal(sta.get_rng_states(), ref.get_rng_states())


def test_static_entry_refuses_what_does_not_fit(dev):
    V, B = 128256, 64  # needs far more than the 32 MiB array
    s = ea.Sampler(V, 0.6, 0.9, 1, max_batch=B)
    x = torch.zeros((B, V), dtype=torch.bfloat16, device=dev)
    with pytest.raises(ea.SamplerError) as err:
        s.sample_batch_static(x)
    assert err.value.code == _capi.INVALID_ARGUMENT
    assert "static scratch" in str(err.value)
    # the handle is still usable, and a problem that fits goes through
    small = ea.Sampler(V, 0.6, 0.9, 1, max_batch=8)
    assert small.sample_batch_static(x[:8]).shape == (8,)
