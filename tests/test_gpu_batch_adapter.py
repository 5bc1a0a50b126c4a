"""ets_sample_from_logits_batch(): the tensor adapter of extension/llm/sampler/util.h:25-55 for a
device-resident tensor and every batch entry (rank 2: each row; rank 3: the last position of each
batch entry), against the oracle's per-row samplers."""
import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W
from util import to_device

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [W.DTYPE_FLOAT, W.DTYPE_HALF, W.DTYPE_BFLOAT16])
@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_rank2_and_rank3(oracle, dev, dtype, temperature):
    rng = np.random.default_rng(3)
    B, S, V = 5, 4, 33000
    x3 = W.to_storage((rng.standard_normal((B, S, V)) * 2.0).astype(np.float32), dtype)
    for rank in (2, 3):
        x = x3[:, -1, :].copy() if rank == 2 else x3
        s = ea.Sampler(V, temperature, 0.9, 600, max_batch=B)
        got = ea.sample_from_logits_batch(to_device(x.reshape(-1, V), dtype, dev).reshape(x.shape), s).cpu().numpy()
        for b in range(B):
            o = oracle.Sampler(V, temperature, 0.9, 600 + b, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
            assert got[b] == o.sample(x3[b, -1].copy(), dtype), (rank, b)


def test_argument_checks(dev):
    V = 1000
    s = ea.Sampler(V, 0.5, 0.9, 1, max_batch=2)
    x = torch.zeros((2, V), dtype=torch.float32, device=dev)
    with pytest.raises(ea.SamplerError) as e:
        ea.sample_from_logits_batch(torch.zeros((3, V), dtype=torch.float32, device=dev), s)  # batch > max_batch
    assert e.value.code == _capi.INVALID_ARGUMENT
    with pytest.raises(ea.SamplerError) as e:
        ea.sample_from_logits_batch(torch.zeros((2, V + 1), dtype=torch.float32, device=dev), s)  # vocab mismatch
    assert e.value.code == _capi.INVALID_ARGUMENT
    with pytest.raises(ea.SamplerError):
        ea.sample_from_logits_batch(x.reshape(2 * V), s)  # rank 1
    assert ea.sample_from_logits_batch(x, s).shape == (2,)
