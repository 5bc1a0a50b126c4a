"""Helpers shared by the tests: moving numpy rows to the device, reference-style inputs."""
from __future__ import annotations

import numpy as np
import torch

from executorch_amd import workloads as W


def to_device(x: np.ndarray, dtype: int, dev) -> torch.Tensor:
    """numpy storage array -> device tensor of the matching torch dtype (same bits)."""
    if dtype == W.DTYPE_BFLOAT16:
        return torch.from_numpy(x.view(np.int16)).to(dev).view(torch.bfloat16)
    if dtype == W.DTYPE_UINT16:
        return torch.from_numpy(x.view(np.int16)).to(dev).view(torch.uint16)
    return torch.from_numpy(x).to(dev)


def f32_bits(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def seq_sum_f32(a: np.ndarray, s0: float = 0.0, thr: float = np.inf):
    """The scalar loop the reference runs: s += a[i] in fp32, stop at the first s > thr."""
    s = np.float32(s0)
    for i, v in enumerate(np.asarray(a, dtype=np.float32)):
        s = np.float32(s + v)
        if s > thr:
            return s, i
    return s, -1
