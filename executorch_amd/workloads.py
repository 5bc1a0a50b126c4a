"""Synthetic logits for the five sampler workloads named by the benchmark contract.

Rows are generated on the host with numpy's PCG64 (``default_rng``), seeded from
``(data_seed, step)``, then rounded to the storage type with round-to-nearest-even.  16-bit
brain-float rows are returned as ``uint16`` bit patterns (numpy has no bfloat16).  The same
arrays feed the HIP sampler and the CPU checker, so both see identical bits.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

# executorch ScalarType codes (runtime/core/portable_type/scalar_type.h:98-125 in the reference)
DTYPE_HALF, DTYPE_FLOAT, DTYPE_BFLOAT16, DTYPE_UINT16 = 5, 6, 15, 27
DTYPE_NAMES = {DTYPE_HALF: "fp16", DTYPE_FLOAT: "fp32", DTYPE_BFLOAT16: "bf16", DTYPE_UINT16: "u16"}
DTYPE_SIZES = {DTYPE_HALF: 2, DTYPE_FLOAT: 4, DTYPE_BFLOAT16: 2, DTYPE_UINT16: 2}


@dataclass(frozen=True)
class Workload:
    name: str
    vocab: int
    batch: int
    dtype: int
    temperature: float
    topp: float
    steps: int
    data_seed: int
    coin_seed: int  # row b's xorshift64* stream starts from coin_seed + b
    kind: str

    @property
    def bytes_per_step(self) -> int:
        return self.batch * self.vocab * DTYPE_SIZES[self.dtype]


WORKLOADS = {
    "cfg1_greedy": Workload("cfg1_greedy", 32000, 1, DTYPE_FLOAT, 0.0, 0.9, 1000, 42, 42, "normal2"),
    "cfg1": Workload("cfg1", 32000, 1, DTYPE_FLOAT, 0.8, 0.9, 1000, 42, 42, "normal2"),
    "cfg2": Workload("cfg2", 128256, 64, DTYPE_BFLOAT16, 0.6, 0.9, 200, 43, 1000, "peaked"),
    "cfg3": Workload("cfg3", 151936, 256, DTYPE_HALF, 1.0, 0.95, 100, 44, 2000, "flat"),
    "cfg4": Workload("cfg4", 128256, 512, DTYPE_FLOAT, 1.0, 1.0, 100, 45, 3000, "normal15"),
    "cfg5": Workload("cfg5", 262144, 1024, DTYPE_BFLOAT16, 0.7, 0.8, 50, 46, 4000, "mixed"),
}


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round-to-nearest-even, NaN -> 0x7FC0."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    out = ((u + bias) >> np.uint32(16)).astype(np.uint16)
    out[np.isnan(a)] = 0x7FC0
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def to_storage(a: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == DTYPE_FLOAT:
        return np.ascontiguousarray(a, dtype=np.float32)
    if dtype == DTYPE_HALF:
        return np.ascontiguousarray(a.astype(np.float16))
    if dtype == DTYPE_BFLOAT16:
        return f32_to_bf16_bits(a)
    raise ValueError(dtype)


def to_f32(a: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == DTYPE_FLOAT:
        return a
    if dtype == DTYPE_HALF:
        return a.astype(np.float32)
    if dtype == DTYPE_BFLOAT16:
        return bf16_bits_to_f32(a)
    if dtype == DTYPE_UINT16:
        return a.astype(np.float32)
    raise ValueError(dtype)


def logits_f32(w: Workload, step: int, rows: int | None = None) -> np.ndarray:
    """fp32 values of step ``step`` before rounding to the storage type ([rows, vocab])."""
    B = w.batch if rows is None else rows
    V = w.vocab
    rng = np.random.default_rng([w.data_seed, step])
    if w.kind == "normal2":
        return rng.standard_normal((B, V), dtype=np.float32) * np.float32(2.0)
    if w.kind == "normal15":
        return rng.standard_normal((B, V), dtype=np.float32) * np.float32(1.5)
    if w.kind == "flat":
        return rng.standard_normal((B, V), dtype=np.float32) * np.float32(0.5)
    if w.kind == "peaked":
        x = rng.standard_normal((B, V), dtype=np.float32)
        for b in range(B):
            ids = rng.choice(V, size=20, replace=False)
            x[b, ids] += np.float32(8.0)
        return x
    if w.kind == "mixed":
        x = rng.standard_normal((B, V), dtype=np.float32)
        odd = np.arange(B) % 2 == 1
        n_odd = int(odd.sum())
        if n_odd:
            u = rng.random((n_odd, V), dtype=np.float32)
            u = np.clip(u, np.float32(1e-7), np.float32(1.0 - 1e-7))
            g = -np.log(-np.log(u))
            hot = rng.integers(0, V, size=n_odd)
            g[np.arange(n_odd), hot] += np.float32(12.0)
            x[odd] = g.astype(np.float32)
        return x
    raise ValueError(w.kind)


def logits(w: Workload, step: int, rows: int | None = None) -> np.ndarray:
    """Step ``step`` of workload ``w`` in its storage type ([rows, vocab], C-contiguous)."""
    return to_storage(logits_f32(w, step, rows), w.dtype)


def coin_seeds(w: Workload, rows: int | None = None, offset: int = 0) -> np.ndarray:
    B = w.batch if rows is None else rows
    return (np.uint64(w.coin_seed + offset) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
