"""CPU restatement of the in-graph Gumbel-max sampler, for the tests only (TEST INFRASTRUCTURE:
nothing in the product imports this).

Follows sample(logits, temperature) of examples/models/qwen3_5_moe/sampler.py:17-60 line by line
in numpy fp32 (the reference is a handful of torch ops on a CUDA graph; it is read, not run):

    logits = logits / temperature.clamp(min=1e-6)                      # :50
    noise  = torch.rand_like(logits)                                   # :56
    gumbel = -torch.log(-torch.log(noise + 1e-20) + 1e-20)             # :57
    return (logits + gumbel).argmax(dim=-1, keepdim=True).float()      # :58

Pins (tests/test_oracle_gumbel.py): constant noise gives the arg-max of the logits; the Gumbel
transform at u = 0.5, 0 and 1 - 2^-24 against values computed in float64; a temperature of 0 is
clamped; the frequencies of 20 000 draws against the softmax.  `uniform_of` is this build's own
generator for the case where the caller passes no noise (no counterpart in the reference, which
uses torch's); it is integer arithmetic, restated bit for bit.
"""
import numpy as np

MASK = (1 << 64) - 1


def uniform_of(state: int, index: np.ndarray) -> np.ndarray:
    """splitmix64 finaliser over (state, index) -> fp32 in [0, 1) with 24 random bits."""
    idx = np.asarray(index, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(state & MASK) + (idx + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return ((z >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)).astype(np.float32)


def gumbel_of(noise: np.ndarray) -> np.ndarray:
    u = np.asarray(noise, dtype=np.float32)
    eps = np.float32(1e-20)
    return (-np.log(-np.log(u + eps, dtype=np.float32) + eps, dtype=np.float32)).astype(np.float32)


def perturbed(logits: np.ndarray, temperature, noise: np.ndarray) -> np.ndarray:
    t = np.maximum(np.atleast_1d(np.asarray(temperature, dtype=np.float32)), np.float32(1e-6))
    x = (np.asarray(logits, dtype=np.float32) / t.reshape(-1, 1)).astype(np.float32)
    return (x + gumbel_of(noise)).astype(np.float32)


def sample(logits: np.ndarray, temperature, noise: np.ndarray) -> np.ndarray:
    return np.argmax(perturbed(logits, temperature, noise), axis=-1).astype(np.int32)  # first maximum
