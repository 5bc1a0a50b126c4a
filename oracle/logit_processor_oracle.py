"""CPU restatement of the logit processors, for the tests only (TEST INFRASTRUCTURE: nothing in
the product imports this).

What the reference fixes is the interface and its contract (extension/llm/sampler/
logit_processor.h:19-40) and three processors in its test file; they are restated here line by
line.  Pins: the expected values of the reference's own tests
(test_logit_processor.cpp:109-223), see tests/test_oracle_logit_processor.py.

  add_bias        AddBiasProcessor      test_logit_processor.cpp:39-63   data[i] += bias
  scale           MultiplyProcessor     test_logit_processor.cpp:65-83   data[i] *= factor
  mask            MaskTokenProcessor    test_logit_processor.cpp:85-104  data[t] = -inf, out of range ignored
  token_bias      no counterpart ("logit bias", logit_processor.h:21)    data[t[j]] += b[j] in list order
  repetition      no counterpart ("repetition penalty", :21); the common rule: each distinct history
                  token once, x < 0 ? x * penalty : x / penalty.  Parity unpinned against the
                  reference (it has no implementation); pinned by hand-computed cases.

Arithmetic: fp32; 16-bit storage is converted to fp32, transformed, and rounded back to nearest
even by every processor, as a processor storing into the tensor does.
"""
import numpy as np


def _bf16_round(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    out = ((u + bias) >> np.uint32(16)) << np.uint32(16)
    out = out.astype(np.uint32)
    out[np.isnan(a)] = 0x7FC00000
    return out.view(np.float32)


def storage_round(a, kind):
    """fp32 values as they read back after a store to `kind` in {"f32", "f16", "bf16"}."""
    a = np.asarray(a, dtype=np.float32)
    if kind == "f32":
        return a
    if kind == "f16":
        with np.errstate(over="ignore"):
            return a.astype(np.float16).astype(np.float32)
    if kind == "bf16":
        return _bf16_round(a)
    raise ValueError(kind)


def last_position(logits):
    """View of what a processor may touch: [batch, vocab] of a rank-2 tensor, the last sequence
    position of a rank-3 one (float_data_at_last_position, test_logit_processor.cpp:29-35)."""
    if logits.ndim == 2:
        return logits
    if logits.ndim == 3:
        return logits[:, -1, :]
    raise ValueError("rank must be 2 or 3")


def add_bias(logits, bias, kind="f32"):
    rows = last_position(logits)
    rows[...] = storage_round(rows + np.float32(bias), kind)


def scale(logits, factor, kind="f32"):
    rows = last_position(logits)
    rows[...] = storage_round(rows * np.float32(factor), kind)


def mask(logits, tokens, kind="f32"):
    rows = last_position(logits)
    vocab = rows.shape[-1]
    for t in np.atleast_1d(tokens):
        if 0 <= t < vocab:
            rows[:, t] = -np.inf


def token_bias(logits, tokens, bias, kind="f32"):
    rows = last_position(logits)
    vocab = rows.shape[-1]
    for t, b in zip(tokens, bias):
        if 0 <= t < vocab:
            rows[:, t] = storage_round(rows[:, t] + np.float32(b), kind)


def repetition_penalty(logits, penalty, history, lengths, kind="f32"):
    rows = last_position(logits)
    vocab = rows.shape[-1]
    p = np.float32(penalty)
    for b in range(rows.shape[0]):
        for t in sorted(set(int(v) for v in history[b, :lengths[b]])):
            if 0 <= t < vocab:
                x = np.float32(rows[b, t])
                y = np.float32(x * p) if x < 0 else np.float32(x / p)
                rows[b, t] = storage_round(np.array([y], dtype=np.float32), kind)[0]
