"""The logit-processor restatement (oracle/logit_processor_oracle.py) against the expected values
of the reference's own tests, extension/llm/sampler/test/test_logit_processor.cpp:109-212."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
from oracle import logit_processor_oracle as lpo  # noqa: E402


def test_single_processor_mutates_logits():  # :109-121
    x = np.array([[1, 2, 3, 4]], dtype=np.float32)
    lpo.add_bias(x, 10.0)
    assert x[0, 0] == 11.0 and x[0, 3] == 14.0


def test_chain_applies_in_order():  # :125-143
    x = np.array([[1, 2, 3, 4]], dtype=np.float32)
    lpo.scale(x, 2.0)
    lpo.add_bias(x, 1.0)
    assert x.tolist() == [[3.0, 5.0, 7.0, 9.0]]


def test_mask_token():  # :147-161 and :165-184
    x = np.array([[0.1, 0.2, 0.99, 0.4]], dtype=np.float32)
    lpo.mask(x, 2)
    assert x[0, 2] == -np.inf and np.argmax(x) == 3
    assert x[0, 0] == np.float32(0.1) and x[0, 1] == np.float32(0.2) and x[0, 3] == np.float32(0.4)
    y = np.array([[1, 2, 3]], dtype=np.float32)
    lpo.mask(y, 99)
    lpo.mask(y, -1)
    assert y.tolist() == [[1.0, 2.0, 3.0]]


def test_last_position_of_rank3():  # :186-212
    x = np.array([[[99, 99, 99, 99], [1, 2, 3, 4]]], dtype=np.float32)
    lpo.add_bias(x, 10.0)
    assert x[0, 0].tolist() == [99.0] * 4
    assert x[0, 1].tolist() == [11.0, 12.0, 13.0, 14.0]


def test_repetition_and_token_bias_by_hand():
    x = np.array([[2.0, -2.0, 0.0, 8.0, 1.0]], dtype=np.float32)
    history = np.array([[0, 1, 0, 2, 7, 3]], dtype=np.int32)
    lpo.repetition_penalty(x, 2.0, history, np.array([5]))  # token 3 lies beyond the length, 7 out of range
    assert x.tolist() == [[1.0, -4.0, 0.0, 8.0, 1.0]]
    lpo.token_bias(x, [4, 4, 9], [0.5, 0.25, 1.0])
    assert x[0, 4] == 1.75
    bf = np.array([[1.0, 1.0]], dtype=np.float32)
    lpo.add_bias(bf, 2.0 ** -9, kind="bf16")  # a quarter of bf16's ulp at 1 (2^-7): stays 1
    assert bf.tolist() == [[1.0, 1.0]]
    lpo.add_bias(bf, 3 * 2.0 ** -9, kind="bf16")  # three quarters of an ulp: rounds up to 1 + 2^-7
    assert bf.tolist() == [[1.0078125, 1.0078125]]
