"""Sampling time in microseconds (the reference's Stats keeps whole milliseconds,
extension/llm/runner/stats.h:46-47, :62-69)."""
import time

import pytest
import torch

import executorch_amd as ea
from executorch_amd import workloads as W
from util import to_device

pytestmark = pytest.mark.gpu


def test_timing_counts_calls_rows_and_microseconds(dev):
    w = W.WORKLOADS["cfg2"]
    rows = 16
    x = to_device(W.logits(w, 0, rows), w.dtype, dev)
    s = ea.Sampler(w.vocab, w.temperature, w.topp, 3, max_batch=rows)
    s.sample_batch(x)
    assert s.stats() == {"calls": 0, "rows": 0, "aggregate_sampling_time_us": 0.0, "last_call_us": 0.0}  # off by default
    s.set_timing(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(40):  # more calls than the event ring holds
        if i % 2:
            s.sample_batch(x)
        else:
            s.sample_batch_configs(x[:8], [(0.8, 0.9, 0, 0)] * 8)
    st = s.stats()
    wall_us = (time.perf_counter() - t0) * 1e6
    assert st["calls"] == 40 and st["rows"] == 20 * 16 + 20 * 8
    assert 40 * 10.0 < st["aggregate_sampling_time_us"] <= wall_us
    assert 10.0 < st["last_call_us"] < 5000.0  # a few dozen microseconds: invisible at millisecond resolution
    s.set_timing(False)
    s.sample_batch(x)
    assert s.stats()["calls"] == 40
    s.reset_stats()
    assert s.stats()["calls"] == 0 and s.stats()["aggregate_sampling_time_us"] == 0.0
