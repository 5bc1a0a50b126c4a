"""Per-row sampling parameters (the batched counterpart of SamplingConfig, llm_session.h:29-34)
through the C ABI: every row must come out as a reference sampler built with that row's
parameters would sample it, whatever else shares the batch."""
import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import _capi
from executorch_amd import workloads as W
from util import f32_bits, to_device

pytestmark = pytest.mark.gpu


def oracle_rows(oracle, x, dtype, cfgs, default_temperature, states):
    """Row by row with the oracle; `states` is advanced in place."""
    want = np.empty(len(cfgs), dtype=np.int32)
    explain = []
    for b, (t, topp, topk, seed) in enumerate(cfgs):
        if seed:
            states[b] = seed
        temperature = default_temperature if t < 0 else t
        tok, ex = oracle.sample_rows(x[b:b + 1], dtype, oracle.inv_temperature(temperature), topp, topk, states[b:b + 1],
                                     mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, explain=True)
        want[b] = tok[0]
        explain.append(ex[0])
    return want, explain


@pytest.mark.parametrize("name,rows", [("cfg2", 24), ("cfg1", 9)])
def test_mixed_batch_matches_per_row_samplers(oracle, dev, name, rows):
    w = W.WORKLOADS[name]
    menu = [(-1.0, 0.9, 0, 0), (0.0, 0.9, 0, 0), (0.6, 0.9, 0, 0), (1.0, 1.0, 0, 0), (0.8, 0.0, 0, 0), (0.7, 0.9, 5, 0),
            (1.3, 0.5, 0, 12345), (0.0, 1.0, 3, 777), (0.9, 0.95, 40, 99), (0.6, 0.3, 0, 0), (2.0, 1.0, 0, 31337)]
    cfgs = [menu[(3 * b + 1) % len(menu)] for b in range(rows)]
    default_temperature = 0.75
    s = ea.Sampler(w.vocab, default_temperature, 0.5, 5000, max_batch=rows)
    states = (np.uint64(5000) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    for step in range(3):
        x = W.logits(w, step, rows)
        if step == 1:
            cfgs = [(t, p, k, 0) for (t, p, k, _) in cfgs]  # streams continue
        if step == 2:
            cfgs = cfgs[1:] + cfgs[:1]  # rows change group
        ddbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
        got = s.sample_batch_configs(to_device(x, w.dtype, dev), cfgs, debug_out=ddbg).cpu().numpy()
        want, ex = oracle_rows(oracle, x, w.dtype, cfgs, default_temperature, states)
        assert np.array_equal(got, want), (name, step, np.nonzero(got != want)[0], got, want)
        assert np.array_equal(s.get_rng_states(rows), states), (name, step)
        dbg = ea.debug_records(ddbg)
        for b in range(rows):
            if ex[b].branch in (oracle.BRANCH_TOPP, oracle.BRANCH_TOPK):
                assert f32_bits(dbg["sum"][b]) == f32_bits(ex[b].sum)
                assert dbg["n_candidates"][b] == ex[b].n_candidates
                assert dbg["position"][b] == ex[b].position


@pytest.mark.parametrize("rows,greedy_every", [(16, 0), (64, 0), (24, 3)])
def test_top_p_rows_with_parameters_of_their_own(oracle, dev, rows, greedy_every):
    """Only top-p rows (and, in one case, greedy ones between them, so that the drawing rows are reached
    through the row map): the launch in which the workgroups of a row exchange their maxima and sums
    inside one kernel reads every row's own temperature and top-p."""
    w = W.WORKLOADS["cfg2"]
    cfgs = []
    for b in range(rows):
        if greedy_every and b % greedy_every == 1:
            cfgs.append((0.0, 0.9, 0, 0))
        else:
            cfgs.append((0.5 + 0.05 * (b % 9), 0.7 + 0.03 * (b % 8), 0, 0))
    s = ea.Sampler(w.vocab, 0.33, 0.5, 900, max_batch=rows)
    states = (np.uint64(900) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    for step in range(2):
        x = W.logits(w, step, rows)
        ddbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
        got = s.sample_batch_configs(to_device(x, w.dtype, dev), cfgs, debug_out=ddbg).cpu().numpy()
        want, ex = oracle_rows(oracle, x, w.dtype, cfgs, 0.33, states)
        assert np.array_equal(got, want), (rows, step, np.nonzero(got != want)[0])
        assert np.array_equal(s.get_rng_states(rows), states)
        dbg = ea.debug_records(ddbg)
        for b in range(rows):
            if ex[b].branch == oracle.BRANCH_TOPP:
                assert f32_bits(dbg["sum"][b]) == f32_bits(ex[b].sum)


def test_unchanged_parameters_are_not_uploaded_again_but_changed_ones_are(oracle, dev):
    """A call whose parameters equal the previous call's reuses the device copy.  That copy is also what a
    Gumbel-max call with one temperature per row writes to, and a call on another stream reads it: in both
    cases, and whenever a parameter changes, the rows must still be sampled with their own parameters."""
    w = W.WORKLOADS["cfg2"]
    rows = 12
    cfgs = [(0.5 + 0.1 * (b % 5), 0.8 + 0.02 * (b % 4), 0, 0) for b in range(rows)]
    s = ea.Sampler(w.vocab, 0.9, 0.5, 4100, max_batch=rows)
    states = (np.uint64(4100) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    other = torch.cuda.Stream()

    def check(step, c):
        x = W.logits(w, step, rows)
        got = s.sample_batch_configs(to_device(x, w.dtype, dev), c).cpu().numpy()
        want, _ = oracle_rows(oracle, x, w.dtype, c, 0.9, states)
        assert np.array_equal(got, want), (step, np.nonzero(got != want)[0])
        assert np.array_equal(s.get_rng_states(rows), states)

    check(0, cfgs)
    check(1, cfgs)  # (nothing to upload)
    x = to_device(W.logits(w, 2, rows), w.dtype, dev)
    s.gumbel_max_batch(x, np.linspace(0.3, 1.4, rows, dtype=np.float32))  # (overwrites the device copy)
    states[:] = s.get_rng_states(rows)  # (its noise is keyed by the rows' coin states and moves them on)
    check(2, cfgs)
    changed = list(cfgs)
    changed[5] = (0.0, 0.9, 0, 0)  # one row turns greedy: another grouping, other row maps
    check(3, changed)
    check(4, cfgs)
    torch.cuda.synchronize()
    with torch.cuda.stream(other):
        check(5, cfgs)  # (the same parameters, on another stream)
        check(6, changed)
    torch.cuda.synchronize()


def test_work_buffers_do_not_depend_on_the_first_call(oracle, dev):
    """The work buffers of the several-workgroups-per-row path are allocated by the first call that needs
    them.  When that call runs two groups of rows side by side, each group gets fewer workgroups per row
    than it would alone; the buffers must still be sized for any later call (and for the second group of
    the same call, which runs beside fewer rows than the first).  A vocabulary large enough for the number
    of workgroups per row to depend on the number of rows (more than 16 x 32 slots)."""
    vocab, rows = 290000, 8
    rng = np.random.default_rng(77)
    x = (rng.standard_normal((rows, vocab)) * 2.0).astype(np.float32)
    s = ea.Sampler(vocab, 0.8, 0.9, 321, max_batch=rows)
    states = (np.uint64(321) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    dx = to_device(W.to_storage(x, W.DTYPE_BFLOAT16), W.DTYPE_BFLOAT16, dev)
    xs = W.to_storage(x, W.DTYPE_BFLOAT16)
    mixed = [(1.0, 1.0, 0, 0)] * 3 + [(0.7, 0.9, 0, 0)] * 5  # three multinomial rows beside five top-p rows
    alone = [(0.7, 0.9, 0, 0)] * rows
    for cfgs in (mixed, alone, mixed):
        got = s.sample_batch_configs(dx, cfgs).cpu().numpy()
        want, _ = oracle_rows(oracle, xs, W.DTYPE_BFLOAT16, cfgs, 0.8, states)
        assert np.array_equal(got, want), (np.nonzero(got != want)[0], got, want)
        assert np.array_equal(s.get_rng_states(rows), states)


def test_uniform_configs_equal_the_plain_batch(dev):
    w = W.WORKLOADS["cfg2"]
    rows = 16
    x = to_device(W.logits(w, 0, rows), w.dtype, dev)
    a = ea.Sampler(w.vocab, w.temperature, w.topp, 42, max_batch=rows)
    b = ea.Sampler(w.vocab, 0.123, 0.456, 42, max_batch=rows)
    plain = a.sample_batch(x).cpu().numpy()
    cfg = b.sample_batch_configs(x, [(w.temperature, w.topp, 0, 0)] * rows).cpu().numpy()
    assert np.array_equal(plain, cfg)
    assert np.array_equal(a.get_rng_states(), b.get_rng_states())


def test_config_errors(dev):
    s = ea.Sampler(64, 1.0, 0.9, 1, max_batch=4)
    x = torch.zeros((4, 64), device=dev)
    with pytest.raises(ea.SamplerError):
        s.sample_batch_configs(x, [(1.0, 0.9, 0, 0)] * 3)
    u16 = torch.zeros((4, 64), dtype=torch.int16, device=dev)
    # greedy rows of UInt16 logits are fine, stochastic ones are refused
    assert s.sample_batch_configs(u16, [(0.0, 0.9, 0, 0)] * 4, dtype=_capi.DTYPE_UINT16).cpu().tolist() == [0, 0, 0, 0]
    with pytest.raises(ea.SamplerError) as e:
        s.sample_batch_configs(u16, [(0.0, 0.9, 0, 0)] * 3 + [(1.0, 0.9, 0, 0)], dtype=_capi.DTYPE_UINT16)
    assert e.value.code == _capi.NOT_SUPPORTED
