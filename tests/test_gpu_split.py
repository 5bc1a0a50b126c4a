"""The path that spreads a row over several workgroups (three launches: slot maxima and approximate
sums; exact exponentials folded per slot under the predicted binade; one workgroup per row that
composes, verifies and draws) against the CPU oracle and against the one-workgroup-per-row kernel.
Bit-exact: tokens, coin states, the sequential softmax sum, the nucleus mass and positions."""
import numpy as np
import pytest
import torch

import executorch_amd as ea
from executorch_amd import workloads as W
import test_gpu_sampler_parity as parity
from util import f32_bits, to_device

pytestmark = pytest.mark.gpu

SPLIT_ON, SPLIT_OFF = 1, 2


@pytest.fixture
def forced_split(monkeypatch):
    monkeypatch.setenv("ETS_ROW_SPLIT", "1")  # the default of ets_sampler_set_row_split() for new handles


@pytest.mark.parametrize("name,rows,steps", [("cfg1", 1, 20), ("cfg2", 64, 2), ("cfg3", 4, 1), ("cfg5", 8, 1)])
def test_workloads_bit_exact_when_split(oracle, dev, forced_split, name, rows, steps):
    parity.run_case(oracle, dev, W.WORKLOADS[name], rows, steps, probs=(name == "cfg2"))


def test_small_and_ragged_vocabularies_when_split(oracle, dev, forced_split):
    parity.test_small_and_ragged_vocabularies(oracle, dev)


@pytest.mark.parametrize("topp,temperature", [(0.5, 0.3), (0.99, 1.0), (0.05, 1.0), (0.9, 0.05), (0.9, 5.0)])
def test_parameter_sweep_when_split(oracle, dev, forced_split, topp, temperature):
    for name, rows in (("cfg1", 2), ("cfg2", 8)):
        parity.run_case(oracle, dev, W.WORKLOADS[name], rows, 1, topp=topp, temperature=temperature)


def sample_both(x, dtype, dev, V, temperature, topp, seed):
    rows = x.shape[0]
    res = []
    for mode in (SPLIT_ON, SPLIT_OFF):
        s = ea.Sampler(V, temperature, topp, seed, max_batch=rows)
        s.set_row_split(mode)
        dbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
        tok = s.sample_batch(to_device(x, dtype, dev), debug_out=dbg).cpu().numpy()
        res.append((tok, ea.debug_records(dbg).copy(), s.get_rng_states(rows)))
    return res


def assert_same(a, b):
    assert np.array_equal(a[0], b[0])
    assert np.array_equal(a[2], b[2])
    for field in ("max_val", "sum", "coin", "cumulative", "r"):
        assert np.array_equal(f32_bits(a[1][field]), f32_bits(b[1][field])), field
    for field in ("n_candidates", "last_idx", "position"):
        assert np.array_equal(a[1][field], b[1][field]), field


@pytest.mark.parametrize("dtype", [W.DTYPE_FLOAT, W.DTYPE_HALF, W.DTYPE_BFLOAT16])
def test_masked_and_degenerate_rows_match_the_one_workgroup_kernel(oracle, dev, dtype):
    """Rows with whole slots of -inf (token masks), a leading masked stretch (the sum stays 0 for
    thousands of entries), one surviving entry, NaN and +inf entries, equal logits (every entry ties),
    and a vocabulary that ends inside a slot."""
    rng = np.random.default_rng(5)
    V = 20000 + 37
    base = (rng.standard_normal((9, V)) * 1.5).astype(np.float32)
    base[0, :6000] = -np.inf
    base[1, 3000:15000] = -np.inf
    base[2, :] = -np.inf
    base[2, 12345] = 0.5
    base[3, 777] = np.nan
    base[4, 778] = np.inf
    base[5, :] = 0.25
    base[6, ::2] = -np.inf
    base[7, :] = -np.inf
    base[8, :512] = 30.0  # the sum leaves many binades inside the first slots
    x = W.to_storage(base, dtype)
    for topp in (0.9, 0.3):
        on, off = sample_both(x, dtype, dev, V, 0.7, topp, 77)
        assert_same(on, off)
        states = (np.uint64(77) + np.arange(9, dtype=np.uint64)).astype(np.uint64)
        want, _ = oracle.sample_rows(x, dtype, oracle.inv_temperature(0.7), topp, 0, states, mode=oracle.MODE_UPCAST,
                                     tie=oracle.TIE_STABLE)
        assert np.array_equal(on[0], want)
        assert np.array_equal(on[2], states)


def test_row_pitch_and_row_map_when_split(oracle, dev):
    """Rows at a pitch larger than the vocabulary (16-byte aligned, so the split path applies), and
    per-row parameters, which reach the kernels through a row map."""
    rng = np.random.default_rng(8)
    V, B, pitch = 50000, 6, 50048
    x = (rng.standard_normal((B, V)) * 2.0).astype(np.float32)
    buf = torch.zeros((B, pitch), dtype=torch.float32, device=dev)
    buf[:, :V] = torch.from_numpy(x).to(dev)
    s = ea.Sampler(V, 0.8, 0.9, 300, max_batch=B)
    s.set_row_split(SPLIT_ON)
    got = s.sample_batch(buf[:, :V]).cpu().numpy()
    states = (np.uint64(300) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
    want, _ = oracle.sample_rows(x, W.DTYPE_FLOAT, oracle.inv_temperature(0.8), 0.9, 0, states, mode=oracle.MODE_UPCAST,
                                 tie=oracle.TIE_STABLE)
    assert np.array_equal(got, want)
    # per-row parameters: top-p rows of different temperatures mixed with greedy and multinomial rows
    cfgs = [(0.8, 0.9, 0, 0), (0.0, 0.9, 0, 0), (0.5, 0.7, 0, 0), (1.0, 1.0, 0, 0), (1.3, 0.95, 0, 0), (0.8, 0.9, 5, 0)]
    s2 = ea.Sampler(V, 0.8, 0.9, 400, max_batch=B)
    s2.set_row_split(SPLIT_ON)
    got2 = s2.sample_batch_configs(buf[:, :V], cfgs).cpu().numpy()
    for b, (t, p, k, _) in enumerate(cfgs):
        o = oracle.Sampler(V, t, p, 400 + b, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE)
        o.set_topk(k)
        assert got2[b] == o.sample(x[b].copy(), W.DTYPE_FLOAT), b


@pytest.mark.parametrize("topp,topk", [(0.9, 0), (1.0, 0), (0.9, 30)])
@pytest.mark.parametrize("mode", [SPLIT_ON, SPLIT_OFF])
def test_more_rows_than_workgroups(oracle, dev, topp, topk, mode):
    """The row kernels launch no more workgroups than the GPU keeps resident and hand the other rows
    out from a counter that is 0 again after every launch: 700 rows, then 300 on the same handle,
    then 700 again, against the oracle (top-p, multinomial, top-k; both paths)."""
    V, rows = 9000, 700
    rng = np.random.default_rng(3)
    s = ea.Sampler(V, 0.8, topp, 41, max_batch=rows)
    s.set_row_split(mode)
    if topk:
        s.set_topk(topk)
    states = (np.uint64(41) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
    inv = oracle.inv_temperature(0.8)
    for n in (rows, 300, rows):
        x = (rng.standard_normal((n, V)) * 1.5).astype(np.float32)
        hot = rng.integers(0, V, size=(n, 6))
        np.put_along_axis(x, hot, np.take_along_axis(x, hot, 1) + 6.0, 1)
        got = s.sample_batch(to_device(x, W.DTYPE_FLOAT, dev)).cpu().numpy()
        st = states[:n].copy()
        want, _ = oracle.sample_rows(x, W.DTYPE_FLOAT, inv, topp, topk, st, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, threads=8)
        states[:n] = st
        assert np.array_equal(got, want), (n, np.nonzero(got != want)[0][:8])
        assert np.array_equal(s.get_rng_states(n), states[:n])


@pytest.mark.parametrize("dtype", [W.DTYPE_BFLOAT16, W.DTYPE_FLOAT, W.DTYPE_HALF])
def test_short_candidate_lists_do_not_change_tokens(oracle, dev, dtype):
    """A call without debug records lets pass 2 list only the largest candidates of a row whose
    largest entries carry the nucleus; a call with them lists every candidate.  Rows on which that
    matters: few to thousands of raised entries (in distinct slots, sharing slots, sharing a lane's
    eight entries, equal to each other), raised by little (the shortcut must not apply) or by much
    (the nucleus is one entry), nuclei of more than 64 entries, a nucleus that ends among equal
    probabilities, thousands of equal largest entries.  Tokens and coin states of both calls must be
    the oracle's."""
    rng = np.random.default_rng(21)
    V = 128256 if dtype == W.DTYPE_BFLOAT16 else 70001
    rows = []
    for k, boost in ((1, 14.0), (3, 9.0), (20, 8.0), (20, 3.0), (70, 7.0), (300, 7.0), (2500, 6.0), (9000, 5.0)):
        x = rng.standard_normal(V).astype(np.float32)
        ids = rng.choice(V, size=k, replace=False)
        x[ids] += boost
        rows.append(x)
    x = rng.standard_normal(V).astype(np.float32)  # raised entries side by side: one slot, some in one lane's eight
    x[40000:40012] += 9.0
    rows.append(x)
    x = rng.standard_normal(V).astype(np.float32)  # equal raised entries: the nucleus ends inside a run of ties
    x[rng.choice(V, size=40, replace=False)] = 7.5
    rows.append(x)
    x = rng.standard_normal(V).astype(np.float32)  # two groups of ties a power of two apart in probability
    x[rng.choice(V, size=16, replace=False)] = 8.0
    x[rng.choice(V, size=16, replace=False)] = 8.0 - np.float32(np.log(2.0))
    rows.append(x)
    x = np.full(V, -30.0, dtype=np.float32)  # almost everything negligible, 100 entries of falling size
    x[rng.choice(V, size=100, replace=False)] = np.linspace(0.0, -6.0, 100, dtype=np.float32)
    rows.append(x)
    x = np.full(V, -20.0, dtype=np.float32)  # thousands of equal largest entries: too many to list as "the largest"
    x[rng.choice(V, size=20000, replace=False)] = 6.0
    rows.append(x)
    x = rng.standard_normal(V).astype(np.float32)  # the raised entries packed into a few slots
    x[9000:12000] += 7.0
    rows.append(x)
    base = W.to_storage(np.stack(rows), dtype)
    B = base.shape[0]
    for temperature, topp in ((0.6, 0.9), (1.0, 0.5), (1.0, 0.99), (0.3, 0.9), (2.0, 0.95), (1.0, 0.01)):
        for seed in (5, 6, 7):
            states = (np.uint64(seed * 1000) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
            after = states.copy()  # (the oracle advances the states it is given)
            want, _ = oracle.sample_rows(base, dtype, oracle.inv_temperature(temperature), topp, 0, after,
                                         mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, threads=8)
            for with_debug in (False, True):
                s = ea.Sampler(V, temperature, topp, 1, max_batch=B)
                s.set_row_split(SPLIT_ON)
                s.set_rng_states(states)
                dbg = torch.zeros((B, 8), dtype=torch.int32, device=dev) if with_debug else None
                got = s.sample_batch(to_device(base, dtype, dev), debug_out=dbg).cpu().numpy()
                assert np.array_equal(got, want), (temperature, topp, seed, with_debug, np.nonzero(got != want)[0])
                assert np.array_equal(s.get_rng_states(B), after)


@pytest.mark.parametrize("dtype", [W.DTYPE_FLOAT, W.DTYPE_HALF])
def test_candidate_lists_longer_than_lds(oracle, dev, dtype):
    """Rows with more top-p candidates than the finish kernel's LDS holds (tens of thousands) and a
    nucleus that still fits its sort: the list continues in the workgroup's scratch row."""
    rng = np.random.default_rng(31)
    V = 128256
    B = 4
    for scale, temperature, topp in ((2.0, 0.8, 0.5), (3.0, 1.0, 0.9), (2.0, 0.8, 0.9)):
        x = W.to_storage((rng.standard_normal((B, V)) * scale).astype(np.float32), dtype)
        for with_debug in (True, False):
            states = (np.uint64(900) + np.arange(B, dtype=np.uint64)).astype(np.uint64)
            s = ea.Sampler(V, temperature, topp, 1, max_batch=B)
            s.set_row_split(SPLIT_ON)
            s.set_rng_states(states)
            dbg = torch.zeros((B, 8), dtype=torch.int32, device=dev) if with_debug else None
            got = s.sample_batch(to_device(x, dtype, dev), debug_out=dbg).cpu().numpy()
            want, ex = oracle.sample_rows(x, dtype, oracle.inv_temperature(temperature), topp, 0, states, mode=oracle.MODE_UPCAST,
                                          tie=oracle.TIE_STABLE, threads=4, explain=True)
            assert np.array_equal(got, want), (scale, temperature, topp, with_debug)
            assert np.array_equal(s.get_rng_states(B), states)
            if with_debug:
                rec = ea.debug_records(dbg)
                assert min(ex[b].n_candidates for b in range(B)) > 16384  # (the case this test is for)
                for b in range(B):
                    assert rec["n_candidates"][b] == ex[b].n_candidates
                    assert rec["last_idx"][b] == ex[b].last_idx


def topk_rows(kind, rows, V, rng):
    if kind == "normal":
        return rng.standard_normal((rows, V)).astype(np.float32)
    if kind == "peaked":
        x = rng.standard_normal((rows, V)).astype(np.float32)
        for b in range(rows):
            x[b, rng.choice(V, 20, replace=False)] += 8.0
        return x
    if kind == "few":  # a dozen distinct values: every bucket of the largest holds thousands of ties
        return rng.integers(0, 12, (rows, V)).astype(np.float32) * 0.5
    if kind == "flat":
        return (rng.standard_normal((rows, V)) * 0.1).astype(np.float32)
    if kind == "one":  # one entry carries the whole mass; the k-1 others are ties far below it
        x = np.full((rows, V), -30.0, dtype=np.float32)
        x[np.arange(rows), rng.integers(0, V, rows)] = 10.0
        return x
    assert kind == "masked"  # fewer finite entries than k in some rows, one NaN row
    x = np.full((rows, V), -np.inf, dtype=np.float32)
    for b in range(rows):
        n = (3, 39, 40, 41, 500, 5000)[b % 6]
        x[b, rng.choice(V, n, replace=False)] = rng.standard_normal(n).astype(np.float32) * 2.0
    x[rows - 1, 77] = np.nan
    return x


@pytest.mark.parametrize("dtype", [W.DTYPE_BFLOAT16, W.DTYPE_FLOAT, W.DTYPE_HALF])
@pytest.mark.parametrize("kind", ["normal", "peaked", "few", "flat", "one", "masked"])
def test_topk_rows_when_split(oracle, dev, dtype, kind):
    """Top-k rows (sampler.cpp:72-120) over several workgroups: the histogram buckets in which the
    slots' two largest exps first number k are listed and the finish kernel keeps the k largest of
    them.  Against the oracle (tokens, coin states) and against the one-workgroup kernel (debug
    records as well), for k = 1, 40, 200, the largest k that takes this path and one above it."""
    V, rows = 128256, 12
    rng = np.random.default_rng(17)
    x = W.to_storage(topk_rows(kind, rows, V, rng), dtype)
    dx = to_device(x, dtype, dev)
    inv = oracle.inv_temperature(0.8)
    for k in (1, 40, 200, 251, 252):
        res = []
        for mode in (SPLIT_ON, SPLIT_OFF):
            s = ea.Sampler(V, 0.8, 0.9, 23, max_batch=rows)
            s.set_topk(k)
            s.set_row_split(mode)
            plain = s.sample_batch(dx).cpu().numpy()
            dbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
            tok = s.sample_batch(dx, debug_out=dbg).cpu().numpy()
            res.append((tok, ea.debug_records(dbg).copy(), s.get_rng_states(rows), plain))
        assert_same(res[0], res[1])
        assert np.array_equal(res[0][3], res[1][3]), k
        states = (np.uint64(23) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
        for step in (3, 0):
            want, _ = oracle.sample_rows(x, dtype, inv, 0.9, k, states, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, threads=8)
            assert np.array_equal(res[0][step], want), (k, step)
        assert np.array_equal(res[0][2], states), k


@pytest.mark.parametrize("dtype", [W.DTYPE_BFLOAT16, W.DTYPE_FLOAT, W.DTYPE_HALF])
@pytest.mark.parametrize("kind", ["normal", "peaked", "few", "flat", "one", "masked"])
def test_multinomial_rows_when_split(oracle, dev, dtype, kind):
    """Multinomial rows (sampler.cpp:58-70) over several workgroups, five launches: the records of the
    sum of exp, its chain, the records of the sum of p = exp / sum, and a chain over those that stops
    where the running sum exceeds the coin.  Against the oracle (tokens, coin states) and against the
    one-workgroup kernel (debug records as well: the sum, the coin, the running sum at the stop),
    at three temperatures, four calls each so that the coins land in different parts of the rows."""
    V, rows = 128256, 12
    rng = np.random.default_rng(29)
    x = W.to_storage(topk_rows(kind, rows, V, rng), dtype)
    dx = to_device(x, dtype, dev)
    for temperature in (1.0, 0.6, 2.5):
        inv = oracle.inv_temperature(temperature)
        samplers = []
        for mode in (SPLIT_ON, SPLIT_OFF):
            s = ea.Sampler(V, temperature, 1.0, 31, max_batch=rows)
            s.set_row_split(mode)
            samplers.append(s)
        states = (np.uint64(31) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
        for call in range(4):
            res = []
            for s in samplers:
                dbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
                tok = s.sample_batch(dx, debug_out=dbg if call % 2 else None).cpu().numpy()
                res.append((tok, ea.debug_records(dbg).copy(), s.get_rng_states(rows)))
            assert_same(res[0], res[1])
            want, _ = oracle.sample_rows(x, dtype, inv, 1.0, 0, states, mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, threads=8)
            assert np.array_equal(res[0][0], want), (temperature, call)
            assert np.array_equal(res[0][2], states), (temperature, call)


@pytest.mark.parametrize("mode", [SPLIT_ON, SPLIT_OFF])
def test_nuclei_of_hundreds_to_thousands_of_keys(oracle, dev, mode):
    """fp32 rows whose nucleus holds from several hundred to several thousand keys: the selected keys
    are sorted by buckets of their probability (up to about 5000 keys), by the bitonic network beyond
    that and where a bucket would be long (many equal probabilities: the rows of a dozen distinct
    values), and the two CDF walks run over them.  Against the oracle: tokens, coin states, the
    nucleus' last index and mass, the position of the draw."""
    V, rows = 32000, 8
    rng = np.random.default_rng(41)
    kinds = {
        "normal": (rng.standard_normal((rows, V)) * 2.0).astype(np.float32),
        "few": rng.integers(0, 12, (rows, V)).astype(np.float32) * 0.5,
    }
    for kind, x in kinds.items():
        dx = to_device(x, W.DTYPE_FLOAT, dev)
        for temperature, topp in ((0.5, 0.9), (0.8, 0.9), (1.0, 0.95), (1.5, 0.9), (0.8, 0.5)):
            s = ea.Sampler(V, temperature, topp, 53, max_batch=rows)
            s.set_row_split(mode)
            dbg = torch.zeros((rows, 8), dtype=torch.int32, device=dev)
            got = s.sample_batch(dx, debug_out=dbg).cpu().numpy()
            rec = ea.debug_records(dbg)
            states = (np.uint64(53) + np.arange(rows, dtype=np.uint64)).astype(np.uint64)
            want, ex = oracle.sample_rows(x, W.DTYPE_FLOAT, oracle.inv_temperature(temperature), topp, 0, states,
                                          mode=oracle.MODE_UPCAST, tie=oracle.TIE_STABLE, explain=True, threads=8)
            assert np.array_equal(got, want), (kind, temperature, topp)
            assert np.array_equal(s.get_rng_states(rows), states)
            for b in range(rows):
                assert rec["last_idx"][b] == ex[b].last_idx, (kind, temperature, topp, b)
                assert rec["position"][b] == ex[b].position, (kind, temperature, topp, b)
                assert f32_bits(np.float32(rec["cumulative"][b])) == f32_bits(np.float32(ex[b].cumulative)), (kind, temperature, topp, b)


@pytest.mark.parametrize("setting", ["fused", "fused_one_read", "fused_nobody_waits", "three_launches"])
@pytest.mark.parametrize("name,rows", [("cfg2", 64), ("cfg2", 8), ("cfg2", 1), ("cfg5", 16), ("cfg3", 24), ("cfg1", 1), ("cfg4", 16), ("cfg4", 3)])
def test_pass1_inside_pass2(oracle, dev, monkeypatch, setting, name, rows):
    """Plain top-p launches (and the first of a multinomial row's two sweeps: cfg4) whose workgroups are all
    resident run pass 1 inside pass 2: the row's
    workgroups hand their slots' maxima and sums to one another through device memory, each record
    tagged with the launch's number, and read one another's a bounded number of times.  With the bound
    at 0 nobody waits: every workgroup works the whole row's maxima and sums out itself; with the
    bound at 1 some do and some do not.  Tokens and coin states must equal the oracle's either way,
    and those of the three separate launches.  The same handle serves every step, with other logits
    each time: the records of the step before are still where this step's are looked for."""
    if setting == "fused_nobody_waits":
        monkeypatch.setenv("ETS_FUSE_SPIN_LIMIT", "0")
    if setting == "fused_one_read":
        monkeypatch.setenv("ETS_FUSE_SPIN_LIMIT", "1")
    if setting == "three_launches":
        monkeypatch.setenv("ETS_FUSE", "0")
    w = W.WORKLOADS[name]
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)
    for step in range(3):
        x = W.logits(w, step, rows)
        states = s.get_rng_states(rows).copy()
        got = s.sample_batch(to_device(x, w.dtype, dev)).cpu().numpy()  # (no debug records: the fused launch)
        want, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states, mode=oracle.MODE_UPCAST,
                                     tie=oracle.TIE_STABLE, threads=8)
        assert np.array_equal(got, want), (setting, name, rows, step)
        assert np.array_equal(s.get_rng_states(rows), states)
        # fewer rows on the same handle
        if rows > 1:
            fewer = (rows + 1) // 2
            x2 = x[:fewer][::-1].copy()
            states2 = s.get_rng_states(fewer).copy()
            got2 = s.sample_batch(to_device(x2, w.dtype, dev)).cpu().numpy()
            want2, _ = oracle.sample_rows(x2, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states2, mode=oracle.MODE_UPCAST,
                                          tie=oracle.TIE_STABLE, threads=8)
            assert np.array_equal(got2, want2), (setting, name, rows, step, "second call")
            assert np.array_equal(s.get_rng_states(fewer), states2)


@pytest.mark.parametrize("name,rows", [("cfg2", 64), ("cfg2", 8)])
def test_fused_step_replayed_from_a_graph(oracle, dev, name, rows):
    """One call captured into a HIP graph and replayed: every replay runs the launch with pass 1 inside
    pass 2 with the same kernel arguments, so what tells this replay's hand-over from the last one's
    lives in device memory (the launch number, which the finish kernel advances).  Other logits are
    copied into the captured input before every replay, with the program's own eager work and
    synchronisations between replays; every replay against the oracle."""
    w = W.WORKLOADS[name]
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)
    x0 = W.logits(w, 0, rows)
    dx = to_device(x0, w.dtype, dev)
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        s.sample_batch(dx, out=out)  # (warm: buffers allocated, kernel attributes set)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            s.sample_batch(dx, out=out)
    torch.cuda.synchronize()
    for step in range(1, 5):
        x = W.logits(w, step, rows)
        dx.copy_(to_device(x, w.dtype, dev))
        states = s.get_rng_states(rows).copy()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        want, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states, mode=oracle.MODE_UPCAST,
                                     tie=oracle.TIE_STABLE, threads=8)
        assert np.array_equal(got, want), (name, rows, step)
        assert np.array_equal(s.get_rng_states(rows), states)
        # eager work of the same handle between the replays
        if step == 2:
            eager = s.sample_batch(dx).cpu().numpy()
            want2, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states, mode=oracle.MODE_UPCAST,
                                          tie=oracle.TIE_STABLE, threads=8)
            assert np.array_equal(eager, want2), (name, rows, step, "eager")


def test_a_launch_without_its_finish_kernel_does_not_lend_its_number(oracle, dev):
    """The workgroups of a launch with pass 1 inside pass 2 tag what they hand over with the launch's
    number, which the finish kernel advances.  A launch whose finish kernel was never issued (an error
    between the two) leaves the number as it was: the handle remembers, and the next such launch is given
    a number of its own before it starts.  Forced here through the test hook; tokens against the oracle."""
    import ctypes
    from executorch_amd import _capi
    w = W.WORKLOADS["cfg2"]
    rows = 8
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)

    def number(mark):
        out = ctypes.c_uint32(0)
        assert _capi.hooks().ets_test_fused_launch_number(s._h, mark, ctypes.byref(out)) == _capi.OK
        return out.value

    def step(k):
        x = W.logits(w, k, rows)
        states = s.get_rng_states(rows).copy()
        got = s.sample_batch(to_device(x, w.dtype, dev)).cpu().numpy()
        want, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states, mode=oracle.MODE_UPCAST,
                                     tie=oracle.TIE_STABLE, threads=8)
        assert np.array_equal(got, want), k
        assert np.array_equal(s.get_rng_states(rows), states)

    step(0)
    n1 = number(0)
    step(1)
    assert number(1) == n1 + 1  # (one launch, one number; and the handle is marked)
    step(2)
    assert number(0) == n1 + 3  # (a number skipped, then the launch's own)
    step(3)
    assert number(0) == n1 + 4


@pytest.mark.parametrize("setting", ["fused", "fused_one_read", "fused_nobody_waits", "three_launches"])
def test_pass1_inside_pass2_top_k_rows(oracle, dev, monkeypatch, setting):
    """The same for launches with top-k rows (sampler.cpp:72-120, :239): top-k 40 and top-k 3 with the
    workload's top-p, and top-k alone (top-p 1)."""
    if setting == "fused_nobody_waits":
        monkeypatch.setenv("ETS_FUSE_SPIN_LIMIT", "0")
    if setting == "fused_one_read":
        monkeypatch.setenv("ETS_FUSE_SPIN_LIMIT", "1")
    if setting == "three_launches":
        monkeypatch.setenv("ETS_FUSE", "0")
    w = W.WORKLOADS["cfg2"]
    rows = 16
    for topk, topp in ((40, w.topp), (3, w.topp), (40, 1.0)):
        s = ea.Sampler(w.vocab, w.temperature, topp, w.coin_seed, max_batch=rows)
        s.set_topk(topk)
        for step in range(2):
            x = W.logits(w, step, rows)
            states = s.get_rng_states(rows).copy()
            got = s.sample_batch(to_device(x, w.dtype, dev)).cpu().numpy()
            want, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), topp, topk, states, mode=oracle.MODE_UPCAST,
                                         tie=oracle.TIE_STABLE, threads=8)
            assert np.array_equal(got, want), (setting, topk, topp, step)
            assert np.array_equal(s.get_rng_states(rows), states)


def test_two_handles_on_two_streams_at_once(oracle, dev):
    """Two launches with pass 1 inside pass 2 at the same time, from two handles on two streams: each was
    sized to fill the compute units on its own, so the workgroups of one can hold the units that the other's
    are waiting for.  Nobody waits for ever (the reads of the others' records are bounded, and a workgroup
    that gives up works the row out itself): tokens and coin states equal the oracle's, call after call."""
    w = W.WORKLOADS["cfg2"]
    rows = 64
    a = ea.Sampler(w.vocab, w.temperature, w.topp, 11, max_batch=rows)
    b = ea.Sampler(w.vocab, w.temperature, w.topp, 22, max_batch=rows)
    xs = [W.logits(w, step, rows) for step in range(3)]
    dxs = [to_device(x, w.dtype, dev) for x in xs]
    sa, sb = torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)
    outs_a = [torch.empty(rows, dtype=torch.int32, device=dev) for _ in xs]
    outs_b = [torch.empty(rows, dtype=torch.int32, device=dev) for _ in xs]
    a.sample_batch(dxs[0], out=outs_a[0])  # (warm: buffers allocated, kernel attributes set)
    b.sample_batch(dxs[0], out=outs_b[0])
    torch.cuda.synchronize()
    states_a, states_b = a.get_rng_states(rows).copy(), b.get_rng_states(rows).copy()
    for k in range(len(xs)):
        with torch.cuda.stream(sa):
            a.sample_batch(dxs[k], out=outs_a[k])
        with torch.cuda.stream(sb):
            b.sample_batch(dxs[k], out=outs_b[k])
    torch.cuda.synchronize()
    for k, x in enumerate(xs):
        want_a, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states_a, mode=oracle.MODE_UPCAST,
                                       tie=oracle.TIE_STABLE, threads=8)
        want_b, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states_b, mode=oracle.MODE_UPCAST,
                                       tie=oracle.TIE_STABLE, threads=8)
        assert np.array_equal(outs_a[k].cpu().numpy(), want_a), ("a", k)
        assert np.array_equal(outs_b[k].cpu().numpy(), want_b), ("b", k)
    assert np.array_equal(a.get_rng_states(rows), states_a)
    assert np.array_equal(b.get_rng_states(rows), states_b)


def test_launch_numbers_come_round(oracle, dev):
    """After 2^32 - 1 launches the launch numbers start again; the number 0, for which the zeros that the
    records of never-used rows still hold would pass for records, is left out.  The word is set close to the
    end through the test hook; a small batch first, then the handle's full batch (rows whose records are
    still zeros) on the launches around the turn; tokens against the oracle."""
    import ctypes
    from executorch_amd import _capi
    w = W.WORKLOADS["cfg2"]
    rows = 16
    s = ea.Sampler(w.vocab, w.temperature, w.topp, w.coin_seed, max_batch=rows)

    def number():
        out = ctypes.c_uint32(0)
        assert _capi.hooks().ets_test_fused_launch_number(s._h, 0, ctypes.byref(out)) == _capi.OK
        return out.value

    def step(k, n):
        x = W.logits(w, k, n)
        states = s.get_rng_states(n).copy()
        got = s.sample_batch(to_device(x, w.dtype, dev)).cpu().numpy()
        want, _ = oracle.sample_rows(x, w.dtype, oracle.inv_temperature(w.temperature), w.topp, 0, states, mode=oracle.MODE_UPCAST,
                                     tie=oracle.TIE_STABLE, threads=8)
        assert np.array_equal(got, want), (k, n)

    step(0, 2)  # (the work buffers exist now; rows 2 .. 15 have never been used)
    assert _capi.hooks().ets_test_set_fused_launch_number(s._h, 0xFFFFFFFC) == _capi.OK
    seen = []
    for k in range(1, 6):
        step(k, rows if k >= 2 else 2)
        seen.append(number())
    assert seen == [0xFFFFFFFD, 0xFFFFFFFE, 0, 1, 2], [hex(v) for v in seen]


@pytest.mark.parametrize("topk", [1, 2, 7, 40, 63, 64, 65, 200])
def test_top_k_rows_with_short_lists(oracle, dev, topk):
    """A top-k row whose lists hold at most 64 entries (at least k of them) is drawn by the finish kernel's
    first wave alone; longer lists, and k beyond 64, take the steps of the whole workgroup.  Peaked rows,
    rows of few distinct values (ties at the k-th place, broken by index) and rows with a dominant entry,
    with top-p 0.9 and with top-p 1; tokens and coin states against the oracle."""
    V, rows = 128256, 8
    rng = np.random.default_rng(1000 + topk)
    peaked = (rng.standard_normal((rows, V)) * 1.0).astype(np.float32)
    for b in range(rows):
        peaked[b, rng.choice(V, size=24, replace=False)] += 8.0
    few = rng.integers(0, 6, (rows, V)).astype(np.float32)
    for b in range(rows):
        few[b, rng.choice(V, size=30, replace=False)] = 9.0  # (thirty equal largest entries)
    dominant = (rng.standard_normal((rows, V)) * 0.5).astype(np.float32)
    dominant[:, 77] = 30.0
    for kind, x32 in (("peaked", peaked), ("few", few), ("dominant", dominant)):
        x = W.to_storage(x32, W.DTYPE_BFLOAT16)
        dx = to_device(x, W.DTYPE_BFLOAT16, dev)
        for topp in (0.9, 1.0):
            s = ea.Sampler(V, 0.7, topp, 5 + topk, max_batch=rows)
            s.set_topk(topk)
            for step in range(2):
                states = s.get_rng_states(rows).copy()
                got = s.sample_batch(dx).cpu().numpy()
                want, _ = oracle.sample_rows(x, W.DTYPE_BFLOAT16, oracle.inv_temperature(0.7), topp, topk, states, mode=oracle.MODE_UPCAST,
                                             tie=oracle.TIE_STABLE, threads=8)
                assert np.array_equal(got, want), (kind, topk, topp, step)
                assert np.array_equal(s.get_rng_states(rows), states)
