"""Device building blocks in isolation, through the library's test hooks: the bit-faithful
expf against libm, and the sequential-sum emulation against the scalar loop."""
import numpy as np
import pytest
import torch

from executorch_amd import _capi
from util import seq_sum_f32

pytestmark = pytest.mark.gpu


def gpu_expf(x, dev):
    dx = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev)
    dy = torch.empty_like(dx)
    assert _capi.hooks().ets_test_expf(dx.data_ptr(), dy.data_ptr(), dx.numel(), None) == _capi.OK
    torch.cuda.synchronize()
    return dy.cpu().numpy()


def libm_expf(oracle, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    oracle.lib().oracle_expf_libm_many(x.ctypes.data, y.ctypes.data, x.size)
    return y


def test_expf_every_negative_float_by_stride(oracle, dev):
    """Every 61st bit pattern of the negative axis and of [0, 89): 4.4e7 inputs, bit-exact."""
    neg = (np.uint64(0x80000000) + np.arange(0, 0x7F800001, 61, dtype=np.uint64)).astype(np.uint32)
    pos = np.arange(0, 0x42B20000, 61, dtype=np.uint64).astype(np.uint32)
    for bits in (neg, pos):
        x = bits.view(np.float32)
        a, b = gpu_expf(x, dev), libm_expf(oracle, x)
        ok = (a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))
        assert ok.all(), (x[~ok][:5], a[~ok][:5], b[~ok][:5])


def test_expf_dense_windows_and_specials(oracle, dev):
    xs = []
    for lo in (-1.0, -16.7, -17.4, -87.4, -103.2, -104.0, -1e-4):
        start = np.float32(lo).view(np.uint32)
        xs.append((np.uint64(start) + np.arange(0, 1 << 21, dtype=np.uint64)).astype(np.uint32).view(np.float32))
    xs.append(np.array([0.0, -0.0, -np.inf, np.inf, np.nan, -88.0, -103.97207, -103.972084, -150.0, 88.72283, 88.72284],
                       dtype=np.float32))
    x = np.concatenate(xs)
    a, b = gpu_expf(x, dev), libm_expf(oracle, x)
    ok = (a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))
    assert ok.all()


def gpu_seq_sum(a, s0, thr, dev):
    da = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dev)
    ds = torch.zeros(1, device=dev)
    dstop = torch.zeros(1, dtype=torch.int32, device=dev)
    st = _capi.hooks().ets_test_seq_sum(da.data_ptr(), da.numel(), float(s0), float(thr), ds.data_ptr(), dstop.data_ptr(), None)
    assert st == _capi.OK
    torch.cuda.synchronize()
    return np.float32(ds.item()), int(dstop.item())


def inputs(kind, n, rng):
    if kind == "wide":
        return np.exp(rng.uniform(-30, 0, n)).astype(np.float32)
    if kind == "edge":
        return np.exp(rng.uniform(-18, -15, n)).astype(np.float32)
    if kind == "pow2":
        return np.ldexp(np.float32(1), -rng.integers(0, 40, n)).astype(np.float32)
    if kind == "fewbits":
        return np.ldexp(rng.integers(1, 8, n).astype(np.float32), -rng.integers(0, 30, n)).astype(np.float32)
    if kind == "peaked":
        a = np.exp(rng.uniform(-25, -14, n)).astype(np.float32)
        hot = rng.random(n) < 0.02
        a[hot] = rng.uniform(0.1, 1.0, hot.sum()).astype(np.float32)
        return a
    if kind == "denormal":
        a = np.ldexp(rng.integers(0, 4096, n).astype(np.float32), (-149 + rng.integers(0, 30, n)).astype(np.int32)).astype(np.float32)
        a[rng.random(n) < 0.3] = 0
        return a
    if kind == "flat":
        return np.full(n, np.float32(1.0) / np.float32(n), dtype=np.float32)
    if kind == "bulk":  # small, similar addends: binade crossings far apart, as in the body of a softmax row
        return rng.uniform(1e-7, 3e-6, n).astype(np.float32)
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["wide", "edge", "pow2", "fewbits", "peaked", "denormal", "flat", "bulk"])
def test_seq_sum_matches_scalar_loop(dev, kind):
    rng = np.random.default_rng([7, len(kind)])
    for n in (1, 3, 64, 4095, 4096, 4097, 8192, 12345, 40000, 150001):
        a = inputs(kind, n, rng)
        total, _ = seq_sum_f32(a)
        for s0, thr in ((0.0, np.inf), (0.0, float(total) * 0.37), (0.0, 0.0), (0.75, float(total) + 0.5), (0.0, float(total))):
            want = seq_sum_f32(a, s0, thr)
            got = gpu_seq_sum(a, s0, thr, dev)
            assert got[0].view(np.uint32) == want[0].view(np.uint32) and got[1] == want[1], (kind, n, s0, thr, got, want)


def test_seq_sum_half_ulp_ties(dev):
    for k in range(8):
        a = np.full(9000, np.float32(2.0 ** -24), dtype=np.float32)
        a[0] = np.float32(1.0) + np.float32((k & 1) * 2.0 ** -23)
        a[17] = np.float32(3 * 2.0 ** -24)
        a[k * 1000 + 20] = np.float32(2.0 ** -23)
        want = seq_sum_f32(a)
        got = gpu_seq_sum(a, 0.0, np.inf, dev)
        assert got[0].view(np.uint32) == want[0].view(np.uint32)


def test_seq_sum_rounding_drift_defeats_prediction(dev):
    """Addends just above half an ulp of the running sum: every add rounds UP to a whole ulp, so
    the sequential sum runs ahead of any plain sum of the same numbers and leaves its binade tens
    of thousands of elements before an estimate from plain sums says so.  Whatever a kernel
    predicts from such estimates has to be caught by its exact checks."""
    for s0, addend, n in ((1.98, 0.6 * 2.0 ** -23, 300000), (0.99, 0.55 * 2.0 ** -24, 400000), (3.97, 0.7 * 2.0 ** -22, 250000)):
        a = np.full(n, np.float32(addend), dtype=np.float32)
        for thr in (np.inf, s0 * 1.009):
            want = seq_sum_f32(a, s0, thr)
            got = gpu_seq_sum(a, s0, thr, dev)
            assert got[0].view(np.uint32) == want[0].view(np.uint32) and got[1] == want[1], (s0, addend, n, thr, got, want)
    # and just below half an ulp: every add is absorbed, the plain sums grow
    a = np.full(300000, np.float32(0.49 * 2.0 ** -23), dtype=np.float32)
    a[0] = np.float32(1.99)
    want = seq_sum_f32(a)
    got = gpu_seq_sum(a, 0.0, np.inf, dev)
    assert got[0].view(np.uint32) == want[0].view(np.uint32), (got, want)
    assert want[0] == np.float32(1.99)
