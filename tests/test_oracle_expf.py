"""The restated glibc expf (what the GPU evaluates) against this machine's libm expf.  The
exhaustive sweep over all 2^32 inputs is oracle/expf_sweep.c (about a minute); here: every
float in a few dense windows, a stride over the whole negative axis, and the special cases."""
import numpy as np


def both(oracle, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    a, b = np.empty_like(x), np.empty_like(x)
    oracle.lib().oracle_expf_restated_many(x.ctypes.data, a.ctypes.data, x.size)
    oracle.lib().oracle_expf_libm_many(x.ctypes.data, b.ctypes.data, x.size)
    return a, b


def same(a, b):
    return (a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))


def test_stride_over_all_floats(oracle):
    bits = np.arange(0, 2**32, 1021, dtype=np.uint64).astype(np.uint32)
    a, b = both(oracle, bits.view(np.float32))
    assert same(a, b).all()


def test_dense_windows(oracle):
    for lo in (-1.0, -16.7, -20.0, -87.5, -103.0, -104.1, -1e-3, 0.5, 88.0):
        start = np.float32(lo).view(np.uint32)
        bits = (np.uint64(start) + np.arange(0, 1 << 20, dtype=np.uint64)).astype(np.uint32)
        a, b = both(oracle, bits.view(np.float32))
        assert same(a, b).all()


def test_special_cases(oracle):
    x = np.array([0.0, -0.0, -np.inf, np.inf, np.nan, -88.0, -103.97207, -103.972084, -150.0, 88.72283, 88.72284, 100.0,
                  1e-30, -1e-30], dtype=np.float32)
    a, b = both(oracle, x)
    assert same(a, b).all()
    assert a[2] == 0.0 and a[0] == 1.0 and np.isinf(a[3])


def test_table_matches_exact_arithmetic(oracle):
    """tab[i] = bits(2^(i/32) correctly rounded) - (i << 47), checked with integers."""
    tab = np.zeros(32, dtype=np.uint64)
    oracle.lib().oracle_exp2_table(tab.ctypes.data)
    for i in range(32):
        target = 1 << (i + 52 * 32 + 32)  # (2^(i/32) * 2^52 * 2)^32
        m = int(round(2.0 ** (i / 32) * 2**52))
        found = None
        for c in range(m - 3, m + 4):
            if (2 * c - 1) ** 32 < target <= (2 * c + 1) ** 32:
                found = c
        assert found is not None
        assert int(tab[i]) == (0x3FF << 52) + (found - (1 << 52)) - (i << 47)
