"""xorshift64* known answers (closed form of sampler.cpp:210-220, cross-checked against the
compiled reference when the fixtures were made) and the closed-form multinomial draws that
follow from them."""
import ctypes as C

import numpy as np
import pytest

KATS = {
    42: [(0x56CE4AB7, 0.3390852212905884), (0xC841EB53, 0.7822558283805847), (0xCA466BE0, 0.790136992931366),
         (0xF1ACC733, 0.9440426230430603)],
    1: [(0x47E4CE4B, 0.28083503246307373), (0xABCFA6A8, 0.6711372137069702), (0xB9D10D8F, 0.7258461117744446),
        (0x4DB418A0, 0.3035292625427246)],
    7: [(0xD1FBAF7F, 0.8202466368675232), (0xEDA46C77, 0.9282901287078857), (0x16DF9D6A, 0.08934956789016724),
        (0x1B8D7895, 0.10762739181518555)],
    99: [(0x4C0AB4D5, 0.29703831672668457), (0xFB83E09B, 0.9824810028076172), (0xEF8AACF1, 0.9357097148895264),
         (0xDD7338A7, 0.8650393486022949)],
    123: [(0x56EC19CE, 0.3395400643348694), (0x24A228DC, 0.14309930801391602), (0x6D25258F, 0.4263480305671692),
          (0xA40A4AFB, 0.6407819986343384)],
}


def py_xorshift(state: int):
    """Independent restatement in Python integers."""
    m = (1 << 64) - 1
    state ^= state >> 12
    state ^= (state << 25) & m
    state ^= state >> 27
    return state, ((state * 0x2545F4914F6CDD1D) & m) >> 32


@pytest.mark.parametrize("seed", sorted(KATS))
def test_u32_and_coin_kats(oracle, seed):
    st = C.c_uint64(seed)
    st2 = C.c_uint64(seed)
    for u32, coin in KATS[seed]:
        assert oracle.lib().oracle_random_u32(C.byref(st)) == u32
        got = oracle.lib().oracle_random_f32(C.byref(st2))
        assert got == np.float32(coin)
        assert got == np.float32((u32 >> 8) / 16777216.0)


def test_state_after_first_coin(oracle):
    st = C.c_uint64(42)
    oracle.lib().oracle_random_u32(C.byref(st))
    assert st.value == 0x54000020


def test_seed_zero_is_a_fixed_point(oracle):
    st = C.c_uint64(0)
    for _ in range(5):
        assert oracle.lib().oracle_random_f32(C.byref(st)) == 0.0
        assert st.value == 0


def test_matches_python_integers(oracle):
    rng = np.random.default_rng(5)
    for seed in [int(v) for v in rng.integers(1, 2**63, size=50, dtype=np.uint64)]:
        st = C.c_uint64(seed)
        s = seed
        for _ in range(20):
            s, u = py_xorshift(s)
            assert oracle.lib().oracle_random_u32(C.byref(st)) == u
            assert st.value == s


@pytest.mark.parametrize("seed,expected", [(42, [1388, 3204, 3236, 3866]), (1, [1150, 2748, 2973, 1243]),
                                           (0, [0, 0, 0, 0])])
def test_uniform_logits_closed_form(oracle, seed, expected):
    """V = 4096 equal logits: every p is exactly 2^-12, so the multinomial draw is
    floor(coin * V); the expected tokens were also observed on the compiled reference."""
    V = 4096
    s = oracle.Sampler(V, 1.0, 1.0, seed)
    got = []
    for _ in range(4):
        x = np.zeros(V, dtype=np.float32)
        got.append(s.sample(x))
        assert np.all(x == np.float32(2.0 ** -12))
    assert got == expected
    st = seed
    for t in got:
        st, u = py_xorshift(st)
        assert t == int(((u >> 8) / 16777216.0) * V)


def test_four_logit_known_answer(oracle):
    """{0.1, 0.2, 0.8, 0.4}, T = 1, top-p 0.9, seed 42 on the compiled reference: token 2 and
    these probabilities left in the buffer."""
    x = np.array([0.1, 0.2, 0.8, 0.4], dtype=np.float32)
    s = oracle.Sampler(4, 1.0, 0.9, 42)
    assert s.sample(x) == 2
    want = np.array([0.182856068, 0.202087194, 0.368226916, 0.246829867], dtype=np.float32)
    assert np.array_equal(x, want)
