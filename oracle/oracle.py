"""ctypes loader for the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg import this
module.  It wraps ``libsampler_oracle.so`` (the repo's restatement of the reference sampler,
``oracle/sampler_oracle.cpp``) and, where it has been built, ``_ref/libref_sampler.so`` (the
reference's own ``extension/llm/sampler/sampler.cpp`` compiled in place).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsampler_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libref_sampler.so")

DTYPE_HALF, DTYPE_FLOAT, DTYPE_BFLOAT16, DTYPE_UINT16 = 5, 6, 15, 27
MODE_NATIVE, MODE_UPCAST = 0, 1
TIE_LIBSTDCXX, TIE_STABLE = 0, 1
BRANCH_ARGMAX, BRANCH_MULTINOMIAL, BRANCH_TOPP, BRANCH_TOPK = 0, 1, 2, 3


class SamplerState(C.Structure):
    _fields_ = [
        ("vocab_size", C.c_int32),
        ("inv_temperature", C.c_float),
        ("topp", C.c_float),
        ("topk", C.c_int32),
        ("rng_state", C.c_uint64),
    ]


class Explain(C.Structure):
    _fields_ = [
        ("branch", C.c_int32),
        ("max_val", C.c_float),
        ("sum", C.c_float),
        ("coin", C.c_float),
        ("n_candidates", C.c_int32),
        ("last_idx", C.c_int32),
        ("cumulative", C.c_float),
        ("r", C.c_float),
        ("position", C.c_int32),
        ("p_token", C.c_float),
    ]


def build(force: bool = False) -> None:
    """Compile the oracle (and the reference build when /root/reference is mounted)."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", HERE, "-B" if force else "-s", "libsampler_oracle.so"])
    if os.path.isdir(os.environ.get("ET_REFERENCE_ROOT", "/root/reference")):
        if force or not os.path.exists(REF_PATH):
            subprocess.check_call([os.path.join(HERE, "build_ref.sh")])


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.oracle_random_u32.restype = C.c_uint32
        L.oracle_random_u32.argtypes = [C.POINTER(C.c_uint64)]
        L.oracle_random_f32.restype = C.c_float
        L.oracle_random_f32.argtypes = [C.POINTER(C.c_uint64)]
        L.oracle_sampler_init.restype = None
        L.oracle_sampler_init.argtypes = [C.POINTER(SamplerState), C.c_int32, C.c_float, C.c_float, C.c_uint64]
        L.oracle_sampler_set_temperature.restype = None
        L.oracle_sampler_set_temperature.argtypes = [C.POINTER(SamplerState), C.c_float]
        L.oracle_sampler_set_topk.restype = None
        L.oracle_sampler_set_topk.argtypes = [C.POINTER(SamplerState), C.c_int32]
        L.oracle_sample.restype = C.c_int32
        L.oracle_sample.argtypes = [C.POINTER(SamplerState), C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                    C.POINTER(Explain), C.c_void_p]
        L.oracle_sample_rows.restype = None
        L.oracle_sample_rows.argtypes = [C.c_int32, C.c_float, C.c_float, C.c_int32, C.c_void_p, C.c_int32,
                                         C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32,
                                         C.c_int32, C.c_void_p]
        L.oracle_sample_from_logits.restype = C.c_int32
        L.oracle_sample_from_logits.argtypes = [C.POINTER(SamplerState), C.c_void_p, C.c_int32, C.c_int32,
                                                C.POINTER(C.c_int64), C.c_int32, C.c_int32]
        L.oracle_exp2_table.restype = None
        L.oracle_exp2_table.argtypes = [C.c_void_p]
        L.oracle_expf_restated.restype = C.c_float
        L.oracle_expf_restated.argtypes = [C.c_float]
        for name in ("oracle_expf_restated_many", "oracle_expf_libm_many"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.oracle_bf16_from_float.restype = C.c_uint16
        L.oracle_bf16_from_float.argtypes = [C.c_float]
        L.oracle_bf16_to_float.restype = C.c_float
        L.oracle_bf16_to_float.argtypes = [C.c_uint16]
        L.oracle_half_from_float.restype = C.c_uint16
        L.oracle_half_from_float.argtypes = [C.c_float]
        L.oracle_half_to_float.restype = C.c_float
        L.oracle_half_to_float.argtypes = [C.c_uint16]
        _lib = L
    return _lib


def np_dtype_code(a: np.ndarray, dtype: int | None) -> int:
    if dtype is not None:
        return dtype
    if a.dtype == np.float32:
        return DTYPE_FLOAT
    if a.dtype == np.float16:
        return DTYPE_HALF
    raise ValueError("pass dtype= for uint16-stored rows (bfloat16 bits or quantised logits)")


class Sampler:
    """Mirror of ``Sampler(vocab_size, temperature, topp, rng_seed)`` on the oracle."""

    def __init__(self, vocab_size: int, temperature: float, topp: float = 0.9, rng_seed: int = 0,
                 mode: int = MODE_NATIVE, tie: int = TIE_LIBSTDCXX):
        self.s = SamplerState()
        lib().oracle_sampler_init(C.byref(self.s), vocab_size, temperature, topp, rng_seed)
        self.mode, self.tie = mode, tie
        self.explain = Explain()

    def set_temperature(self, t: float) -> None:
        lib().oracle_sampler_set_temperature(C.byref(self.s), t)

    def set_topk(self, k: int) -> None:
        lib().oracle_sampler_set_topk(C.byref(self.s), k)

    @property
    def rng_state(self) -> int:
        return int(self.s.rng_state)

    def sample(self, logits: np.ndarray, dtype: int | None = None, probs_out: np.ndarray | None = None) -> int:
        """Native mode overwrites ``logits`` with probabilities, like the reference."""
        assert logits.flags.c_contiguous and logits.size >= self.s.vocab_size
        code = np_dtype_code(logits, dtype)
        po = probs_out.ctypes.data if probs_out is not None else None
        return lib().oracle_sample(C.byref(self.s), logits.ctypes.data, code, self.mode, self.tie,
                                   C.byref(self.explain), po)


def sample_rows(logits: np.ndarray, dtype: int, inv_temperature: float, topp: float, topk: int,
                rng_states: np.ndarray, mode: int = MODE_UPCAST, tie: int = TIE_STABLE,
                explain: bool = False, threads: int = 1):
    """Sample every row of a [B, V] array; row b uses and advances ``rng_states[b]``.

    Returns (tokens[int32 B], explains or None).  ``threads`` > 1 splits rows over a thread
    pool (ctypes drops the GIL during the call; rows are independent).
    """
    assert logits.ndim == 2 and logits.flags.c_contiguous
    B, V = logits.shape
    assert rng_states.dtype == np.uint64 and rng_states.shape == (B,)
    tokens = np.empty(B, dtype=np.int32)
    ex = (Explain * B)() if explain else None
    exp_ptr = C.addressof(ex) if explain else None
    L = lib()

    def run(lo: int, hi: int) -> None:
        L.oracle_sample_rows(V, inv_temperature, topp, topk, logits.ctypes.data, dtype, V, lo, hi,
                             rng_states.ctypes.data, tokens.ctypes.data, mode, tie, exp_ptr)

    if threads <= 1 or B < 2:
        run(0, B)
    else:
        threads = min(threads, B)
        cuts = [B * i // threads for i in range(threads + 1)]
        with ThreadPoolExecutor(threads) as pool:
            list(pool.map(lambda i: run(cuts[i], cuts[i + 1]), range(threads)))
    return tokens, ex


def inv_temperature(temperature: float) -> float:
    """sampler.cpp:178 -- ``1.0f / temperature`` in float, 0 for temperature 0."""
    t = np.float32(temperature)
    return float(np.float32(1.0) / t) if t != 0 else 0.0


# ---------------------------------------------------------------------------------------
# the compiled reference (container only)


def have_ref() -> bool:
    return os.path.exists(REF_PATH)


_ref = None


def ref() -> C.CDLL:
    global _ref
    if _ref is None:
        R = C.CDLL(REF_PATH)
        R.ref_sampler_create.restype = C.c_void_p
        R.ref_sampler_create.argtypes = [C.c_int32, C.c_float, C.c_float, C.c_ulonglong]
        R.ref_sampler_destroy.restype = None
        R.ref_sampler_destroy.argtypes = [C.c_void_p]
        R.ref_sampler_set_temperature.restype = None
        R.ref_sampler_set_temperature.argtypes = [C.c_void_p, C.c_float]
        R.ref_sampler_set_topk.restype = None
        R.ref_sampler_set_topk.argtypes = [C.c_void_p, C.c_int32]
        R.ref_sampler_sample.restype = C.c_int32
        R.ref_sampler_sample.argtypes = [C.c_void_p, C.c_void_p, C.c_int32]
        _ref = R
    return _ref


class RefSampler:
    """The reference's own Sampler object (oracle/_ref)."""

    def __init__(self, vocab_size: int, temperature: float, topp: float, rng_seed: int):
        self.h = ref().ref_sampler_create(vocab_size, temperature, topp, rng_seed)

    def __del__(self):
        if getattr(self, "h", None):
            ref().ref_sampler_destroy(self.h)
            self.h = None

    def set_temperature(self, t: float) -> None:
        ref().ref_sampler_set_temperature(self.h, t)

    def set_topk(self, k: int) -> None:
        ref().ref_sampler_set_topk(self.h, k)

    def sample(self, logits: np.ndarray, dtype: int | None = None) -> int:
        assert logits.flags.c_contiguous
        return ref().ref_sampler_sample(self.h, logits.ctypes.data, np_dtype_code(logits, dtype))
