"""ctypes bindings of include/et_sampler.h (the C ABI of libet_sampler.so).

The library is loaded from this package's directory; there is no fallback: if it has not been
built (``python -m executorch_amd.build``) loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libet_sampler.so")
HOOKS_PATH = os.path.join(HERE, "libet_sampler_hooks.so")  # csrc/ets_test_hooks.h: tests and the benchmark only

OK, INTERNAL, INVALID_STATE, NOT_SUPPORTED, INVALID_ARGUMENT, MEMORY_ALLOCATION_FAILED = 0x00, 0x01, 0x02, 0x10, 0x12, 0x21
DTYPE_HALF, DTYPE_FLOAT, DTYPE_BFLOAT16, DTYPE_UINT16 = 5, 6, 15, 27


class SamplerStats(C.Structure):
    _fields_ = [("calls", C.c_uint64), ("rows", C.c_uint64), ("aggregate_sampling_time_us", C.c_double),
                ("last_call_us", C.c_double)]


class RowDebug(C.Structure):
    _fields_ = [
        ("max_val", C.c_float),
        ("sum", C.c_float),
        ("coin", C.c_float),
        ("cumulative", C.c_float),
        ("r", C.c_float),
        ("n_candidates", C.c_int32),
        ("last_idx", C.c_int32),
        ("position", C.c_int32),
    ]


# name -> (restype, argtypes); every symbol declared in include/et_sampler.h
SIGNATURES = {
    "ets_sampler_create": (C.c_int32, [C.c_int32, C.c_float, C.c_float, C.c_uint64, C.c_int32, C.POINTER(C.c_void_p)]),
    "ets_sampler_create_default": (C.c_int32, [C.c_int32, C.c_float, C.c_int32, C.POINTER(C.c_void_p)]),
    "ets_sampler_destroy": (C.c_int32, [C.c_void_p]),
    "ets_sampler_set_temperature": (C.c_int32, [C.c_void_p, C.c_float]),
    "ets_sampler_set_topk": (C.c_int32, [C.c_void_p, C.c_int32]),
    "ets_sampler_set_topp": (C.c_int32, [C.c_void_p, C.c_float]),
    "ets_sampler_set_row_split": (C.c_int32, [C.c_void_p, C.c_int32]),
    "ets_sampler_sample": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.POINTER(C.c_int32)]),
    "ets_sampler_sample_batch": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p]),
    "ets_sampler_sample_batch_static": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p]),
    "ets_sampler_sample_batch_configs": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p,
                                         C.c_void_p, C.c_void_p, C.c_void_p]),
    "ets_sampler_sample_batch_debug": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p,
                                                   C.c_void_p, C.c_void_p, C.c_void_p]),
    "ets_sampler_gumbel_max_batch": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p, C.c_int32,
                                     C.c_void_p, C.c_void_p, C.c_void_p]),
    "ets_sampler_set_timing": (C.c_int32, [C.c_void_p, C.c_int32]),
    "ets_sampler_get_stats": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "ets_sampler_reset_stats": (C.c_int32, [C.c_void_p]),
    "ets_sampler_set_rng_states": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "ets_sampler_get_rng_states": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "ets_sample_from_logits": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "ets_sample_from_logits_batch": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.c_void_p, C.c_void_p]),
    "ets_logits_to_token": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.c_float, C.POINTER(C.c_int32)]),
    "ets_random_u32": (C.c_uint32, [C.POINTER(C.c_uint64)]),
    "ets_random_f32": (C.c_float, [C.POINTER(C.c_uint64)]),
    "ets_sampler_last_error": (C.c_char_p, [C.c_void_p]),
    "ets_version": (C.c_char_p, []),
}

# every symbol declared in include/et_logit_processor.h
CHAIN_SIGNATURES = {
    "ets_logit_chain_create": (C.c_int32, [C.POINTER(C.c_void_p)]),
    "ets_logit_chain_destroy": (C.c_int32, [C.c_void_p]),
    "ets_logit_chain_size": (C.c_int32, [C.c_void_p]),
    "ets_logit_chain_add_bias": (C.c_int32, [C.c_void_p, C.c_float]),
    "ets_logit_chain_add_scale": (C.c_int32, [C.c_void_p, C.c_float]),
    "ets_logit_chain_add_mask": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32]),
    "ets_logit_chain_add_token_bias": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]),
    "ets_logit_chain_add_repetition_penalty": (C.c_int32, [C.c_void_p, C.c_float, C.c_void_p, C.c_int64, C.c_void_p]),
    "ets_logit_chain_process": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.c_void_p]),
    "ets_sampler_sample_batch_chain": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_void_p,
                                       C.c_void_p]),
    "ets_logit_chain_last_error": (C.c_char_p, [C.c_void_p]),
}

# csrc/ets_test_hooks.h (libet_sampler_hooks.so)
TEST_HOOKS = {
    "ets_test_signal_floor": (C.c_int32, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
    "ets_test_last_error": (C.c_char_p, []),
    "ets_test_handle_buffers": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "ets_test_fused_launch_number": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p]),
    "ets_test_set_fused_launch_number": (C.c_int32, [C.c_void_p, C.c_uint32]),
    "ets_test_expf": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "ets_test_seq_sum": (C.c_int32, [C.c_void_p, C.c_int32, C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]),
    "ets_test_split_timers": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int32]),
    "ets_test_empty_launch": (C.c_int32, [C.c_void_p]),
    "ets_test_copy_probe": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "ets_test_read_floor": (C.c_int32, [C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]),
}

_lib = None
_hooks = None


def _load(path: str, tables) -> C.CDLL:
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: build it with `python -m executorch_amd.build` "
            "(there is no CPU fallback for the sampler)")
    L = C.CDLL(path)
    for table in tables:
        for name, (res, args) in table.items():
            f = getattr(L, name)
            f.restype = res
            f.argtypes = args
    return L


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load(LIB_PATH, (SIGNATURES, CHAIN_SIGNATURES))
    return _lib


def hooks() -> C.CDLL:
    """The test and measurement hooks: a library of their own, not part of the product."""
    global _hooks
    if _hooks is None:
        _hooks = _load(HOOKS_PATH, (TEST_HOOKS,))
    return _hooks
