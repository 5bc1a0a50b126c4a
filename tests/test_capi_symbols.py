"""The C-ABI library loads and exports every function include/et_sampler.h declares; the
bindings table in executorch_amd/_capi.py covers the same set.  No compute call is made."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "et_sampler.h")
CHAIN_HEADER = os.path.join(ROOT, "include", "et_logit_processor.h")
HOOKS = os.path.join(ROOT, "executorch_amd", "csrc", "ets_test_hooks.h")


def declared(path):
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"ETS_API\s+[\w\s\*]+?\b(ets_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared(HEADER)
    for must in ("ets_sampler_create", "ets_sampler_create_default", "ets_sampler_destroy", "ets_sampler_set_temperature",
                 "ets_sampler_set_topk", "ets_sampler_sample", "ets_sampler_sample_batch", "ets_sample_from_logits",
                 "ets_logits_to_token", "ets_random_u32", "ets_random_f32", "ets_sampler_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from executorch_amd import _capi

    assert os.path.exists(_capi.LIB_PATH), "build the library first: python -m executorch_amd.build"
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for name in declared(HEADER) + declared(CHAIN_HEADER):
        assert hasattr(lib, name), name
    # the test and measurement hooks live in a library of their own, and only there
    assert os.path.exists(_capi.HOOKS_PATH)
    hooks = ctypes.CDLL(_capi.HOOKS_PATH)
    for name in declared(HOOKS):
        assert hasattr(hooks, name), name
        assert not hasattr(lib, name), name
    assert sorted(_capi.SIGNATURES) == declared(HEADER)
    assert sorted(_capi.CHAIN_SIGNATURES) == declared(CHAIN_HEADER)
    assert sorted(_capi.TEST_HOOKS) == declared(HOOKS)


def test_host_side_rng_needs_no_gpu():
    from executorch_amd import _capi

    st = ctypes.c_uint64(42)
    assert _capi.lib().ets_random_u32(ctypes.byref(st)) == 0x56CE4AB7
    assert st.value == 0x54000020
    st = ctypes.c_uint64(42)
    assert _capi.lib().ets_random_f32(ctypes.byref(st)) == pytest.approx(0.3390852212905884, abs=0)
    assert b"gfx950" in _capi.lib().ets_version()


def test_argument_errors_without_a_device():
    from executorch_amd import _capi

    L = _capi.lib()
    h = ctypes.c_void_p()
    assert L.ets_sampler_create(0, 1.0, 0.9, 1, 1, ctypes.byref(h)) == _capi.INVALID_ARGUMENT
    assert b"vocab_size" in L.ets_sampler_last_error(None)
    assert L.ets_sampler_create(10, 1.0, 0.9, 1, 0, ctypes.byref(h)) == _capi.INVALID_ARGUMENT
    assert L.ets_sampler_create(10, 1.0, 0.9, 1, 1, None) == _capi.INVALID_ARGUMENT
    assert L.ets_sampler_set_topk(None, 3) == _capi.INVALID_ARGUMENT
    assert L.ets_sampler_destroy(None) == _capi.OK


def test_no_silent_cpu_fallback():
    """Without a GPU the sampler must fail loudly, never answer from the host."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    import executorch_amd as ea

    with pytest.raises(ea.SamplerError):
        ea.Sampler(100, 1.0, 0.9, 1)
