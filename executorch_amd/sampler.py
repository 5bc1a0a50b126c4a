"""Host-side mirror of ExecuTorch's ``extension/llm/sampler`` interface over the HIP library.

``Sampler(vocab_size, temperature, topp, rng_seed)`` / ``sample(logits)`` follow
``extension/llm/sampler/sampler.h:37-83``; ``sample_from_logits`` / ``logits_to_token`` follow
``extension/llm/sampler/util.h:25-71``.  ``sample_batch`` is the batched ``[B, vocab]`` entry over
device-resident logits.  torch is used only for device memory and streams.
"""
from __future__ import annotations

import ctypes as C
import time

import numpy as np
import torch

from . import _capi
from ._capi import DTYPE_BFLOAT16, DTYPE_FLOAT, DTYPE_HALF, DTYPE_UINT16, RowDebug

K_TOPP = 0.9  # sampler.h:29


# layout of ets_sampling_config (include/et_sampler.h): float, float, int32, 4 bytes of padding, uint64
SAMPLING_CONFIG_DTYPE = np.dtype({"names": ["temperature", "top_p", "top_k", "seed"], "formats": ["f4", "f4", "i4", "u8"],
                                  "offsets": [0, 4, 8, 16], "itemsize": 24})


class SamplerError(RuntimeError):
    """A non-Ok status from the C ABI; ``code`` holds the executorch Error value."""

    def __init__(self, code: int, message: str):
        super().__init__(f"ets status 0x{code:02x}: {message}")
        self.code = code


_TORCH_DTYPES = {
    torch.float32: DTYPE_FLOAT,
    torch.float16: DTYPE_HALF,
    torch.bfloat16: DTYPE_BFLOAT16,
    torch.uint16: DTYPE_UINT16,
}
_NUMPY_DTYPES = {np.dtype(np.float32): DTYPE_FLOAT, np.dtype(np.float16): DTYPE_HALF}


def dtype_code(t) -> int:
    """executorch ScalarType code of a torch tensor or numpy array."""
    if isinstance(t, torch.Tensor):
        if t.dtype not in _TORCH_DTYPES:
            raise SamplerError(_capi.INVALID_ARGUMENT, "Unsupported dtype in sample_from_logits")
        return _TORCH_DTYPES[t.dtype]
    if t.dtype not in _NUMPY_DTYPES:
        raise SamplerError(_capi.INVALID_ARGUMENT, "Unsupported dtype in sample_from_logits (pass dtype= for uint16 storage)")
    return _NUMPY_DTYPES[t.dtype]


class Sampler:
    """``Sampler(vocab_size, temperature, topp, rng_seed)``; the 2-argument form uses
    ``topp = 0.9`` and a clock seed like the reference (sampler.cpp:183-187).

    ``max_batch`` sizes the per-row coin streams of :meth:`sample_batch`; row ``b`` starts from
    ``rng_seed + b``.
    """

    def __init__(self, vocab_size: int, temperature: float, topp: float | None = None,
                 rng_seed: int | None = None, max_batch: int = 1):
        self._h = C.c_void_p()
        L = _capi.lib()
        if topp is None and rng_seed is None:
            st = L.ets_sampler_create_default(vocab_size, temperature, max_batch, C.byref(self._h))
        else:
            st = L.ets_sampler_create(vocab_size, temperature, K_TOPP if topp is None else topp,
                                      int(time.time()) if rng_seed is None else rng_seed, max_batch,
                                      C.byref(self._h))
        if st != _capi.OK:
            raise SamplerError(st, L.ets_sampler_last_error(None).decode())
        self.vocab_size = vocab_size
        self.max_batch = max_batch

    def close(self) -> None:
        if getattr(self, "_h", None) and self._h.value:
            _capi.lib().ets_sampler_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, st: int) -> None:
        if st != _capi.OK:
            raise SamplerError(st, _capi.lib().ets_sampler_last_error(self._h).decode())

    # ---- sampler.h:48-60
    def set_temperature(self, temperature: float) -> None:
        self._check(_capi.lib().ets_sampler_set_temperature(self._h, temperature))

    def set_topk(self, topk: int) -> None:
        self._check(_capi.lib().ets_sampler_set_topk(self._h, topk))

    def set_topp(self, topp: float) -> None:
        self._check(_capi.lib().ets_sampler_set_topp(self._h, topp))

    def set_row_split(self, mode: int) -> None:
        """0 = automatic, 1 = several workgroups per row wherever that path applies, 2 = never."""
        self._check(_capi.lib().ets_sampler_set_row_split(self._h, mode))

    # ---- sampler.cpp:222-251
    def sample(self, logits, dtype: int | None = None) -> int:
        """One row of ``vocab_size`` logits in host memory (numpy array or CPU tensor)."""
        if isinstance(logits, torch.Tensor):
            if logits.is_cuda:
                return int(self.sample_batch(logits.reshape(1, -1))[0].item())
            code = dtype_code(logits) if dtype is None else dtype
            logits = logits.contiguous()
            ptr, n = logits.data_ptr(), logits.numel()
        else:
            logits = np.ascontiguousarray(logits)
            code = dtype_code(logits) if dtype is None else dtype
            ptr, n = logits.ctypes.data, logits.size
        if n < self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "logits shorter than vocab_size")
        tok = C.c_int32(-1)
        self._check(_capi.lib().ets_sampler_sample(self._h, ptr, code, C.byref(tok)))
        return tok.value

    def sample_batch(self, logits: torch.Tensor, out: torch.Tensor | None = None, dtype: int | None = None,
                     probs_out: torch.Tensor | None = None, debug_out: torch.Tensor | None = None) -> torch.Tensor:
        """Rows of a device tensor ``[B, vocab]`` (row stride >= vocab); returns int32 ``[B]``
        on the same device, asynchronously on the current stream."""
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise SamplerError(_capi.INVALID_ARGUMENT, "sample_batch wants a device tensor [B, vocab] with unit inner stride")
        B, V = logits.shape
        if V != self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "last dimension differs from vocab_size")
        code = dtype_code(logits) if dtype is None else dtype
        if out is None:
            out = torch.empty(B, dtype=torch.int32, device=logits.device)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        L = _capi.lib()
        if probs_out is None and debug_out is None:
            st = L.ets_sampler_sample_batch(self._h, logits.data_ptr(), code, B, logits.stride(0), out.data_ptr(), stream)
        else:
            st = L.ets_sampler_sample_batch_debug(
                self._h, logits.data_ptr(), code, B, logits.stride(0), out.data_ptr(),
                probs_out.data_ptr() if probs_out is not None else None,
                debug_out.data_ptr() if debug_out is not None else None, stream)
        self._check(st)
        return out

    def sample_batch_static(self, logits: torch.Tensor, out: torch.Tensor | None = None, dtype: int | None = None) -> torch.Tensor:
        """``sample_batch`` through the entry point that allocates nothing: the kernels' work buffers
        come from a fixed array inside the library (so the problem size is limited); ``out`` should
        be passed by callers that must not allocate either."""
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise SamplerError(_capi.INVALID_ARGUMENT, "sample_batch_static wants a device tensor [B, vocab] with unit inner stride")
        B, V = logits.shape
        if V != self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "last dimension differs from vocab_size")
        code = dtype_code(logits) if dtype is None else dtype
        if out is None:
            out = torch.empty(B, dtype=torch.int32, device=logits.device)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        self._check(_capi.lib().ets_sampler_sample_batch_static(self._h, logits.data_ptr(), code, B, logits.stride(0),
                                                                out.data_ptr(), stream))
        return out

    def sample_batch_configs(self, logits: torch.Tensor, configs, out: torch.Tensor | None = None,
                             dtype: int | None = None, debug_out: torch.Tensor | None = None) -> torch.Tensor:
        """``sample_batch`` with one ``SamplingConfig`` per row (llm_session.h:29-34): ``configs`` is a
        sequence of ``(temperature, top_p, top_k, seed)`` tuples or a structured array of dtype
        ``SAMPLING_CONFIG_DTYPE``; temperature < 0 means this sampler's own, seed 0 continues the
        row's coin stream."""
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise SamplerError(_capi.INVALID_ARGUMENT, "sample_batch_configs wants a device tensor [B, vocab] with unit inner stride")
        B, V = logits.shape
        if V != self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "last dimension differs from vocab_size")
        cfg = np.ascontiguousarray(np.asarray(configs, dtype=SAMPLING_CONFIG_DTYPE) if not isinstance(configs, np.ndarray)
                                   else configs.astype(SAMPLING_CONFIG_DTYPE, copy=False))
        if cfg.shape != (B,):
            raise SamplerError(_capi.INVALID_ARGUMENT, "one config per row is required")
        code = dtype_code(logits) if dtype is None else dtype
        if out is None:
            out = torch.empty(B, dtype=torch.int32, device=logits.device)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        st = _capi.lib().ets_sampler_sample_batch_configs(
            self._h, logits.data_ptr(), code, B, logits.stride(0), cfg.ctypes.data, out.data_ptr(),
            debug_out.data_ptr() if debug_out is not None else None, stream)
        self._check(st)
        return out

    def sample_batch_chain(self, logits: torch.Tensor, chain, out: torch.Tensor | None = None,
                           dtype: int | None = None) -> torch.Tensor:
        """``chain.process(logits)`` followed by ``sample_batch(logits)`` in one call
        (text_token_generator.h:141-148).  Same tokens; the chain's trailing biases and factors may
        be applied while the sampler reads the rows instead of being stored into ``logits``."""
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise SamplerError(_capi.INVALID_ARGUMENT, "sample_batch_chain wants a device tensor [B, vocab] with unit inner stride")
        B, V = logits.shape
        if V != self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "last dimension differs from vocab_size")
        code = dtype_code(logits) if dtype is None else dtype
        if out is None:
            out = torch.empty(B, dtype=torch.int32, device=logits.device)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        self._check(_capi.lib().ets_sampler_sample_batch_chain(
            self._h, chain._h, logits.data_ptr(), code, B, logits.stride(0), out.data_ptr(), stream))
        return out

    def gumbel_max_batch(self, logits: torch.Tensor, temperature, noise: torch.Tensor | None = None,
                         out: torch.Tensor | None = None, dtype: int | None = None) -> torch.Tensor:
        """The in-graph Gumbel-max sampler (examples/models/qwen3_5_moe/sampler.py:17-60):
        ``argmax(logits / T.clamp(min=1e-6) + gumbel)``.  ``temperature`` is a float or one per row;
        ``noise`` is a device fp32 ``[B, vocab]`` tensor of uniforms (``torch.rand_like(logits)`` in the
        reference) or None for the library's own generator."""
        if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1:
            raise SamplerError(_capi.INVALID_ARGUMENT, "gumbel_max_batch wants a device tensor [B, vocab] with unit inner stride")
        B, V = logits.shape
        if V != self.vocab_size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "last dimension differs from vocab_size")
        t = np.ascontiguousarray(np.atleast_1d(np.asarray(temperature, dtype=np.float32)))
        if noise is not None and not (noise.is_cuda and noise.dtype == torch.float32 and noise.shape == (B, V)
                                      and noise.is_contiguous()):
            raise SamplerError(_capi.INVALID_ARGUMENT, "noise must be a contiguous device fp32 tensor [B, vocab]")
        code = dtype_code(logits) if dtype is None else dtype
        if out is None:
            out = torch.empty(B, dtype=torch.int32, device=logits.device)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        self._check(_capi.lib().ets_sampler_gumbel_max_batch(
            self._h, logits.data_ptr(), code, B, logits.stride(0), t.ctypes.data, t.size,
            noise.data_ptr() if noise is not None else None, out.data_ptr(), stream))
        return out

    # ---- sampling time in microseconds (stats.h:46-47, :62-69 keep it in whole milliseconds)
    def set_timing(self, enabled: bool = True) -> None:
        self._check(_capi.lib().ets_sampler_set_timing(self._h, 1 if enabled else 0))

    def stats(self) -> dict:
        st = _capi.SamplerStats()
        self._check(_capi.lib().ets_sampler_get_stats(self._h, C.byref(st)))
        return {"calls": st.calls, "rows": st.rows, "aggregate_sampling_time_us": st.aggregate_sampling_time_us,
                "last_call_us": st.last_call_us}

    def reset_stats(self) -> None:
        self._check(_capi.lib().ets_sampler_reset_stats(self._h))

    # ---- per-row xorshift64* states (sampler.h:82)
    def set_rng_states(self, states, first_row: int = 0) -> None:
        a = np.ascontiguousarray(states, dtype=np.uint64)
        self._check(_capi.lib().ets_sampler_set_rng_states(self._h, first_row, a.size, a.ctypes.data))

    def get_rng_states(self, count: int | None = None, first_row: int = 0) -> np.ndarray:
        n = self.max_batch - first_row if count is None else count
        a = np.empty(n, dtype=np.uint64)
        self._check(_capi.lib().ets_sampler_get_rng_states(self._h, first_row, n, a.ctypes.data))
        return a


def debug_records(debug_out: torch.Tensor) -> np.ndarray:
    """View a ``[B, 8]`` int32 debug tensor (filled by ``sample_batch(debug_out=...)``) as records."""
    raw = debug_out.cpu().numpy()
    dt = np.dtype([("max_val", "f4"), ("sum", "f4"), ("coin", "f4"), ("cumulative", "f4"), ("r", "f4"),
                   ("n_candidates", "i4"), ("last_idx", "i4"), ("position", "i4")])
    return raw.view(dt).reshape(-1)


def _host_tensor_args(logits, dtype):
    if isinstance(logits, torch.Tensor):
        t = logits.contiguous().cpu()
        return t, t.data_ptr(), dtype_code(t) if dtype is None else dtype, list(t.shape)
    a = np.ascontiguousarray(logits)
    return a, a.ctypes.data, dtype_code(a) if dtype is None else dtype, list(a.shape)


def sample_from_logits(logits, sampler: Sampler, dtype: int | None = None) -> int:
    """util.h:25-55: rank 3 ``[1, S, V]`` samples the last position of batch 0."""
    keep, ptr, code, shape = _host_tensor_args(logits, dtype)
    sizes = (C.c_int64 * len(shape))(*shape)
    tok = C.c_int32(-1)
    sampler._check(_capi.lib().ets_sample_from_logits(sampler._h, ptr, code, len(shape), sizes, C.byref(tok)))
    return tok.value


def sample_from_logits_batch(logits: torch.Tensor, sampler: Sampler, out: torch.Tensor | None = None,
                             dtype: int | None = None) -> torch.Tensor:
    """The batched adapter over a DEVICE tensor ``[B, V]`` or ``[B, S, V]`` (last position of every
    batch entry); returns int32 ``[B]`` on the device.  The reference's adapter (util.h:25-55) reads
    a host tensor and batch 0 only."""
    if not logits.is_cuda or not logits.is_contiguous() or logits.dim() not in (2, 3):
        raise SamplerError(_capi.INVALID_ARGUMENT, "sample_from_logits_batch wants a contiguous device tensor of rank 2 or 3")
    code = dtype_code(logits) if dtype is None else dtype
    if out is None:
        out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
    sizes = (C.c_int64 * logits.dim())(*logits.shape)
    stream = torch.cuda.current_stream(logits.device).cuda_stream
    sampler._check(_capi.lib().ets_sample_from_logits_batch(sampler._h, logits.data_ptr(), code, logits.dim(), sizes,
                                                            out.data_ptr(), stream))
    return out


def logits_to_token(logits, temperature: float = 0.0, dtype: int | None = None) -> int:
    """util.h:64-71: a temporary 2-argument Sampler over the tensor's last dimension."""
    keep, ptr, code, shape = _host_tensor_args(logits, dtype)
    sizes = (C.c_int64 * len(shape))(*shape)
    tok = C.c_int32(-1)
    L = _capi.lib()
    st = L.ets_logits_to_token(ptr, code, len(shape), sizes, temperature, C.byref(tok))
    if st != _capi.OK:
        raise SamplerError(st, L.ets_sampler_last_error(None).decode())
    return tok.value
