"""Python mirror of the logit-processor interface (extension/llm/sampler/logit_processor.h:19-40)
over the C ABI of include/et_logit_processor.h.

``LogitProcessor.process(logits)`` keeps the reference's contract: in place, rank 2 = every row,
rank 3 = last sequence position, non-Ok (here: ``SamplerError``) on an element type the processor
does not handle.  ``LogitChain`` is the list a runner holds
(extension/llm/runner/text_token_generator.h:44-66): processors run in registration order, as one
kernel launch on the current stream.  The classes named like the reference's test processors
(test_logit_processor.cpp:39-104) are single-processor chains.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _capi
from .sampler import SamplerError, dtype_code


class LogitChain:
    def __init__(self):
        h = C.c_void_p()
        st = _capi.lib().ets_logit_chain_create(C.byref(h))
        if st != _capi.OK:
            raise SamplerError(st, _capi.lib().ets_logit_chain_last_error(None).decode())
        self._h = h
        self._keep = []  # device tensors the chain reads at process time

    def close(self):
        if getattr(self, "_h", None):
            _capi.lib().ets_logit_chain_destroy(self._h)
            self._h = None

    __del__ = close

    def _check(self, st):
        if st != _capi.OK:
            raise SamplerError(st, _capi.lib().ets_logit_chain_last_error(self._h).decode())

    def __len__(self):
        return _capi.lib().ets_logit_chain_size(self._h)

    # ---- registration, in order (TextTokenGenerator::add_logit_processor, text_token_generator.h:44-48)
    def add_bias(self, bias: float) -> "LogitChain":
        self._check(_capi.lib().ets_logit_chain_add_bias(self._h, float(bias)))
        return self

    def add_scale(self, factor: float) -> "LogitChain":
        self._check(_capi.lib().ets_logit_chain_add_scale(self._h, float(factor)))
        return self

    def add_mask(self, tokens) -> "LogitChain":
        ids = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
        self._check(_capi.lib().ets_logit_chain_add_mask(self._h, ids.ctypes.data, ids.size))
        return self

    def add_token_bias(self, tokens, bias) -> "LogitChain":
        ids = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
        val = np.ascontiguousarray(bias, dtype=np.float32).reshape(-1)
        if ids.size != val.size:
            raise SamplerError(_capi.INVALID_ARGUMENT, "one bias per token id is required")
        self._check(_capi.lib().ets_logit_chain_add_token_bias(self._h, ids.ctypes.data, val.ctypes.data, ids.size))
        return self

    def add_repetition_penalty(self, penalty: float, history: torch.Tensor, lengths: torch.Tensor) -> "LogitChain":
        """``history``: device int32 ``[batch, L]``; ``lengths``: device int32 ``[batch]``.  Both are read
        when ``process`` runs, so the caller appends tokens to them in place between steps."""
        if not (history.is_cuda and lengths.is_cuda and history.dtype == torch.int32 and lengths.dtype == torch.int32
                and history.dim() == 2 and history.stride(1) == 1 and lengths.is_contiguous()):
            raise SamplerError(_capi.INVALID_ARGUMENT, "history [batch, L] and lengths [batch] must be int32 device tensors")
        self._keep += [history, lengths]
        self._check(_capi.lib().ets_logit_chain_add_repetition_penalty(self._h, float(penalty), history.data_ptr(),
                                                                       history.stride(0), lengths.data_ptr()))
        return self

    # ---- LogitProcessor::process (logit_processor.h:37-38)
    def process(self, logits: torch.Tensor, dtype: int | None = None) -> None:
        if not logits.is_cuda or not logits.is_contiguous():
            raise SamplerError(_capi.INVALID_ARGUMENT, "process wants a contiguous device tensor")
        code = dtype_code(logits) if dtype is None else dtype
        sizes = (C.c_int64 * max(1, logits.dim()))(*logits.shape)
        stream = torch.cuda.current_stream(logits.device).cuda_stream
        self._check(_capi.lib().ets_logit_chain_process(self._h, logits.data_ptr(), code, logits.dim(), sizes, stream))


class LogitProcessor:
    """Base of the single-processor classes; ``process`` is the reference's one virtual."""

    def __init__(self):
        self._chain = LogitChain()

    def process(self, logits: torch.Tensor) -> None:
        self._chain.process(logits)


class AddBiasProcessor(LogitProcessor):  # test_logit_processor.cpp:39-63
    def __init__(self, bias: float):
        super().__init__()
        self._chain.add_bias(bias)


class MultiplyProcessor(LogitProcessor):  # test_logit_processor.cpp:65-83
    def __init__(self, factor: float):
        super().__init__()
        self._chain.add_scale(factor)


class MaskTokenProcessor(LogitProcessor):  # test_logit_processor.cpp:85-104
    def __init__(self, banned_token):
        super().__init__()
        self._chain.add_mask(np.atleast_1d(np.asarray(banned_token, dtype=np.int64)).astype(np.int32))
