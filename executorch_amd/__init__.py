"""MI355X-native LLM token sampler: a drop-in for ExecuTorch's ``extension/llm/sampler``."""
from .sampler import (K_TOPP, SAMPLING_CONFIG_DTYPE, Sampler, SamplerError, debug_records, logits_to_token,  # noqa: F401
                      sample_from_logits, sample_from_logits_batch)
