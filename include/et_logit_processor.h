/*
 * et_logit_processor.h -- C ABI of the device-side logit processor chain (MI355X, gfx950).
 *
 * Replaces, for logits that live in device memory, the host loop that ExecuTorch's
 * TextTokenGenerator runs between the forward pass and the sampler
 * (extension/llm/runner/text_token_generator.h:143 applies the registered
 * extension/llm/sampler/logit_processor.h:19-40 processors in registration order).
 * The contract of LogitProcessor::process(Tensor) is kept:
 *   - the transform is IN PLACE on the logits tensor, each processor sees the edits of the
 *     processors registered before it;
 *   - rank 2 [batch, vocab]      -> every row, full last dimension;
 *   - rank 3 [batch, seq, vocab] -> the LAST sequence position of every batch entry, earlier
 *     positions are not touched (test_logit_processor.cpp:186-212);
 *   - other ranks and element types a processor does not handle -> ETS_INVALID_ARGUMENT
 *     (the reference leaves other ranks undefined and has its test processors return
 *     InvalidArgument for other dtypes, test_logit_processor.cpp:217-223).
 * Element types: Float, Half, BFloat16.  16-bit rows are converted to fp32, transformed, and
 * rounded back (to nearest even) by every processor, as separate processors storing into the
 * tensor would.
 *
 * The chain is one kernel launch whatever its length: the row is cut into tiles, a workgroup owns
 * a tile and runs every processor over it in order.
 *
 * Status codes and dtype codes are those of et_sampler.h.
 */
#ifndef ET_LOGIT_PROCESSOR_H_
#define ET_LOGIT_PROCESSOR_H_

#include "et_sampler.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ets_logit_chain ets_logit_chain;

/* The std::vector<std::shared_ptr<LogitProcessor>> a runner holds
 * (test_logit_processor.cpp:125-143); lives on the current HIP device. */
ETS_API ets_status ets_logit_chain_create(ets_logit_chain** out);
ETS_API ets_status ets_logit_chain_destroy(ets_logit_chain* c);

/* Number of processors registered so far. */
ETS_API int32_t ets_logit_chain_size(const ets_logit_chain* c);

/* data[i] += bias for the whole row  -- AddBiasProcessor, test_logit_processor.cpp:39-63. */
ETS_API ets_status ets_logit_chain_add_bias(ets_logit_chain* c, float bias);

/* data[i] *= factor for the whole row  -- MultiplyProcessor, test_logit_processor.cpp:65-83. */
ETS_API ets_status ets_logit_chain_add_scale(ets_logit_chain* c, float factor);

/* data[token] = -inf for each listed token  -- MaskTokenProcessor,
 * test_logit_processor.cpp:85-104 (one banned token there; a list here, the pattern grammar
 * masks follow).  `tokens` is a HOST array, copied; ids outside [0, vocab) are ignored
 * (test_logit_processor.cpp:165-184). */
ETS_API ets_status ets_logit_chain_add_mask(ets_logit_chain* c, const int32_t* tokens, int32_t count);

/* data[tokens[j]] += bias[j], j in order ("logit bias", named as an example at
 * logit_processor.h:21; no implementation in the reference).  HOST arrays, copied; ids outside
 * [0, vocab) are ignored; an id listed twice receives both additions in list order. */
ETS_API ets_status ets_logit_chain_add_token_bias(ets_logit_chain* c, const int32_t* tokens, const float* bias,
                                                 int32_t count);

/* Repetition penalty (named at logit_processor.h:21; no implementation in the reference, the
 * rule is the common one): every DISTINCT token id in row b's history has its logit x replaced
 * by x < 0 ? x * penalty : x / penalty, once.  The history is read on the device at process
 * time: `d_history` is a DEVICE pointer to int32 [batch, history_stride], `d_history_len` a
 * DEVICE pointer to `batch` int32 lengths (<= history_stride); the caller may update both
 * between calls.  Ids outside [0, vocab) are ignored.  Needs vocab <= 1 048 576. */
ETS_API ets_status ets_logit_chain_add_repetition_penalty(ets_logit_chain* c, float penalty, const int32_t* d_history,
                                                         int64_t history_stride, const int32_t* d_history_len);

/* LogitProcessor::process(Tensor) for the whole chain  -- logit_processor.h:37-38, applied as
 * text_token_generator.h:143 applies it.  `d_logits` is a DEVICE pointer to the tensor's first
 * element (contiguous), `sizes` a HOST array of `rank` extents.  Asynchronous on `hip_stream`;
 * a sampler call issued on the same stream afterwards sees the processed logits. */
ETS_API ets_status ets_logit_chain_process(ets_logit_chain* c, void* d_logits, int32_t dtype, int32_t rank,
                                          const int64_t* sizes, void* hip_stream);

/* The two steps of text_token_generator.h:141-148 in one call: the chain over rows
 * [batch, vocab] (`row_stride_elems` elements apart), then ets_sampler_sample_batch() on them --
 * the same tokens, coin streams and errors as ets_logit_chain_process() followed by
 * ets_sampler_sample_batch() on the same stream.  What differs is what is left in the tensor:
 * when the rows take the sampler's several-workgroups-per-row path (stochastic top-p rows of at
 * least 8192 entries, 16-byte aligned), the chain's LAST processors, as far as they are biases
 * and factors (up to four), are not stored into the tensor but applied while the sampler reads
 * it -- rounded to the element type after each, as the stores would -- which saves a pass over
 * the tensor that reads and writes every entry.  The processors in front of those still run in
 * place.  A caller that reads the logits after sampling uses the two calls instead.
 * `d_logits` and `d_tokens` are DEVICE pointers; asynchronous on `hip_stream`. */
ETS_API ets_status ets_sampler_sample_batch_chain(ets_sampler* s, ets_logit_chain* c, void* d_logits, int32_t dtype,
                                                 int32_t batch, int64_t row_stride_elems, int32_t* d_tokens,
                                                 void* hip_stream);

/* Text of the last error on this chain ("" if none). */
ETS_API const char* ets_logit_chain_last_error(const ets_logit_chain* c);

#ifdef __cplusplus
}
#endif

#endif /* ET_LOGIT_PROCESSOR_H_ */
