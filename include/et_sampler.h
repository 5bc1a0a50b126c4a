/*
 * et_sampler.h -- C ABI of the MI355X (gfx950) LLM token sampler.
 *
 * A drop-in for ExecuTorch's `extension/llm/sampler` path: every entry point below names the
 * reference interface it replaces (paths relative to the ExecuTorch tree).  Plain pointers
 * and sizes only; no C++ or torch types cross this boundary.  The C++ class
 * `executorch::extension::llm::Sampler` in include/executorch_amd/sampler.h and the Python
 * class `executorch_amd.Sampler` are thin wrappers over these functions.
 *
 * Semantics shared by all sampling entry points (Sampler::sample<T>, sampler.cpp:222-251):
 *   temperature == 0          -> arg-max, lowest index wins ties, no coin is drawn;
 *   otherwise                 -> logits * (1/temperature), softmax, ONE xorshift64* coin, then
 *     0 < topk < vocab        -> top-k draw            (sampler.cpp:72-120)
 *     topp <= 0 || topp >= 1  -> multinomial draw      (sampler.cpp:58-70)
 *     else                    -> top-p (nucleus) draw  (sampler.cpp:122-171)
 * Arithmetic: rows of every dtype are converted to fp32 (exactly) and the fp32 instantiation
 * of the reference is followed bit for bit, including the order of its sequential float
 * additions; fp16/bf16 rows therefore give what the reference gives after the "convert the
 * row to float, then sample<float>" step several of its own runners perform
 * (examples/models/gemma4/runner/gemma4_runner.cpp:166-182).  Among candidates whose
 * probabilities are exactly equal the lower token index is ordered first (the reference
 * leaves that order to std::sort).  The logits buffer is never written: the reference's
 * side effect of leaving probabilities in it (sampler.cpp:231-235) is not reproduced.
 *
 * Every function returns an ets_status; none aborts.  Calls on one handle must be serialized
 * by the caller (as for the reference, text_decoder_runner.h:81-82); distinct handles are
 * independent.  A handle's work buffers are reused from call to call: issue its calls on ONE
 * stream, or order a call on another stream behind the previous one yourself (the per-row
 * parameter and temperature tables are the exception: the library orders their reuse).
 */
#ifndef ET_SAMPLER_H_
#define ET_SAMPLER_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define ETS_API
#else
#define ETS_API __attribute__((visibility("default")))
#endif

/* Status codes: numeric values of executorch::runtime::Error (runtime/core/error.h:35-61). */
typedef int32_t ets_status;
#define ETS_OK 0x00
#define ETS_INTERNAL 0x01          /* a HIP call failed; see ets_sampler_last_error()       */
#define ETS_INVALID_STATE 0x02
#define ETS_NOT_SUPPORTED 0x10     /* e.g. stochastic sampling of UInt16 rows               */
#define ETS_INVALID_ARGUMENT 0x12  /* null pointer, bad size, unknown dtype, batch too big  */
#define ETS_MEMORY_ALLOCATION_FAILED 0x21

/* Element types: numeric values of executorch ScalarType
 * (runtime/core/portable_type/scalar_type.h:98-125); the four that
 * sample_from_logits() accepts (util.h:36-43). */
#define ETS_DTYPE_HALF 5
#define ETS_DTYPE_FLOAT 6
#define ETS_DTYPE_BFLOAT16 15
#define ETS_DTYPE_UINT16 27

typedef struct ets_sampler ets_sampler;

/* Intermediate values of one row's draw, written by the *_debug entry point (tests only). */
typedef struct {
  float max_val;        /* row maximum of logits * inv_temperature                          */
  float sum;            /* softmax normaliser, accumulated like the reference (index order) */
  float coin;           /* the row's xorshift64* coin                                        */
  float cumulative;     /* mass of the nucleus / of the top-k set                            */
  float r;              /* coin scaled into that mass                                        */
  int32_t n_candidates; /* entries >= the top-p cutoff (vocab for top-k)                     */
  int32_t last_idx;     /* last sorted position inside the nucleus                           */
  int32_t position;     /* sorted position of the returned token                             */
} ets_row_debug;

/* Sampler::Sampler(int32_t vocab_size, float temperature, float topp, unsigned long long
 * rng_seed)  -- sampler.cpp:173-181.  No clamping of temperature (a negative value gives a
 * negative inverse, as there).  `max_batch` (>= 1) is the largest batch later passed to
 * ets_sampler_sample_batch(); row b starts with xorshift64* state rng_seed + b, so row 0 is
 * the reference object's own stream.  The handle lives on the current HIP device.
 * vocab_size must be below 2^24 and max_batch at most 65535 (ETS_NOT_SUPPORTED otherwise). */
ETS_API ets_status ets_sampler_create(int32_t vocab_size, float temperature, float topp, uint64_t rng_seed,
                                      int32_t max_batch, ets_sampler** out);

/* Sampler::Sampler(int32_t vocab_size, float temperature)  -- sampler.cpp:183-187:
 * topp = kTopp = 0.9f (sampler.h:29), seed = time(NULL). */
ETS_API ets_status ets_sampler_create_default(int32_t vocab_size, float temperature, int32_t max_batch,
                                              ets_sampler** out);

/* Sampler's implicit destructor. */
ETS_API ets_status ets_sampler_destroy(ets_sampler* s);

/* Sampler::set_temperature  -- sampler.h:48-53 (negative values are reset to 0). */
ETS_API ets_status ets_sampler_set_temperature(ets_sampler* s, float temperature);

/* Sampler::set_topk  -- sampler.h:58-60 (k <= 0 or k >= vocab disables top-k). */
ETS_API ets_status ets_sampler_set_topk(ets_sampler* s, int32_t topk);

/* No counterpart: the reference fixes top-p at construction (sampler.h:78).  Provided so one
 * handle can serve requests with different nucleus sizes. */
ETS_API ets_status ets_sampler_set_topp(ets_sampler* s, float topp);

/* No counterpart (the reference is one scalar loop).  How the stochastic path uses the GPU:
 *   ETS_ROW_SPLIT_AUTO  rows of 8192 entries and more, 16-byte aligned, take the launches in which
 *                       several workgroups share a row; everything else takes one launch with one
 *                       workgroup per row;
 *   ETS_ROW_SPLIT_ON    several workgroups per row wherever that path applies, whatever the
 *                       vocabulary size;
 *   ETS_ROW_SPLIT_OFF   always one workgroup per row.
 * Several workgroups per row, by draw: top-p rows three launches (two when every workgroup of
 * the launch is resident at once, about batch x workgroups-per-row <= compute units, every
 * temperature of the launch is finite, no probabilities are asked for and no other launch of
 * the call runs beside it: the first two are then one kernel, whose workgroups hand each
 * other their results with bounded waits);
 * top-k rows with k <= ceil(vocab / 512) the same three (or two) launches, larger k one workgroup per row;
 * multinomial rows (top_p <= 0 or >= 1) FIVE launches (four under the same conditions: the
 * first two are one kernel then, too), or one workgroup per row when the
 * probabilities are asked for.  All launches of a call go to the call's stream, in order.
 * Work buffers of that path are allocated at the first call that needs them and kept: per row of
 * max_batch about 16 bytes x ceil(vocab / 512) slots x 2 + 40 prepared slots of 2.6 KB, plus per
 * (row, workgroup) of the largest launch a 2048-bucket histogram, a candidate list of up to
 * 16384 x 8 bytes and, for 16-bit rows, a pattern histogram of up to 96 KB -- about 240 MB at
 * max_batch 1024 and vocab 151936.
 * The tokens, coin states and debug records are the same on every setting. */
#define ETS_ROW_SPLIT_AUTO 0
#define ETS_ROW_SPLIT_ON 1
#define ETS_ROW_SPLIT_OFF 2
ETS_API ets_status ets_sampler_set_row_split(ets_sampler* s, int32_t mode);

/* Sampler::sample<T>(T* logits)  -- sampler.cpp:222-251, instantiations :253-258.
 * `logits` is a HOST pointer to vocab_size elements of `dtype`; the row is copied to the
 * device, sampled there and the token copied back (synchronous).  Consumes row 0's coin. */
ETS_API ets_status ets_sampler_sample(ets_sampler* s, const void* logits, int32_t dtype, int32_t* token_out);

/* Batched form of Sampler::sample<T> (no counterpart; the reference is batch-1, util.h:48-51).
 * `d_logits` is a DEVICE pointer to `batch` rows of vocab_size elements, row b starting at
 * element b * row_stride_elems (>= vocab_size); `d_tokens` is a DEVICE pointer to `batch`
 * int32.  Row b uses and advances its own coin stream, so the result equals `batch`
 * reference objects seeded rng_seed + b and does not depend on how rows are batched.
 * Asynchronous on `hip_stream` (a hipStream_t, NULL = the default stream). */
ETS_API ets_status ets_sampler_sample_batch(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                           int64_t row_stride_elems, int32_t* d_tokens, void* hip_stream);

/* No counterpart in the reference.  ets_sampler_sample_batch() for callers that cannot allocate
 * device memory at the time of the call -- code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc: same arguments, same tokens and coin states, but every work
 * buffer of the kernels (partial results, slot records, candidate lists and histograms, sort
 * keys) lies in a 32 MiB array that is part of the library's device image (one copy per GPU, held
 * until the process ends), and the call allocates and frees nothing.  The price is a limit: the
 * buffers of `batch` rows of vocab_size entries must fit (about 17 * batch * vocab_size bytes plus
 * 0.6 MiB per row; batch 8 at vocab 128256 does), else ETS_INVALID_ARGUMENT with the sizes in
 * ets_sampler_last_error().  Every call on a GPU, from any handle, uses that GPU's one array:
 * calls that overlap in time on one GPU race; serialize them (one stream, or events). */
ETS_API ets_status ets_sampler_sample_batch_static(ets_sampler* s, const void* d_logits, int32_t dtype,
                                                  int32_t batch, int64_t row_stride_elems, int32_t* d_tokens,
                                                  void* hip_stream);

/* As above, plus per-row intermediates for the parity tests: `d_probs` (nullable) receives the
 * fp32 softmax probabilities [batch, vocab_size] that the reference would leave in its buffer,
 * `d_debug` (nullable) one ets_row_debug per row.  Both are DEVICE pointers. */
ETS_API ets_status ets_sampler_sample_batch_debug(ets_sampler* s, const void* d_logits, int32_t dtype,
                                                 int32_t batch, int64_t row_stride_elems, int32_t* d_tokens,
                                                 float* d_probs, ets_row_debug* d_debug, void* hip_stream);

/* SamplingConfig  -- extension/llm/runner/llm_session.h:29-34 (same fields, same defaults:
 * temperature -1 = "implementation default", here the handle's temperature; top_p 1.0;
 * top_k 0 = disabled; seed 0 = unset). */
typedef struct ets_sampling_config {
  float temperature;
  float top_p;
  int32_t top_k;
  uint64_t seed;
} ets_sampling_config;

/* ets_sampler_sample_batch() with one SamplingConfig per row, for batches that mix requests
 * (LLMSession::decode_one(const SamplingConfig&), llm_session.h:97-98, takes one per call; the
 * reference's engines serve one session per call).  `configs` is a HOST array of `batch` entries,
 * consumed before the call returns.  Row b is sampled as a reference object constructed with
 * (vocab_size, temperature_b, top_p_b) and set_topk(top_k_b) would sample it: temperature 0 is the
 * arg-max and consumes no coin, and the branch order is the reference's (sampler.cpp:238-249).
 * seed_b != 0 restarts row b's coin stream at seed_b before this call's draw (the state a new
 * object with that seed has); seed_b == 0 continues the row's stream.  `d_debug` may be null.
 * Rows are grouped by draw and launched group by group on `hip_stream`; asynchronous. */
ETS_API ets_status ets_sampler_sample_batch_configs(ets_sampler* s, const void* d_logits, int32_t dtype,
                                                   int32_t batch, int64_t row_stride_elems,
                                                   const ets_sampling_config* configs, int32_t* d_tokens,
                                                   ets_row_debug* d_debug, void* hip_stream);

/* The in-graph Gumbel-max sampler, sample(logits, temperature) of
 * examples/models/qwen3_5_moe/sampler.py:17-60 (the same draw as backends/mlx/llm/sampling.py:39-44
 * asks of its backend): token = argmax_i(logits_i / max(T, 1e-6) + g_i) with
 * g_i = -log(-log(u_i + 1e-20) + 1e-20) in fp32, lowest index on ties.  It draws from
 * softmax(logits / T) like the Sampler above but is NOT the same arithmetic: one pass over the
 * row, no softmax sum, so its tokens differ from ets_sampler_sample_batch() for the same seed.
 *   `temperatures`  HOST: one value (a 0-D temperature) or `batch` values (1-D, one per row);
 *   `d_noise`       DEVICE fp32 [batch, vocab_size] of uniforms in [0, 1) -- what
 *                   torch.rand_like(logits) is in the reference -- or NULL: then u_i comes from
 *                   a counter-based generator keyed by row b's coin state and i, and the state
 *                   advances by one xorshift64* step per call;
 *   element types   Float (the reference's contract), Half, BFloat16 (converted to fp32).
 * Asynchronous on `hip_stream`. */
ETS_API ets_status ets_sampler_gumbel_max_batch(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                               int64_t row_stride_elems, const float* temperatures,
                                               int32_t n_temperatures, const float* d_noise, int32_t* d_tokens,
                                               void* hip_stream);

/* Sampling time at microsecond resolution.  The reference's Stats keeps
 * aggregate_sampling_time_ms from host clocks in whole milliseconds
 * (extension/llm/runner/stats.h:46-47, on_sampling_begin / on_sampling_end :62-69), which reads 0
 * for a sampler that takes tens of microseconds.  With timing enabled every
 * ets_sampler_sample_batch*() call is bracketed by HIP events on its stream; the totals are
 * device time of the call's launches. */
typedef struct ets_sampler_stats {
  uint64_t calls;                    /* timed calls that have completed                      */
  uint64_t rows;                     /* rows sampled by them                                 */
  double aggregate_sampling_time_us; /* Stats::aggregate_sampling_time_ms, in microseconds   */
  double last_call_us;               /* the most recent completed call                       */
} ets_sampler_stats;

/* Off by default (two event records per call when on). */
ETS_API ets_status ets_sampler_set_timing(ets_sampler* s, int32_t enabled);
/* Waits for the timed calls still in flight, then copies the totals. */
ETS_API ets_status ets_sampler_get_stats(ets_sampler* s, ets_sampler_stats* out);
/* Stats::reset()  -- stats.h:83-110. */
ETS_API ets_status ets_sampler_reset_stats(ets_sampler* s);

/* Per-row xorshift64* states (sampler.h:82 `rng_state_`, one per row here).  HOST pointers to
 * `count` values for rows [first_row, first_row + count).  Lets a run be replayed or resumed. */
ETS_API ets_status ets_sampler_set_rng_states(ets_sampler* s, int32_t first_row, int32_t count,
                                              const uint64_t* states);
ETS_API ets_status ets_sampler_get_rng_states(ets_sampler* s, int32_t first_row, int32_t count, uint64_t* states);

/* sample_from_logits(const Tensor&, Sampler&)  -- util.h:25-55.  The tensor is passed as
 * (HOST data, dtype, rank, sizes[rank]); rank 3 samples the last position of batch 0, the
 * last dimension must equal the handle's vocab_size.  An unsupported dtype returns
 * ETS_INVALID_ARGUMENT where the reference aborts (util.h:30-34). */
ETS_API ets_status ets_sample_from_logits(ets_sampler* s, const void* data, int32_t dtype, int32_t rank,
                                          const int64_t* sizes, int32_t* token_out);

/* The batched adapter: sample_from_logits() for a tensor that lives in DEVICE memory and for
 * every batch entry (the reference's adapter reads a host tensor and batch 0 only, util.h:25-55,
 * :48-51).  `d_data` is a DEVICE pointer to a contiguous [batch, vocab] (rank 2) or
 * [batch, seq, vocab] (rank 3: the last position of every batch entry) tensor, `sizes` a HOST
 * array of `rank` extents, `d_tokens` a DEVICE pointer to `batch` int32.  This is the call a
 * runner makes when its delegate leaves the logits on the GPU
 * (backends/cuda/runtime/cuda_backend.cpp:80-81): only the tokens cross to the host.  Row b uses
 * its own coin stream, as in ets_sampler_sample_batch(); asynchronous on `hip_stream`. */
ETS_API ets_status ets_sample_from_logits_batch(ets_sampler* s, const void* d_data, int32_t dtype, int32_t rank,
                                                const int64_t* sizes, int32_t* d_tokens, void* hip_stream);

/* logits_to_token(const Tensor&, float temperature = 0)  -- util.h:64-71: a temporary
 * 2-argument Sampler over the tensor's last dimension.  The reference builds that object per
 * call, which costs it nothing; a handle here owns device buffers, so every calling THREAD keeps
 * the handle of its last call (about vocab x 4 bytes of row staging plus the work buffers of the
 * draw, held until the thread ends) and reuses it while device and vocabulary stay the same; the
 * 2-argument constructor's parameters and a clock seed are set again on every call.  The cached
 * handle is dropped without freeing when the HIP runtime has been torn down or the device reset. */
ETS_API ets_status ets_logits_to_token(const void* data, int32_t dtype, int32_t rank, const int64_t* sizes,
                                       float temperature, int32_t* token_out);

/* random_u32 / random_f32  -- sampler.cpp:210-220, on the host (exported so callers can
 * predict or replay a row's coins). */
ETS_API uint32_t ets_random_u32(uint64_t* state);
ETS_API float ets_random_f32(uint64_t* state);

/* Text of the last error on this handle ("" if none); valid until the next call on it.
 * With s == NULL: the last error of a failed create / handle-less call on this thread. */
ETS_API const char* ets_sampler_last_error(const ets_sampler* s);

/* Library version string. */
ETS_API const char* ets_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ET_SAMPLER_H_ */
