/* TEST INFRASTRUCTURE ONLY -- C interface of the CPU restatement of ExecuTorch's LLM
 * token sampler (see sampler_oracle.cpp for the reference file:line each function follows).
 * Loaded by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; never by the
 * product library. */
#ifndef ET_SAMPLER_ORACLE_H_
#define ET_SAMPLER_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* executorch ScalarType codes (runtime/core/portable_type/scalar_type.h:98-125) */
#define ORACLE_DTYPE_HALF 5
#define ORACLE_DTYPE_FLOAT 6
#define ORACLE_DTYPE_BFLOAT16 15
#define ORACLE_DTYPE_UINT16 27

/* arithmetic mode */
#define ORACLE_MODE_NATIVE 0 /* Sampler::sample<T> on the caller's T buffer (mutated)      */
#define ORACLE_MODE_UPCAST 1 /* convert the row to fp32, then Sampler::sample<float>       */

/* order among exactly equal probabilities when sorting candidates */
#define ORACLE_TIE_LIBSTDCXX 0 /* whatever std::sort / std::partial_sort leave (reference) */
#define ORACLE_TIE_STABLE 1    /* ascending token index                                    */

#define ORACLE_BRANCH_ARGMAX 0
#define ORACLE_BRANCH_MULTINOMIAL 1
#define ORACLE_BRANCH_TOPP 2
#define ORACLE_BRANCH_TOPK 3

typedef struct {
  int32_t vocab_size;
  float inv_temperature;
  float topp;
  int32_t topk;
  uint64_t rng_state;
} oracle_sampler_t;

/* Intermediate values of one sample() call, for classifying token mismatches. */
typedef struct {
  int32_t branch;
  float max_val;      /* row maximum after temperature scaling                  */
  float sum;          /* softmax normaliser as accumulated by the reference      */
  float coin;
  int32_t n_candidates; /* entries that survived the top-p cutoff (or V for top-k) */
  int32_t last_idx;     /* last sorted position inside the nucleus                 */
  float cumulative;     /* probability mass of the nucleus                         */
  float r;              /* coin scaled into the nucleus                            */
  int32_t position;     /* sorted position of the returned token                   */
  float p_token;        /* probability of the returned token                       */
} oracle_explain_t;

uint32_t oracle_random_u32(uint64_t* state);
float oracle_random_f32(uint64_t* state);

void oracle_sampler_init(oracle_sampler_t* s, int32_t vocab_size, float temperature, float topp,
                         uint64_t rng_seed);
void oracle_sampler_set_temperature(oracle_sampler_t* s, float temperature);
void oracle_sampler_set_topk(oracle_sampler_t* s, int32_t topk);

/* One sample() call.  Returns the token; -1 where the reference's behaviour is undefined
 * (no candidate survives, integer divide by zero), -2 for an unsupported dtype. */
int32_t oracle_sample(oracle_sampler_t* s, void* logits, int32_t dtype, int32_t mode, int32_t tie,
                      oracle_explain_t* explain, float* probs_out);

void oracle_sample_rows(int32_t vocab_size, float inv_temperature, float topp, int32_t topk,
                        const void* logits, int32_t dtype, int64_t row_stride_elems, int32_t row_begin,
                        int32_t row_end, uint64_t* rng_states, int32_t* tokens, int32_t mode, int32_t tie,
                        oracle_explain_t* explains);

int32_t oracle_sample_from_logits(oracle_sampler_t* s, void* data, int32_t dtype, int32_t rank,
                                  const int64_t* sizes, int32_t mode, int32_t tie);

void oracle_exp2_table(uint64_t* out32);
float oracle_expf_restated(float x);
void oracle_expf_restated_many(const float* x, float* y, int64_t n);
void oracle_expf_libm_many(const float* x, float* y, int64_t n);

uint16_t oracle_bf16_from_float(float f);
float oracle_bf16_to_float(uint16_t h);
uint16_t oracle_half_from_float(float f);
float oracle_half_to_float(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif /* ET_SAMPLER_ORACLE_H_ */
