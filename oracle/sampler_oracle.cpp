// TEST INFRASTRUCTURE ONLY -- CPU restatement of ExecuTorch's LLM token sampler.
//
// This file is the checker that the HIP sampler is compared against.  Only tests/,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it; the product
// library (executorch_amd/csrc) never links, calls or falls back to it.
//
// What it restates (all paths relative to the reference tree):
//   extension/llm/sampler/sampler.cpp:44-56    argmax          -> arg_max()
//   extension/llm/sampler/sampler.cpp:58-70    multinomial     -> draw_multinomial()
//   extension/llm/sampler/sampler.cpp:72-120   top-k           -> draw_topk()
//   extension/llm/sampler/sampler.cpp:122-171  top-p (nucleus) -> draw_topp()
//   extension/llm/sampler/sampler.cpp:173-187  constructors    -> oracle_sampler_init()
//   extension/llm/sampler/sampler.cpp:189-208  softmax         -> soft_max()
//   extension/llm/sampler/sampler.cpp:210-220  xorshift64* RNG -> oracle_random_u32/f32()
//   extension/llm/sampler/sampler.cpp:222-251  dispatch        -> sample_row()
//   extension/llm/sampler/sampler.h:48-60      setters         -> oracle_sampler_set_*()
//   extension/llm/sampler/util.h:25-55         tensor adapter  -> oracle_sample_from_logits()
// Scalar semantics of the 16-bit types (every arithmetic result is computed in float and
// rounded back to the storage type):
//   runtime/core/portable_type/c10/torch/headeronly/util/BFloat16.h:100-114,186-228
//   runtime/core/portable_type/c10/torch/headeronly/util/Half.h:118-299,501-547
//
// Third-party arithmetic the reference relies on and how it is treated here:
//   * expf  -- glibc libm (2.35 in this image).  The oracle calls the same libm, and also
//     carries oracle_expf_restated(), a restatement of glibc's published algorithm
//     (sysdeps/ieee754/flt-32/e_expf.c, the Arm "optimized routines" exp2f-table scheme)
//     which is what the GPU evaluates.  tests/test_oracle_expf.py pins the restatement
//     against libm over sampled and boundary inputs; oracle/expf_sweep.c does it
//     exhaustively over every float.
//   * std::sort / std::partial_sort -- libstdc++ (GCC 11).  ORACLE_TIE_LIBSTDCXX calls the
//     same templates on the same record layout, so tie order matches the reference build;
//     ORACLE_TIE_STABLE orders equal probabilities by ascending index (the rule the GPU
//     uses).  The two can only differ where probabilities tie exactly.
//
// Parity status: every function here is pinned -- by the reference's own test expectations
// (tests/test_reference_expectations.py), closed forms and brute force
// (tests/test_oracle_pins.py), golden vectors written from the compiled reference
// (tests/golden/) and, where /root/reference is mounted, a bit-for-bit A/B against
// oracle/_ref (tests/test_oracle_vs_ref.py).

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <memory>
#include <vector>

#include "sampler_oracle.h"

namespace {

inline uint32_t f2u(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float u2f(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// ---- 16-bit storage types: conversions --------------------------------------------------

// BFloat16.h:100-114: NaN -> 0x7FC0, otherwise round-to-nearest-even on the dropped 16 bits.
inline uint16_t bf16_from_float(float f) {
  if (f != f) return 0x7FC0;
  uint32_t u = f2u(f);
  uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
  return static_cast<uint16_t>((u + bias) >> 16);
}
inline float bf16_to_float(uint16_t h) { return u2f(static_cast<uint32_t>(h) << 16); }

// Half.h:118-299: IEEE binary16 <-> binary32, round-to-nearest-even, NaN -> sign|0x7E00.
inline float half_to_float(uint16_t h) {
  uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  if (exp == 0x1Fu) return u2f(sign | 0x7F800000u | (man << 13));
  if (exp != 0) return u2f(sign | ((exp + 112u) << 23) | (man << 13));
  if (man == 0) return u2f(sign);
  // subnormal half: man * 2^-24, exact in float
  float v = static_cast<float>(man) * 5.9604644775390625e-08f;
  return u2f(f2u(v) | sign);
}
inline uint16_t half_from_float(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return sign | 0x7E00u;       // NaN
  if (a >= 0x477FF000u) return sign | 0x7C00u;      // >= 65520 rounds to inf (also inf)
  if (a < 0x33000001u) return sign;                 // <= 2^-25 rounds to zero (tie to even)
  int32_t e = static_cast<int32_t>(a >> 23) - 127;  // unbiased exponent
  uint32_t m = (a & 0x7FFFFFu) | 0x800000u;         // 24-bit significand
  int shift;                                        // bits dropped from m
  uint32_t base;
  if (e >= -14) {
    shift = 13;
    base = static_cast<uint32_t>(e + 15) << 10;
    m &= 0x7FFFFFu;
  } else {
    shift = 13 + (-14 - e);
    base = 0;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1;  // carries propagate into the exponent
  return sign | static_cast<uint16_t>(base + q);
}

// ---- arithmetic policies -----------------------------------------------------------------
// Each policy says how a value of the logits type is stored, read as float, and how a float
// result is rounded on assignment.  `rnd(x)` is "assign float x to a T, read it back".

struct PolicyF32 {
  using store_t = float;
  static constexpr int kDtype = ORACLE_DTYPE_FLOAT;
  static float load(store_t v) { return v; }
  static store_t store(float v) { return v; }
  static float rnd(float v) { return v; }
};
struct PolicyBF16 {
  using store_t = uint16_t;
  static constexpr int kDtype = ORACLE_DTYPE_BFLOAT16;
  static float load(store_t v) { return bf16_to_float(v); }
  static store_t store(float v) { return bf16_from_float(v); }
  static float rnd(float v) { return bf16_to_float(bf16_from_float(v)); }
};
struct PolicyF16 {
  using store_t = uint16_t;
  static constexpr int kDtype = ORACLE_DTYPE_HALF;
  static float load(store_t v) { return half_to_float(v); }
  static store_t store(float v) { return half_from_float(v); }
  static float rnd(float v) { return half_to_float(half_from_float(v)); }
};

// Record sorted by top-p / top-k: same layout as sampler.h:31-35 for each T so that the
// libstdc++ sort templates make the same moves as in the reference build.
template <typename S>
struct Cand {
  S prob;
  int32_t index;
};

// ---- sampler.cpp:44-56 -------------------------------------------------------------------
template <typename P>
int32_t arg_max(const typename P::store_t* v, int32_t n) {
  int32_t best = 0;
  float best_v = P::load(v[0]);
  for (int32_t i = 1; i < n; ++i) {
    float x = P::load(v[i]);
    if (x > best_v) {  // strict: the lowest index wins ties; NaN never wins
      best = i;
      best_v = x;
    }
  }
  return best;
}

// ---- sampler.cpp:189-208 -----------------------------------------------------------------
// In place.  Every intermediate is rounded to the storage type, in index order.
template <typename P>
void soft_max(typename P::store_t* x, int32_t n, float* max_out, float* sum_out) {
  float m = P::load(x[0]);
  for (int32_t i = 1; i < n; ++i) {
    float v = P::load(x[i]);
    if (v > m) m = v;
  }
  float sum = P::rnd(0.0f);
  for (int32_t i = 0; i < n; ++i) {
    float d = P::rnd(P::load(x[i]) - m);
    float e = P::rnd(expf(d));
    x[i] = P::store(e);
    sum = P::rnd(sum + e);
  }
  for (int32_t i = 0; i < n; ++i) {
    x[i] = P::store(P::load(x[i]) / sum);
  }
  if (max_out) *max_out = m;
  if (sum_out) *sum_out = sum;
}

// ---- sampler.cpp:58-70 -------------------------------------------------------------------
template <typename P>
int32_t draw_multinomial(const typename P::store_t* p, int32_t n, float coin) {
  float cdf = P::rnd(0.0f);
  for (int32_t i = 0; i < n; ++i) {
    cdf = P::rnd(cdf + P::load(p[i]));
    if (coin < cdf) return i;
  }
  return n - 1;
}

template <typename P>
void order_candidates(Cand<typename P::store_t>* c, int32_t n0, int32_t k_partial, int tie) {
  using C = Cand<typename P::store_t>;
  if (tie == ORACLE_TIE_STABLE) {
    auto by_prob_then_index = [](const C& a, const C& b) {
      float pa = P::load(a.prob), pb = P::load(b.prob);
      if (pa > pb) return true;
      if (pa < pb) return false;
      return a.index < b.index;
    };
    if (k_partial >= 0) {
      std::partial_sort(c, c + k_partial, c + n0, by_prob_then_index);
    } else {
      std::sort(c, c + n0, by_prob_then_index);
    }
  } else {
    auto by_prob = [](const C& a, const C& b) { return P::load(a.prob) > P::load(b.prob); };
    if (k_partial >= 0) {
      std::partial_sort(c, c + k_partial, c + n0, by_prob);
    } else {
      std::sort(c, c + n0, by_prob);
    }
  }
}

// ---- sampler.cpp:72-120 ------------------------------------------------------------------
template <typename P>
int32_t draw_topk(const typename P::store_t* p, int32_t n, int32_t topk, float coin, int tie,
                  oracle_explain_t* ex) {
  using C = Cand<typename P::store_t>;
  const int32_t k = std::min(topk, n);
  if (k <= 0) return 0;
  std::unique_ptr<C[]> c(new C[n]());
  for (int32_t i = 0; i < n; ++i) {
    c[i].index = i;
    c[i].prob = p[i];
  }
  order_candidates<P>(c.get(), n, k, tie);
  float total = 0.0f;  // float accumulators for every T
  for (int32_t i = 0; i < k; ++i) total += P::load(c[i].prob);
  const float r = coin * total;
  float cdf = 0.0f;
  int32_t pos = k - 1;
  for (int32_t i = 0; i < k; ++i) {
    cdf += P::load(c[i].prob);
    if (r < cdf) {
      pos = i;
      break;
    }
  }
  if (ex) {
    ex->n_candidates = n;
    ex->last_idx = k - 1;
    ex->cumulative = total;
    ex->r = r;
    ex->position = pos;
    ex->p_token = P::load(c[pos].prob);
  }
  return c[pos].index;
}

// ---- sampler.cpp:122-171 -----------------------------------------------------------------
template <typename P>
int32_t draw_topp(const typename P::store_t* p, int32_t n, float topp, float coin, int tie,
                  oracle_explain_t* ex) {
  using C = Cand<typename P::store_t>;
  std::unique_ptr<C[]> c(new C[n]());
  const float cutoff = (1.0f - topp) / (n - 1);
  int32_t n0 = 0;
  for (int32_t i = 0; i < n; ++i) {
    if (P::load(p[i]) >= cutoff) {
      c[n0].index = i;
      c[n0].prob = p[i];
      ++n0;
    }
  }
  order_candidates<P>(c.get(), n0, -1, tie);

  float cumulative = P::rnd(0.0f);
  int32_t last_idx = n0 - 1;
  for (int32_t i = 0; i < n0; ++i) {
    cumulative = P::rnd(cumulative + P::load(c[i].prob));
    if (cumulative > topp) {
      last_idx = i;
      break;
    }
  }
  const float r = P::rnd(coin * cumulative);
  float cdf = P::rnd(0.0f);
  int32_t pos = last_idx;
  for (int32_t i = 0; i <= last_idx; ++i) {
    cdf = P::rnd(cdf + P::load(c[i].prob));
    if (r < cdf) {
      pos = i;
      break;
    }
  }
  if (ex) {
    ex->n_candidates = n0;
    ex->last_idx = last_idx;
    ex->cumulative = cumulative;
    ex->r = r;
    ex->position = pos;
    ex->p_token = pos >= 0 ? P::load(c[pos].prob) : 0.0f;
  }
  // The reference reads probindex[-1] when no entry survives the cutoff (NaN rows):
  // undefined there, reported as -1 here.
  return pos >= 0 ? c[pos].index : -1;
}

// ---- sampler.cpp:222-251 -----------------------------------------------------------------
template <typename P>
int32_t sample_row(oracle_sampler_t* s, typename P::store_t* logits, int tie,
                   oracle_explain_t* ex) {
  const int32_t n = s->vocab_size;
  if (ex) std::memset(ex, 0, sizeof(*ex));
  if (s->inv_temperature == 0.0f) {
    if (ex) ex->branch = ORACLE_BRANCH_ARGMAX;
    return arg_max<P>(logits, n);
  }
  // sampler.cpp:231-233.  For the 16-bit types the only viable operator*= takes a T on the
  // right, so the inverse temperature is rounded to T first.
  const float inv = P::rnd(s->inv_temperature);
  for (int32_t q = 0; q < n; ++q) logits[q] = P::store(P::load(logits[q]) * inv);
  float m = 0.f, sum = 0.f;
  soft_max<P>(logits, n, &m, &sum);
  const float coin = oracle_random_f32(&s->rng_state);
  if (ex) {
    ex->max_val = m;
    ex->sum = sum;
    ex->coin = coin;
  }
  if (s->topk > 0 && s->topk < n) {
    if (ex) ex->branch = ORACLE_BRANCH_TOPK;
    return draw_topk<P>(logits, n, s->topk, coin, tie, ex);
  }
  if (s->topp <= 0 || s->topp >= 1) {
    if (ex) ex->branch = ORACLE_BRANCH_MULTINOMIAL;
    return draw_multinomial<P>(logits, n, coin);
  }
  if (ex) ex->branch = ORACLE_BRANCH_TOPP;
  return draw_topp<P>(logits, n, s->topp, coin, tie, ex);
}

// ---- the uint16_t instantiation (sampler.cpp:254) ----------------------------------------
// Integer arithmetic throughout: the scaled logit is truncated back to uint16, "exp" is
// expf(int) truncated to 0/1, the sum and the division are integer.  Kept for completeness;
// its only sensible use in the reference is argmax over quantised logits.
int32_t sample_row_u16(oracle_sampler_t* s, uint16_t* logits, int tie, oracle_explain_t* ex) {
  const int32_t n = s->vocab_size;
  if (ex) std::memset(ex, 0, sizeof(*ex));
  if (s->inv_temperature == 0.0f) {
    if (ex) ex->branch = ORACLE_BRANCH_ARGMAX;
    int32_t best = 0;
    uint16_t bv = logits[0];
    for (int32_t i = 1; i < n; ++i)
      if (logits[i] > bv) {
        best = i;
        bv = logits[i];
      }
    return best;
  }
  for (int32_t q = 0; q < n; ++q) {
    float v = static_cast<float>(logits[q]) * s->inv_temperature;
    logits[q] = static_cast<uint16_t>(static_cast<int32_t>(v));  // x86 truncation, low 16 bits
  }
  uint16_t m = logits[0];
  for (int32_t i = 1; i < n; ++i)
    if (logits[i] > m) m = logits[i];
  uint16_t sum = 0;
  for (int32_t i = 0; i < n; ++i) {
    int d = static_cast<int>(logits[i]) - static_cast<int>(m);
    logits[i] = static_cast<uint16_t>(static_cast<int32_t>(expf(static_cast<float>(d))));
    sum = static_cast<uint16_t>(sum + logits[i]);
  }
  if (sum == 0) return -1;  // the reference divides by zero here
  for (int32_t i = 0; i < n; ++i) logits[i] = static_cast<uint16_t>(logits[i] / sum);
  const float coin = oracle_random_f32(&s->rng_state);
  if (ex) {
    ex->max_val = m;
    ex->sum = sum;
    ex->coin = coin;
  }
  using C = Cand<uint16_t>;
  auto desc = [tie](const C& a, const C& b) {
    if (a.prob != b.prob) return a.prob > b.prob;
    return tie == ORACLE_TIE_STABLE ? a.index < b.index : false;
  };
  if (s->topk > 0 && s->topk < n) {
    const int32_t k = std::min(s->topk, n);
    std::unique_ptr<C[]> c(new C[n]());
    for (int32_t i = 0; i < n; ++i) c[i] = C{logits[i], i};
    std::partial_sort(c.get(), c.get() + k, c.get() + n, desc);
    float total = 0.f;
    for (int32_t i = 0; i < k; ++i) total += static_cast<float>(c[i].prob);
    const float r = coin * total;
    float cdf = 0.f;
    for (int32_t i = 0; i < k; ++i) {
      cdf += static_cast<float>(c[i].prob);
      if (r < cdf) return c[i].index;
    }
    return c[k - 1].index;
  }
  if (s->topp <= 0 || s->topp >= 1) {
    uint16_t cdf = 0;
    for (int32_t i = 0; i < n; ++i) {
      cdf = static_cast<uint16_t>(cdf + logits[i]);
      if (coin < static_cast<float>(cdf)) return i;
    }
    return n - 1;
  }
  std::unique_ptr<C[]> c(new C[n]());
  const float cutoff = (1.0f - s->topp) / (n - 1);
  int32_t n0 = 0;
  for (int32_t i = 0; i < n; ++i)
    if (static_cast<float>(logits[i]) >= cutoff) c[n0++] = C{logits[i], i};
  std::sort(c.get(), c.get() + n0, desc);
  uint16_t cumulative = 0;
  int32_t last_idx = n0 - 1;
  for (int32_t i = 0; i < n0; ++i) {
    cumulative = static_cast<uint16_t>(cumulative + c[i].prob);
    if (static_cast<float>(cumulative) > s->topp) {
      last_idx = i;
      break;
    }
  }
  const uint16_t r = static_cast<uint16_t>(static_cast<int32_t>(coin * static_cast<float>(cumulative)));
  uint16_t cdf = 0;
  for (int32_t i = 0; i <= last_idx; ++i) {
    cdf = static_cast<uint16_t>(cdf + c[i].prob);
    if (r < cdf) return c[i].index;
  }
  return last_idx >= 0 ? c[last_idx].index : -1;
}

template <typename P>
int32_t sample_upcast(oracle_sampler_t* s, const typename P::store_t* logits, int tie,
                      oracle_explain_t* ex, float* probs_out) {
  // The "convert the row to fp32, then sample<float>" convention of
  // examples/models/gemma4/runner/gemma4_runner.cpp:166-182 and
  // examples/models/voxtral_realtime/voxtral_realtime_runner.cpp:256-282.
  const int32_t n = s->vocab_size;
  std::vector<float> tmp;
  float* buf = probs_out;
  if (!buf) {
    tmp.resize(n);
    buf = tmp.data();
  }
  for (int32_t i = 0; i < n; ++i) buf[i] = P::load(logits[i]);
  return sample_row<PolicyF32>(s, buf, tie, ex);
}

}  // namespace

extern "C" {

// ---- sampler.cpp:210-220 -----------------------------------------------------------------
uint32_t oracle_random_u32(uint64_t* state) {
  uint64_t s = *state;
  s ^= s >> 12;
  s ^= s << 25;
  s ^= s >> 27;
  *state = s;
  return static_cast<uint32_t>((s * 0x2545F4914F6CDD1Dull) >> 32);
}

float oracle_random_f32(uint64_t* state) {
  return static_cast<float>(oracle_random_u32(state) >> 8) / 16777216.0f;
}

// ---- sampler.cpp:173-181 (the 2-argument form at :183-187 seeds from the clock and has no
// deterministic restatement; callers pass topp = 0.9f and a seed of their choice) -------------
void oracle_sampler_init(oracle_sampler_t* s, int32_t vocab_size, float temperature, float topp,
                         uint64_t rng_seed) {
  s->vocab_size = vocab_size;
  s->inv_temperature = (temperature != 0.0f) ? 1.0f / temperature : 0.0f;  // no clamping
  s->topp = topp;
  s->topk = 0;
  s->rng_state = rng_seed;
}

// ---- sampler.h:48-53 ---------------------------------------------------------------------
void oracle_sampler_set_temperature(oracle_sampler_t* s, float temperature) {
  if (temperature < 0.0f) temperature = 0.0f;
  s->inv_temperature = (temperature != 0.0f) ? 1.0f / temperature : 0.0f;
}

// ---- sampler.h:58-60 ---------------------------------------------------------------------
void oracle_sampler_set_topk(oracle_sampler_t* s, int32_t topk) { s->topk = topk; }

int32_t oracle_sample(oracle_sampler_t* s, void* logits, int32_t dtype, int32_t mode, int32_t tie,
                      oracle_explain_t* explain, float* probs_out) {
  if (mode == ORACLE_MODE_NATIVE) {
    switch (dtype) {
      case ORACLE_DTYPE_FLOAT:
        return sample_row<PolicyF32>(s, static_cast<float*>(logits), tie, explain);
      case ORACLE_DTYPE_BFLOAT16:
        return sample_row<PolicyBF16>(s, static_cast<uint16_t*>(logits), tie, explain);
      case ORACLE_DTYPE_HALF:
        return sample_row<PolicyF16>(s, static_cast<uint16_t*>(logits), tie, explain);
      case ORACLE_DTYPE_UINT16:
        return sample_row_u16(s, static_cast<uint16_t*>(logits), tie, explain);
      default:
        return -2;
    }
  }
  // ORACLE_MODE_UPCAST: the caller's buffer is left untouched; probabilities (fp32) go to
  // probs_out when given.
  switch (dtype) {
    case ORACLE_DTYPE_FLOAT:
      return sample_upcast<PolicyF32>(s, static_cast<const float*>(logits), tie, explain, probs_out);
    case ORACLE_DTYPE_BFLOAT16:
      return sample_upcast<PolicyBF16>(s, static_cast<const uint16_t*>(logits), tie, explain, probs_out);
    case ORACLE_DTYPE_HALF:
      return sample_upcast<PolicyF16>(s, static_cast<const uint16_t*>(logits), tie, explain, probs_out);
    case ORACLE_DTYPE_UINT16: {
      // quantised logits are integers; as floats they are exact up to 65535
      const int32_t n = s->vocab_size;
      std::vector<float> tmp(n);
      const uint16_t* q = static_cast<const uint16_t*>(logits);
      for (int32_t i = 0; i < n; ++i) tmp[i] = static_cast<float>(q[i]);
      int32_t t = sample_row<PolicyF32>(s, tmp.data(), tie, explain);
      if (probs_out) std::memcpy(probs_out, tmp.data(), sizeof(float) * n);
      return t;
    }
    default:
      return -2;
  }
}

// Batched form used by the parity tests and the CPU baseline: row b has its own sampler
// state (rng_states[b]); all rows share temperature / top-p / top-k.  Rows [row_begin,
// row_end) are processed so that callers can split a batch over threads.
void oracle_sample_rows(int32_t vocab_size, float inv_temperature, float topp, int32_t topk,
                        const void* logits, int32_t dtype, int64_t row_stride_elems, int32_t row_begin,
                        int32_t row_end, uint64_t* rng_states, int32_t* tokens, int32_t mode, int32_t tie,
                        oracle_explain_t* explains) {
  const size_t esz = (dtype == ORACLE_DTYPE_FLOAT) ? 4 : 2;
  std::vector<unsigned char> scratch(static_cast<size_t>(vocab_size) * esz);
  for (int32_t b = row_begin; b < row_end; ++b) {
    oracle_sampler_t s;
    s.vocab_size = vocab_size;
    s.inv_temperature = inv_temperature;
    s.topp = topp;
    s.topk = topk;
    s.rng_state = rng_states[b];
    const unsigned char* src = static_cast<const unsigned char*>(logits) + static_cast<size_t>(b) * row_stride_elems * esz;
    std::memcpy(scratch.data(), src, scratch.size());  // native mode mutates its input
    tokens[b] = oracle_sample(&s, scratch.data(), dtype, mode, tie, explains ? explains + b : nullptr, nullptr);
    rng_states[b] = s.rng_state;
  }
}

// ---- util.h:25-55 ------------------------------------------------------------------------
// Tensor described by (data, dtype, rank, sizes): rank 3 samples the last position of
// batch 0, any other rank samples the first `vocab` elements.  Returns -2 for a dtype the
// reference would abort on.
int32_t oracle_sample_from_logits(oracle_sampler_t* s, void* data, int32_t dtype, int32_t rank,
                                  const int64_t* sizes, int32_t mode, int32_t tie) {
  if (dtype != ORACLE_DTYPE_FLOAT && dtype != ORACLE_DTYPE_HALF && dtype != ORACLE_DTYPE_BFLOAT16 &&
      dtype != ORACLE_DTYPE_UINT16)
    return -2;
  const int64_t vocab = sizes[rank - 1];
  const size_t esz = (dtype == ORACLE_DTYPE_FLOAT) ? 4 : 2;
  unsigned char* p = static_cast<unsigned char*>(data);
  if (rank == 3) p += static_cast<size_t>((sizes[1] - 1) * vocab) * esz;
  (void)vocab;
  return oracle_sample(s, p, dtype, mode, tie, nullptr, nullptr);
}

// ---- glibc expf, restated (sysdeps/ieee754/flt-32/e_expf.c + exp2f table data) -----------
// exp(x) = 2^(k/32) * 2^(r/32) with k = round(x*32/ln2); 2^(k/32) comes from a 32-entry table
// of doubles, 2^(r/32) from a cubic in r, everything in double, one final rounding to float.
// Written with explicit fused multiply-adds at every multiply-add of the source, which is
// what the x86-64 FMA build of glibc (the variant its ifunc selects on the hosts used here)
// compiles to: with the reduction r = fma(32/ln2, x, -k) fused, expf_sweep finds 0 of 2^32
// inputs that differ from libm; unfused it finds 2 (x = 0x1.04845ep+5 and -0x1.f8cbb2p+5).
static uint64_t g_exp2_tab[32];
static bool g_exp2_tab_ready = false;

static void build_exp2_table() {
  // tab[i] = bits(2^(i/32)) - (i << 47); exp2() of a double with 5 fractional bits is
  // correctly rounded in glibc (its error bound is far below the distance of these values
  // to a rounding boundary), tests pin the first/last entries against published constants.
  for (int i = 0; i < 32; ++i) {
    double v = exp2(static_cast<double>(i) / 32.0);
    uint64_t b;
    std::memcpy(&b, &v, 8);
    g_exp2_tab[i] = b - (static_cast<uint64_t>(i) << 47);
  }
  g_exp2_tab_ready = true;
}

void oracle_exp2_table(uint64_t* out32) {
  if (!g_exp2_tab_ready) build_exp2_table();
  std::memcpy(out32, g_exp2_tab, sizeof(g_exp2_tab));
}

float oracle_expf_restated(float x) {
  if (!g_exp2_tab_ready) build_exp2_table();
  const uint32_t ux = f2u(x);
  const uint32_t abstop = (ux >> 20) & 0x7FFu;
  if (abstop >= 0x42Bu) {  // |x| >= 88 or NaN/inf
    if (ux == 0xFF800000u) return 0.0f;
    if (abstop >= 0x7F8u) return x + x;
    if (x > 88.72283172607421875f) return INFINITY;      // 0x1.62e42ep6f
    if (x < -103.97207641601562500f) return 0.0f;        // -0x1.9fe368p6f
  }
  const double invln2n = 0x1.71547652b82fep+0 * 32.0;
  const double shift = 0x1.8p+52;
  const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
  const double c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
  const double c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
  const double xd = static_cast<double>(x);
  double kd = __builtin_fma(invln2n, xd, shift);  // round(x*32/ln2) lands in the low bits
  uint64_t ki;
  std::memcpy(&ki, &kd, 8);
  kd -= shift;
  const double r = __builtin_fma(invln2n, xd, -kd);
  uint64_t t = g_exp2_tab[ki % 32];
  t += ki << 47;
  double s;
  std::memcpy(&s, &t, 8);
  const double zz = __builtin_fma(c0, r, c1);
  const double r2 = r * r;
  double y = __builtin_fma(c2, r, 1.0);
  y = __builtin_fma(zz, r2, y);
  y = y * s;
  return static_cast<float>(y);
}

// Bulk helpers so that Python can compare long ranges without a per-call round trip.
void oracle_expf_restated_many(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = oracle_expf_restated(x[i]);
}
void oracle_expf_libm_many(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = expf(x[i]);
}

// Type conversions, exported so that tests can pin them against numpy / torch.
uint16_t oracle_bf16_from_float(float f) { return bf16_from_float(f); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
uint16_t oracle_half_from_float(float f) { return half_from_float(f); }
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

}  // extern "C"
