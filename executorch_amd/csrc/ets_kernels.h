// gfx950 kernels of the token sampler.
//
//   argmax_kernel        temperature == 0 (Sampler::sample_argmax, sampler.cpp:44-56)
//   sample_rows_kernel   temperature != 0: scale, softmax, coin, top-k / multinomial / top-p
//                        (sampler.cpp:58-171, 189-251), one workgroup per row
//
// Everything that the reference computes with a sequential fp32 loop (the softmax sum, the
// nucleus mass, the CDF walks) goes through seq_sum_block(), so the results carry the same
// rounding as the scalar loops they replace.
#pragma once

#include "ets_device.h"

namespace ets {

struct RowDebug {  // layout of ets_row_debug in include/et_sampler.h
  float max_val, sum, coin, cumulative, r;
  int32_t n_candidates, last_idx, position;
};

struct RowParams {
  const void* logits;
  int64_t row_stride;  // elements between rows
  int32_t vocab;
  float inv_temperature;
  float topp;
  int32_t topk;
  uint64_t* rng;      // [batch] xorshift64* states
  int32_t* tokens;    // [batch]
  float* probs;       // [batch, vocab] or null
  RowDebug* debug;    // [batch] or null
  uint64_t* scratch;  // [batch, scratch_stride] candidate keys
  int64_t scratch_stride;
  int32_t lds_keys;   // power of two: keys that fit in the dynamic LDS buffer
};

// ---- argmax ---------------------------------------------------------------------------------
// Order-preserving key of a float: larger float <=> larger key; -0 == +0; NaN lowest.
__device__ __forceinline__ uint32_t order_key(float v) {
  if (v != v) return 0u;
  uint32_t b = __float_as_uint(v);
  if (b == 0x80000000u) b = 0u;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    const uint64_t o = __shfl_xor(static_cast<unsigned long long>(v), d);
    v = o > v ? o : v;
  }
  return v;
}

constexpr int kArgmaxBlock = 256;

// grid = (splits, batch).  Each workgroup scans one segment of a row; the workgroup that
// finishes a row last combines the partial results.  counters[] must be zero on entry and is
// left zero.
template <int DT>
__global__ void __launch_bounds__(kArgmaxBlock)
argmax_kernel(const void* logits_all, int64_t row_stride, int32_t vocab, uint64_t* partials, uint32_t* counters,
              int32_t* tokens) {
  __shared__ uint64_t red[kArgmaxBlock / 64];
  __shared__ int is_last;
  const int row = blockIdx.y;
  const int splits = gridDim.x;
  const int tid = threadIdx.x;
  const char* logits = static_cast<const char*>(logits_all) + static_cast<int64_t>(row) * row_stride * ElemSize<DT>::value;
  const int seg = (vocab + splits - 1) / splits;
  const int lo = blockIdx.x * seg;
  const int hi = min(vocab, lo + seg);
  uint64_t best = 0;
  for (int i = lo + tid; i < hi; i += kArgmaxBlock) {
    uint32_t key;
    if (DT == kDtypeUInt16) {
      key = static_cast<uint32_t>(static_cast<const uint16_t*>(static_cast<const void*>(logits))[i]) + 1u;
    } else {
      key = order_key(load_elem<DT>(logits, i));
    }
    // ties go to the lower index: larger (0xffffffff - i)
    const uint64_t packed = (static_cast<uint64_t>(key) << 32) | (0xffffffffu - static_cast<uint32_t>(i));
    best = packed > best ? packed : best;
  }
  best = wave_max_u64(best);
  if ((tid & 63) == 0) red[tid >> 6] = best;
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < kArgmaxBlock / 64; ++w) best = red[w] > best ? red[w] : best;
    partials[static_cast<int64_t>(row) * splits + blockIdx.x] = best;
    __threadfence();
    const uint32_t done = atomicAdd(&counters[row], 1u);
    is_last = (done == static_cast<uint32_t>(splits - 1));
  }
  __syncthreads();
  if (is_last && tid == 0) {
    __threadfence();
    uint64_t b = 0;
    for (int sp = 0; sp < splits; ++sp) {
      const uint64_t v = __atomic_load_n(&partials[static_cast<int64_t>(row) * splits + sp], __ATOMIC_RELAXED);
      b = v > b ? v : b;
    }
    int32_t token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(b));
    if (DT != kDtypeUInt16) {
      // `x > NaN` is never true: a NaN in slot 0 stays the maximum (sampler.cpp:47-50)
      const float x0 = load_elem<DT>(logits, 0);
      if (x0 != x0) token = 0;
    }
    tokens[row] = token;
    counters[row] = 0u;
  }
}

// ---- sorting candidate keys -----------------------------------------------------------------
// Bitonic merge sub-stages j = j_start, j_start/2, ..., 1 of merge size k on a tile of T keys
// held in LDS whose first key has global position gbase.
__device__ void lds_merge_stages(uint64_t* t, int T, int gbase, int k, int j_start) {
  for (int j = j_start; j > 0; j >>= 1) {
    for (int q = threadIdx.x; q < (T >> 1); q += kBlock) {
      const int i = ((q & ~(j - 1)) << 1) | (q & (j - 1));
      const int l = i | j;
      const bool up = ((gbase + i) & k) == 0;
      const uint64_t a = t[i], b = t[l];
      if ((a > b) == up) {
        t[i] = b;
        t[l] = a;
      }
    }
    __syncthreads();
  }
}

// Ascending sort of keys[0, N), N a power of two, by one workgroup.  `keys` is global memory;
// `lds` holds T keys (T a power of two).  N <= T sorts entirely in LDS.
__device__ void sort_keys_block(uint64_t* keys, int N, uint64_t* lds, int T) {
  const int tid = threadIdx.x;
  if (T > N) T = N;
  for (int base = 0; base < N; base += T) {
    for (int i = tid; i < T; i += kBlock) lds[i] = keys[base + i];
    __syncthreads();
    for (int k = 2; k <= T; k <<= 1) lds_merge_stages(lds, T, base, k, k >> 1);
    for (int i = tid; i < T; i += kBlock) keys[base + i] = lds[i];
    __syncthreads();
  }
  for (int k = T << 1; k <= N; k <<= 1) {
    for (int j = k >> 1; j >= T; j >>= 1) {
      for (int q = tid; q < (N >> 1); q += kBlock) {
        const int i = ((q & ~(j - 1)) << 1) | (q & (j - 1));
        const int l = i | j;
        const bool up = (i & k) == 0;
        const uint64_t a = keys[i], b = keys[l];
        if ((a > b) == up) {
          keys[i] = b;
          keys[l] = a;
        }
      }
      __syncthreads();
    }
    for (int base = 0; base < N; base += T) {
      for (int i = tid; i < T; i += kBlock) lds[i] = keys[base + i];
      __syncthreads();
      lds_merge_stages(lds, T, base, k, T >> 1);
      for (int i = tid; i < T; i += kBlock) keys[base + i] = lds[i];
      __syncthreads();
    }
  }
}

// Candidate key: ascending key order == descending probability, then ascending token index.
__device__ __forceinline__ uint64_t cand_key(float p, int index) {
  return (static_cast<uint64_t>(0xffffffffu - __float_as_uint(p)) << 32) | static_cast<uint32_t>(index);
}
__device__ __forceinline__ float cand_prob(uint64_t key) {
  return __uint_as_float(0xffffffffu - static_cast<uint32_t>(key >> 32));
}

__device__ __forceinline__ int pow2_ceil(int n) {
  int p = 2;
  while (p < n) p <<= 1;
  return p;
}

// ---- the stochastic path: one workgroup per row -------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(kBlock) sample_rows_kernel(RowParams p) {
  extern __shared__ __align__(16) uint64_t lds_keys[];
  __shared__ BlockScratch sm;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int V = p.vocab;
  const float inv = p.inv_temperature;
  const char* logits = static_cast<const char*>(p.logits) + static_cast<int64_t>(row) * p.row_stride * ElemSize<DT>::value;
  float* probs = p.probs ? p.probs + static_cast<int64_t>(row) * V : nullptr;
  uint64_t* scratch = p.scratch + static_cast<int64_t>(row) * p.scratch_stride;
  const float kInf = __uint_as_float(0x7f800000u);
  const float kNaN = __uint_as_float(0x7fc00000u);

  if (tid < 32) sm.exp2tab[tid] = kExp2Table[tid];

  // ---- row maximum of x = logit * inv_temperature (sampler.cpp:231-233, 191-197)
  float m = -kInf;
  for (int i = tid; i < V; i += kBlock) {
    const float x = load_elem<DT>(logits, i) * inv;
    if (x > m) m = x;
  }
  m = wave_max_ignoring_nan(m);
  if (lane == 0) sm.red_f[wave] = m;
  __syncthreads();
  m = sm.red_f[0];
  for (int w = 1; w < kWaves; ++w) m = (sm.red_f[w] > m) ? sm.red_f[w] : m;
  {
    const float x0 = load_elem<DT>(logits, 0) * inv;
    if (x0 != x0) m = x0;  // max_val starts at x[0]; nothing compares greater than NaN
  }
  __syncthreads();

  // ---- softmax normaliser: sum of expf(x - max) in index order (sampler.cpp:199-203)
  bool saw_nan = false;
  auto fetch_e = [&](int i) -> float {
    const float x = load_elem<DT>(logits, i) * inv;
    const float e = expf_exact(x - m, sm.exp2tab);
    if (e != e) {
      saw_nan = true;
      return 0.0f;
    }
    return e;
  };
  float S = seq_sum_block(fetch_e, V, 0.0f, kInf, sm).sum;
  {
    const uint64_t any = __ballot(saw_nan);
    if (lane == 0) sm.red_u[wave] = any ? 1u : 0u;
    __syncthreads();
    uint32_t nan_row = 0;
    for (int w = 0; w < kWaves; ++w) nan_row |= sm.red_u[w];
    if (nan_row) S = kNaN;  // one NaN addend poisons the running sum for good
    __syncthreads();
  }

  // ---- one coin per call (sampler.cpp:237, 210-220)
  if (tid == 0) {
    uint64_t st = p.rng[row];
    st ^= st >> 12;
    st ^= st << 25;
    st ^= st >> 27;
    p.rng[row] = st;
    const uint32_t u = static_cast<uint32_t>((st * 0x2545F4914F6CDD1Dull) >> 32);
    sm.red_f[0] = static_cast<float>(u >> 8) / 16777216.0f;
  }
  __syncthreads();
  const float coin = sm.red_f[0];
  __syncthreads();

  auto prob_at = [&](int i) -> float {
    const float x = load_elem<DT>(logits, i) * inv;
    return expf_exact(x - m, sm.exp2tab) / S;  // sampler.cpp:205-207: a true division
  };
  if (probs) {
    for (int i = tid; i < V; i += kBlock) probs[i] = prob_at(i);
  }

  RowDebug dbg = {m, S, coin, 0.0f, 0.0f, 0, 0, 0};
  int32_t token;
  const bool use_topk = p.topk > 0 && p.topk < V;
  const bool use_mult = !use_topk && (p.topp <= 0.0f || p.topp >= 1.0f);

  if (S != S) {
    // Every probability is NaN.  The multinomial walk never fires and returns the last
    // index; top-p keeps no candidate and top-k's comparisons are all false, which the
    // reference does not define: report -1.
    token = use_mult ? V - 1 : -1;
  } else if (use_mult) {
    // ---- sampler.cpp:58-70
    const SeqSumResult res = seq_sum_block(prob_at, V, 0.0f, coin, sm);
    token = res.stop_index >= 0 ? res.stop_index : V - 1;
    dbg.cumulative = res.sum;
    dbg.position = token;
  } else {
    // ---- candidates: top-p keeps p >= (1 - topp) / (V - 1) (sampler.cpp:136-143); top-k
    // ranks the whole row (sampler.cpp:87-92)
    const float cutoff = use_topk ? 0.0f : (1.0f - p.topp) / static_cast<float>(V - 1);
    if (tid == 0) sm.counter = 0u;
    __syncthreads();
    for (int base = 0; base < V; base += kBlock) {
      const int i = base + tid;
      float pi = 0.0f;
      bool keep = false;
      if (i < V) {
        pi = prob_at(i);
        keep = pi >= cutoff;
      }
      const uint64_t mask = __ballot(keep);
      if (mask) {
        uint32_t slot0 = 0;
        const int leader = __ffsll(static_cast<long long>(mask)) - 1;
        if (lane == leader) slot0 = atomicAdd(&sm.counter, static_cast<uint32_t>(__popcll(mask)));
        slot0 = __shfl(slot0, leader);
        if (keep) {
          const uint32_t slot = slot0 + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
          scratch[slot] = cand_key(pi, i);
        }
      }
    }
    __syncthreads();
    const int n0 = static_cast<int>(sm.counter);
    dbg.n_candidates = n0;
    if (n0 == 0) {
      token = -1;  // the reference reads probindex[-1] here
    } else {
      const int N = pow2_ceil(n0);
      for (int i = n0 + tid; i < N; i += kBlock) scratch[i] = ~0ull;
      __syncthreads();
      sort_keys_block(scratch, N, lds_keys, p.lds_keys);
      const uint64_t* keys = scratch;
      if (N <= p.lds_keys) {  // the sorted tile is still in LDS
        keys = lds_keys;
      }
      auto sorted_prob = [&](int i) -> float { return cand_prob(keys[i]); };
      int last_idx;
      float mass;
      if (use_topk) {
        // ---- sampler.cpp:103-119: float accumulators over the k best
        last_idx = p.topk - 1;
        mass = seq_sum_block(sorted_prob, p.topk, 0.0f, kInf, sm).sum;
      } else {
        // ---- sampler.cpp:150-159: first position where the running mass exceeds topp
        const SeqSumResult res = seq_sum_block(sorted_prob, n0, 0.0f, p.topp, sm);
        last_idx = res.stop_index >= 0 ? res.stop_index : n0 - 1;
        mass = res.sum;
      }
      const float r = coin * mass;  // sampler.cpp:109 / :162
      const SeqSumResult walk = seq_sum_block(sorted_prob, last_idx + 1, 0.0f, r, sm);
      const int pos = walk.stop_index >= 0 ? walk.stop_index : last_idx;
      token = static_cast<int32_t>(static_cast<uint32_t>(keys[pos]));
      dbg.last_idx = last_idx;
      dbg.cumulative = mass;
      dbg.r = r;
      dbg.position = pos;
    }
  }
  if (tid == 0) {
    p.tokens[row] = token;
    if (p.debug) p.debug[row] = dbg;
  }
}

// Evaluates expf_exact over an array (test hook for the exhaustive comparison with libm).
__global__ void __launch_bounds__(256) expf_exact_kernel(const float* x, float* y, int64_t n) {
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = kExp2Table[threadIdx.x];
  __syncthreads();
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += 256ll * gridDim.x) y[i] = expf_exact(x[i], tab);
}

// Sequential float sum of an array by one workgroup (test hook for seq_sum_block).
__global__ void __launch_bounds__(kBlock)
seq_sum_kernel(const float* a, int32_t n, float s0, float threshold, float* sum_out, int32_t* stop_out) {
  __shared__ BlockScratch sm;
  auto fetch = [&](int i) -> float { return a[i]; };
  const SeqSumResult r = seq_sum_block(fetch, n, s0, threshold, sm);
  if (threadIdx.x == 0) {
    *sum_out = r.sum;
    *stop_out = r.stop_index;
  }
}

}  // namespace ets
