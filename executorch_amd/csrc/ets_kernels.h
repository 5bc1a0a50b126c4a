// gfx950 kernels of the token sampler.
//
//   argmax_*_kernel      temperature == 0 (Sampler::sample_argmax, sampler.cpp:44-56)
//   sample_rows_kernel   temperature != 0: scale, softmax, coin, top-k / multinomial / top-p
//                        (sampler.cpp:58-171, 189-251), one workgroup per row
//
// Everything that the reference computes with a sequential fp32 loop (the softmax sum, the
// nucleus mass, the CDF walks) goes through seq_sum_chunk(), so the results carry the same
// rounding as the scalar loops they replace.
#pragma once

#include <type_traits>

#include "ets_device.h"

namespace ets {

struct RowDebug {  // layout of ets_row_debug in include/et_sampler.h
  float max_val, sum, coin, cumulative, r;
  int32_t n_candidates, last_idx, position;
};

// Sampling parameters of one row when they differ from row to row (the batched counterpart of
// SamplingConfig, extension/llm/runner/llm_session.h:29-34, already resolved by the host).
struct RowConfig {
  float inv_temperature;
  float topp;
  int32_t topk;
};

// Logit processors that touch every entry of a row the same way (logit_processor.h:19-40: a bias, a
// factor), applied to each logit as it is read instead of by a pass of their own over the tensor.
// After each of them the value is rounded to the tensor's element type, as the processor's store
// into the tensor would.
constexpr int kMaxFusedOps = 4;
struct FusedOps {
  int32_t n;
  int32_t scale[kMaxFusedOps];  // 1: multiply by value, 0: add value
  float value[kMaxFusedOps];
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
  uint64_t* scratch;  // [batch, scratch_stride] candidate keys (rows that overflow LDS)
  int64_t scratch_stride;
  int32_t lds_keys;   // power of two: keys that fit in the dynamic LDS buffer
  const int32_t* row_map;    // workgroup -> row, or null for the identity
  const RowConfig* row_cfg;  // [batch] per-row parameters (by row), or null for the launch-wide ones
  FusedOps fused;            // logit processors applied as the logits are read (several-workgroups-per-row path only)
  // One workgroup per row, but no more workgroups than the launch's grid: a workgroup that is done
  // with a row takes the next one from `ticket` (0 before and after every launch), and the row's
  // scratch is the workgroup's, not the row's.
  int32_t rows;
  uint32_t* ticket;
  int32_t grid_cap;  // (host side only: the most workgroups the launch may have, i.e. scratch rows behind `scratch`)
};

// Rows beyond the launch's workgroups are handed out by `ticket`: a workgroup asks for its next row
// when it starts on one (the answer has arrived long before the row is done) and picks it up with
// take_row().  Rows 0 .. gridDim.x - 1 are the workgroups' first ones, asked for by nobody; every
// row a workgroup works on costs one request, so the launch makes p.rows of them, and whoever makes
// the last one puts the counter back to 0 for the next launch.  A launch with a workgroup per row
// touches no counter.
// (`units`: what is handed out, when it is not single rows)
__device__ __forceinline__ void request_row(const RowParams& p, int* lds_slot, int units) {
  if (static_cast<int>(gridDim.x) < units && threadIdx.x == 0) {
    const uint32_t t = atomicAdd(p.ticket, 1u);
    if (t + 1u == static_cast<uint32_t>(units)) atomicExch(p.ticket, 0u);
    *lds_slot = static_cast<int>(gridDim.x + t);
  }
}
__device__ __forceinline__ int take_row(const RowParams& p, const int* lds_slot, int units) {
  if (static_cast<int>(gridDim.x) >= units) return units;
  __syncthreads();
  const int next = *lds_slot;
  __syncthreads();
  return next;
}
__device__ __forceinline__ void request_row(const RowParams& p, int* lds_slot) { request_row(p, lds_slot, p.rows); }
__device__ __forceinline__ int take_row(const RowParams& p, const int* lds_slot) { return take_row(p, lds_slot, p.rows); }

// A float rounded to the row's element type and back (round to nearest even; a NaN stays a NaN).
template <int DT>
__device__ __forceinline__ float round_to_elem(float v) {
  if constexpr (DT == kDtypeBFloat16) {
    const uint32_t b = __float_as_uint(v);
    return __uint_as_float((b + 0x7fffu + ((b >> 16) & 1u)) & 0xffff0000u);  // (NaNs made from 16-bit values keep clear low bits)
  } else if constexpr (DT == kDtypeHalf) {
    asm volatile("" : "+v"(v));  // round to fp32 first, to half second: no single mixed-precision rounding
    return static_cast<float>(static_cast<_Float16>(v));
  } else {
    return v;
  }
}

// Two floats rounded to bf16 and back by the conversion instruction (one for the pair).
typedef __bf16 ets_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ets_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void round_pair_bf16(float& a, float& b) {
  const ets_f32x2 v = {a, b};
  const uint32_t u = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ets_bf16x2));
  a = __uint_as_float(u << 16);
  b = __uint_as_float(u & 0xffff0000u);
}

// The fused logit processors on R values at once.
template <int DT, int R>
__device__ __forceinline__ void apply_fused(float* x, const FusedOps& f) {
  for (int k = 0; k < f.n; ++k) {
    const float v = f.value[k];
    if (f.scale[k]) {
#pragma unroll
      for (int e = 0; e < R; ++e) x[e] = x[e] * v;
    } else {
#pragma unroll
      for (int e = 0; e < R; ++e) x[e] = x[e] + v;
    }
    if constexpr (DT == kDtypeBFloat16 && R % 2 == 0) {
#pragma unroll
      for (int e = 0; e < R; e += 2) round_pair_bf16(x[e], x[e + 1]);
    } else {
#pragma unroll
      for (int e = 0; e < R; ++e) x[e] = round_to_elem<DT>(x[e]);
    }
  }
}

// One logit of the row, processors applied; a NaN comes out as the canonical one a store into the
// tensor would leave.
template <int DT>
__device__ __forceinline__ float load_logit(const char* logits, int64_t i, const FusedOps& f) {
  float x = load_elem<DT>(logits, i);
  if (f.n > 0) {
    apply_fused<DT, 1>(&x, f);
    if (DT == kDtypeBFloat16 && x != x) x = __uint_as_float(0x7fc00000u);
  }
  return x;
}

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

// The arg-max and the Gumbel-max draw are two launches each: a partial kernel, grid = (splits,
// rows), in which every workgroup reduces one segment of a row to one 64-bit (key, ~index)
// maximum, and a finish kernel, one wave per row, that combines the row's partial results.  The
// kernel boundary orders the two; a single kernel with a device-scope fence per workgroup costs
// several times more on a part whose L2 is split over 8 dies.
__device__ __forceinline__ uint64_t pack_best(uint32_t key, int index) {
  // ties go to the lower index: larger (0xffffffff - index)
  return (static_cast<uint64_t>(key) << 32) | (0xffffffffu - static_cast<uint32_t>(index));
}

__device__ __forceinline__ void store_block_best(uint64_t best, uint64_t* slot) {
  __shared__ uint64_t red[kArgmaxBlock / 64];
  best = wave_max_u64(best);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxBlock / 64; ++w) best = red[w] > best ? red[w] : best;
    *slot = best;
  }
}

// ALIGNED: the row's base and pitch are multiples of 16 bytes (128-bit loads).
template <int DT, bool ALIGNED>
__global__ void __launch_bounds__(kArgmaxBlock)
argmax_partial_kernel(const void* logits_all, int64_t row_stride, int32_t vocab, uint64_t* partials,
                      const int32_t* row_map) {
  constexpr int VE = VecElems<DT>::value;
  const int row = row_map ? row_map[blockIdx.y] : blockIdx.y;
  const int splits = gridDim.x;
  const int tid = threadIdx.x;
  const char* logits = static_cast<const char*>(logits_all) + static_cast<int64_t>(row) * row_stride * ElemSize<DT>::value;
  uint64_t best = 0;
  auto visit = [&](float value, uint32_t raw16, int index) {
    const uint32_t key = DT == kDtypeUInt16 ? raw16 + 1u : order_key(value);
    const uint64_t packed = pack_best(key, index);
    best = packed > best ? packed : best;
  };
  int scalar_lo = 0, scalar_hi = vocab;  // entries left to the scalar loop
  if (ALIGNED && DT != kDtypeUInt16) {
    const int nvec = vocab / VE;
    const int seg = (nvec + splits - 1) / splits;
    const int lo = blockIdx.x * seg, hi = min(nvec, lo + seg);
    const uint4* vec = reinterpret_cast<const uint4*>(logits);
    for (int j = lo + tid; j < hi; j += 4 * kArgmaxBlock) {  // four loads in flight; extra ones re-read vec[j]
      uint4 r[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int jk = j + k * kArgmaxBlock;
        r[k] = vec[jk < hi ? jk : j];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int jk = j + k * kArgmaxBlock;
        if (jk < hi) {
          float v[VE];
          decode_vec<DT>(r[k], v);
#pragma unroll
          for (int e = 0; e < VE; ++e) visit(v[e], 0u, jk * VE + e);
        }
      }
    }
    // the last workgroup of the row also takes the entries behind the last full vector
    scalar_lo = blockIdx.x == splits - 1 ? nvec * VE : vocab;
  } else {
    const int seg = (vocab + splits - 1) / splits;
    scalar_lo = blockIdx.x * seg;
    scalar_hi = min(vocab, scalar_lo + seg);
  }
  for (int i = scalar_lo + tid; i < scalar_hi; i += kArgmaxBlock) {
    if (DT == kDtypeUInt16) {
      visit(0.0f, static_cast<uint32_t>(static_cast<const uint16_t*>(static_cast<const void*>(logits))[i]), i);
    } else {
      visit(load_elem<DT>(logits, i), 0u, i);
    }
  }
  store_block_best(best, &partials[static_cast<int64_t>(blockIdx.y) * splits + blockIdx.x]);
}

// grid = (rows), 64 lanes: lane l reads the row's l-th partial result (splits <= 64).
template <int DT>
__global__ void __launch_bounds__(64)
argmax_finish_kernel(const void* logits_all, int64_t row_stride, const uint64_t* partials, int32_t splits,
                     int32_t* tokens, const int32_t* row_map) {
  const int row = row_map ? row_map[blockIdx.x] : blockIdx.x;
  const int lane = threadIdx.x;
  uint64_t b = lane < splits ? partials[static_cast<int64_t>(blockIdx.x) * splits + lane] : 0ull;
  b = wave_max_u64(b);
  if (lane != 0) return;
  int32_t token = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(b));
  if (DT != kDtypeUInt16) {
    // `x > NaN` is never true: a NaN in slot 0 stays the maximum (sampler.cpp:47-50)
    const char* logits = static_cast<const char*>(logits_all) + static_cast<int64_t>(row) * row_stride * ElemSize<DT>::value;
    const float x0 = load_elem<DT>(logits, 0);
    if (x0 != x0) token = 0;
  }
  tokens[row] = token;
}

// ---- Gumbel-max draw -------------------------------------------------------------------------
// argmax_i(logit_i / T + g_i), g_i = -log(-log(u_i + 1e-20) + 1e-20), the in-graph sampler of
// examples/models/qwen3_5_moe/sampler.py:52-60: one pass over the row, no sequential dependency.
// u comes from `noise` ([batch, vocab] fp32, e.g. torch.rand_like(logits)) or, when that is
// null, from a counter-based generator keyed by the row's coin state and the entry's index; the
// finish kernel then advances the row's xorshift64* state by one step.
__device__ __forceinline__ float uniform_of(uint64_t state, uint32_t index) {
  // splitmix64 finaliser over (state, index); 24 random bits -> [0, 1)
  uint64_t z = state + (static_cast<uint64_t>(index) + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return static_cast<float>(static_cast<uint32_t>(z >> 40)) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ float gumbel_of(float u) { return -logf(-logf(u + 1e-20f) + 1e-20f); }

template <int DT>
__global__ void __launch_bounds__(kArgmaxBlock)
gumbel_partial_kernel(const void* logits_all, int64_t row_stride, int32_t vocab, float temperature,
                      const float* row_temperatures, const float* noise, const uint64_t* rng, uint64_t* partials) {
  const int row = blockIdx.y;
  const int splits = gridDim.x;
  const int tid = threadIdx.x;
  const char* logits = static_cast<const char*>(logits_all) + static_cast<int64_t>(row) * row_stride * ElemSize<DT>::value;
  // logits / temperature.clamp(min=1e-6)  (sampler.py:50)
  const RowDivisor div = row_divisor(__builtin_fmaxf(row_temperatures ? row_temperatures[row] : temperature, 1e-6f));
  const uint64_t state = rng[row];
  const float* u_row = noise ? noise + static_cast<int64_t>(row) * vocab : nullptr;
  const int seg = (vocab + splits - 1) / splits;
  const int lo = blockIdx.x * seg;
  const int hi = min(vocab, lo + seg);
  uint64_t best = 0;
  for (int i = lo + tid; i < hi; i += kArgmaxBlock) {
    const float x = div_row_signed(load_elem<DT>(logits, i), div);
    const float u = u_row ? u_row[i] : uniform_of(state, static_cast<uint32_t>(i));
    const uint64_t packed = pack_best(order_key(x + gumbel_of(u)), i);
    best = packed > best ? packed : best;
  }
  store_block_best(best, &partials[static_cast<int64_t>(row) * splits + blockIdx.x]);
}

static __global__ void __launch_bounds__(64)
gumbel_finish_kernel(const uint64_t* partials, int32_t splits, int32_t advance_rng, uint64_t* rng, int32_t* tokens) {
  const int row = blockIdx.x;
  const int lane = threadIdx.x;
  uint64_t b = lane < splits ? partials[static_cast<int64_t>(row) * splits + lane] : 0ull;
  b = wave_max_u64(b);
  if (lane != 0) return;
  tokens[row] = static_cast<int32_t>(0xffffffffu - static_cast<uint32_t>(b));
  if (advance_rng) {  // one step of the row's stream per call (sampler.cpp:210-214)
    uint64_t rs = rng[row];
    rs ^= rs >> 12;
    rs ^= rs << 25;
    rs ^= rs >> 27;
    rng[row] = rs;
  }
}

// Sort keys in LDS are addressed as LDS, never through a generic pointer: a helper that is left
// out of line would otherwise use flat loads and stores for them unless the compiler happens to
// see the same buffer at every call site.
typedef __attribute__((address_space(3))) uint64_t* LdsKeys;

// ---- sorting candidate keys -----------------------------------------------------------------
// Ascending sort of N keys (a power of two) that already sit in LDS (and are visible to the
// workgroup).  Bitonic network; every wave owns a contiguous run of W keys, and the sub-stages
// whose partners lie inside one run (distance < W) are done by that wave alone, without workgroup
// barriers (a fence that waits for the wave's own accesses separates them), so only the
// log2(N / W) long-distance sub-stages of each merge pay a barrier.  Ends with a barrier.
constexpr int kRankSort = 256;
__device__ void sort_keys_lds(LdsKeys lds, int N) {
  if (N <= kRankSort) {
    // A short list: every lane counts the keys below its own (all lanes read the same key at a
    // time, which LDS broadcasts) and stores its key at that rank.  The keys are distinct but for
    // the padding (~0) behind the last real key, which stays where it is.
    const int i = threadIdx.x;
    uint64_t key = ~0ull;
    int rank = i;
    if (i < N) {
      key = lds[i];
      if (key != ~0ull) {
        rank = 0;
        for (int j = 0; j < N; j += 2) {
          const uint64_t a = lds[j], b = lds[j + 1];
          rank += (a < key ? 1 : 0) + (b < key ? 1 : 0);
        }
      }
    }
    __syncthreads();
    if (i < N) lds[rank] = key;
    __syncthreads();
    return;
  }
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  int waves = N / 128;  // at least two keys per lane of a participating wave
  waves = waves < 1 ? 1 : (waves > kWaves ? kWaves : waves);
  const int W = N / waves;
  LdsKeys mine = lds + wave * W;
  for (int k = 2; k <= N; k <<= 1) {
    int j = k >> 1;
    for (; j >= W; j >>= 1) {
      for (int q = threadIdx.x; q < (N >> 1); q += kBlock) {
        const int i = ((q & ~(j - 1)) << 1) | (q & (j - 1));
        const int l = i | j;
        const bool up = (i & k) == 0;
        const uint64_t a = lds[i], b = lds[l];
        if ((a > b) == up) {
          lds[i] = b;
          lds[l] = a;
        }
      }
      __syncthreads();
    }
    if (wave < waves) {
      for (; j > 0; j >>= 1) {
        for (int q = lane; q < (W >> 1); q += 64) {
          const int i = ((q & ~(j - 1)) << 1) | (q & (j - 1));
          const int l = i | j;
          const bool up = ((wave * W + i) & k) == 0;
          const uint64_t a = mine[i], b = mine[l];
          if ((a > b) == up) {
            mine[i] = b;
            mine[l] = a;
          }
        }
        // other lanes of this wave read these keys next.  The stores must have been performed, not
        // merely issued: a workgroup-scope fence makes the wave wait for its outstanding LDS (and
        // flat) accesses, whichever instructions the compiler chose for the pointer, and the wave
        // barrier keeps the sub-stages apart in the instruction stream.
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
        __builtin_amdgcn_wave_barrier();
      }
    }
    if (k >= W) __syncthreads();  // the next merge starts with a long-distance sub-stage, or this was the last
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

// Wave-aggregated append: lanes with `keep` get consecutive slots from *counter.
__device__ __forceinline__ uint32_t wave_append_slot(bool keep, uint32_t* counter, int lane) {
  const uint64_t mask = __ballot(keep);
  uint32_t slot0 = 0;
  if (mask) {
    const int leader = __ffsll(static_cast<long long>(mask)) - 1;
    if (lane == leader) slot0 = atomicAdd(counter, static_cast<uint32_t>(__popcll(mask)));
    slot0 = __shfl(slot0, leader);
  }
  return slot0 + static_cast<uint32_t>(__popcll(mask & ((1ull << lane) - 1ull)));
}

// The CDF walk for short lists (n <= kSmallWalk; the nucleus of a peaked row is a handful of entries,
// and a workgroup-wide scan would spend its time in barriers): the first wave takes the
// probabilities sixty-four at a time, one per lane, and adds them in order with the single-wave
// scheme of the sequential sums (increments under the running sum's ulp; the lane in which the sum
// changes binade, meets a tie or crosses the threshold adds natively).
constexpr int kSmallWalk = 512;
template <typename Keys>
__device__ SeqSumResult seq_sum_small(Keys keys, int n, float threshold, BlockScratch& sm) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    float s = 0.0f;
    int found = -1;
    for (int base = 0; base < n && found < 0; base += 64) {
      const uint32_t bits[1] = {base + lane < n ? __float_as_uint(cand_prob(keys[base + lane])) : 0u};
      // (a sum that is still 0 behind the first group -- every probability 0 -- starts the next one like a row)
      wave_resolve<1>(s, found, bits, base + lane, n, threshold);
    }
    if (lane == 0) {
      sm.bc_sum = s;
      sm.bc_found = found;
    }
  }
  __syncthreads();
  const SeqSumResult r = {sm.bc_sum, sm.bc_found};
  __syncthreads();
  return r;
}

// The two CDF walks over candidates sorted by descending probability (sampler.cpp:150-170,
// :103-119 for top-k).  Returns the sorted position of the draw, or -2 when `n_sorted` entries
// were not enough to decide where the nucleus ends (top-p only, when more candidates exist).
template <typename Keys>
__device__ int draw_from_sorted(Keys keys, int n_sorted, int n_total, bool use_topk, int topk, float topp, float coin,
                                RowDebug& dbg, BlockScratch& sm) {
  const float kInf = __uint_as_float(0x7f800000u);
  auto sorted_prob = [&](int i) -> float { return cand_prob(keys[i]); };
  auto behind_prefix = [&](int i) -> float { return cand_prob(keys[i + kSmallWalk]); };
  int last_idx;
  float mass;
  if (use_topk) {
    last_idx = topk - 1;
    mass = (topk <= kSmallWalk) ? seq_sum_small(keys, topk, kInf, sm).sum
                                : seq_sum_block<4>(sorted_prob, topk, 0.0f, kInf, sm).sum;
  } else {
    // a short prefix usually holds the whole nucleus
    SeqSumResult res = {0.0f, -1};
    bool decided = false;
    if (n_sorted <= kSmallWalk) {
      res = seq_sum_small(keys, n_sorted, topp, sm);
      decided = true;
    } else {
      res = seq_sum_small(keys, kSmallWalk, topp, sm);
      decided = res.stop_index >= 0;
    }
    if (!decided) {  // on from where the prefix ended
      res = seq_sum_block<4>(behind_prefix, n_sorted - kSmallWalk, res.sum, topp, sm);
      if (res.stop_index >= 0) res.stop_index += kSmallWalk;
    }
    if (res.stop_index < 0 && n_sorted < n_total) return -2;
    last_idx = res.stop_index >= 0 ? res.stop_index : n_sorted - 1;
    mass = res.sum;
  }
  const float r = coin * mass;  // sampler.cpp:109 / :162
  // (the largest probabilities come first: the walk often ends among them)
  SeqSumResult walk = seq_sum_small(keys, last_idx + 1 < kSmallWalk ? last_idx + 1 : kSmallWalk, r, sm);
  if (walk.stop_index < 0 && last_idx + 1 > kSmallWalk) {
    walk = seq_sum_block<4>(behind_prefix, last_idx + 1 - kSmallWalk, walk.sum, r, sm);
    if (walk.stop_index >= 0) walk.stop_index += kSmallWalk;
  }
  const int pos = walk.stop_index >= 0 ? walk.stop_index : last_idx;
  dbg.last_idx = last_idx;
  dbg.cumulative = mass;
  dbg.r = r;
  dbg.position = pos;
  return pos;
}

// 32 bits filled with the storage pattern of +inf / -inf.
template <int DT>
struct InfPattern;
template <>
struct InfPattern<kDtypeFloat> {
  static constexpr uint32_t plus = 0x7f800000u, minus = 0xff800000u;
};
template <>
struct InfPattern<kDtypeHalf> {
  static constexpr uint32_t plus = 0x7c007c00u, minus = 0xfc00fc00u;
};
template <>
struct InfPattern<kDtypeBFloat16> {
  static constexpr uint32_t plus = 0x7f807f80u, minus = 0xff80ff80u;
};

// What one pass over the row accumulates.
//   kScanSum   e_i = expf(x_i - max), sequential sum; optionally lists top-p candidates
//   kScanWalk  p_i = e_i / S, sequential sum until it exceeds the coin (multinomial draw)
//   kScanWalkCached  the same walk over a row of fp32 e_i that a kScanSum pass kept (keep_e)
constexpr int kScanSum = 0, kScanWalk = 1, kScanWalkCached = 2;

struct ScanArgs {
  const char* logits;
  int V;
  float inv;
  float m;          // row maximum of x
  RowDivisor div;   // kScanWalk: the normaliser S and its reciprocal
  float threshold;  // kScanWalk: the coin; kScanSum: +inf
  float cutoff;     // kScanSum with listing: the reference's top-p cutoff
  uint64_t* list;   // kScanSum with listing: (exp bits << 32 | index) of possible candidates;
                    //   entry j lives in lds_list[j] while j < lds_list_cap, else in list[j]
  float* lut;       // bf16 rows: table of expf(x - max) by logit bit pattern (see build_exp_lut)
  int lut_base1;    //   (first live magnitude) - 1
  int lut_top;      //   index of the "beyond" slot inside one sign half
  int lut_half;     //   entries per sign half
  uint64_t* lds_list;
  int lds_list_cap;
  float list_floor;  // kListAppend with FLOOR (top-k rows): entries with exp below this are not listed
  float* keep_e;     // kScanSum without a table: where to keep every e_i (global memory, V floats), or null
};

constexpr int kLutCountWords = 12288;  // a table entry's counter sits 48 KiB above its e

// ---- expf by table for bf16 rows ----------------------------------------------------------------
// A bf16 logit has 65536 possible bit patterns and e = expf(fl(fl(l * inv) - max)) is a function of
// the pattern alone, so a row needs one exact expf per DISTINCT relevant pattern, not per entry.
// Relevant magnitudes span a few dozen binades: below them |l * inv| is under an eighth of an ulp of
// max, so x - max rounds to -max ("tiny" slot); above them a negative logit gives x - max < -104
// (e == 0, "beyond" slot) and a positive one would exceed the maximum (cannot occur).  Layout per
// sign half: [0] tiny, [1 .. R] live patterns in increasing magnitude, [R + 1] beyond.  Every entry
// also has a counter (zeroed here), kLutCountWords words above its e, that the top-p scan uses as
// a histogram of the row over the table's entries; e and the counters are separate arrays so that
// the look-ups of e spread over all LDS banks.
// Returns false (no table; the caller evaluates expf per entry) when inv or max are not positive
// finite in the way the bounds need, or when the table would not fit in `cap` floats.
// COUNTERS = false builds the table alone (`cap` then only has to hold its 2 * half floats).
// The threads from `first_thread` on share the entries; the ones before it only learn where the table lies.
// `seen`, when given, is a byte per eight consecutive 16-bit patterns (8192 bytes): only the entries of
// patterns whose byte is set are worked out (and the two ends, which stand for many patterns); the others
// are left as they are, for a caller that will only look up patterns it has marked.
template <bool COUNTERS = true>
__device__ bool build_exp_lut(float* lut, int cap, float inv, float m, const uint64_t* tab, int& base1, int& top,
                              int& half, int first_thread = 0, const uint8_t* seen = nullptr) {
  const float kInf = __uint_as_float(0x7f800000u);
  if (!(inv > 0.0f && inv < kInf && m > -kInf && m < kInf)) return false;
  const uint32_t ib = __float_as_uint(inv);
  const int ei = static_cast<int>(ib >> 23);  // biased exponent of inv: 2^(ei-127) <= inv < 2^(ei-126)
  if (ei == 0) return false;
  const uint32_t mb = __float_as_uint(__builtin_fabsf(m));
  const int em = (mb >> 23) ? static_cast<int>(mb >> 23) : 1;  // ulp(max) = 2^(em - 150)
  // tiny: |l| < 2^(E+1-127) and inv < 2^(ei-126) give |l * inv| < 2^(E + ei - 252), to stay below
  // ulp(max) / 8 = 2^(em - 153)
  int e_lo = em - ei + 100;  // first live binade (biased exponent of the logit)
  if (e_lo < 0) e_lo = 0;
  // beyond: |l| >= 2^(E-127) and inv >= 2^(ei-127) give |l * inv| >= 2^(E + ei - 254), to reach
  // |max| + 104 < 2^(et - 126) with et the biased exponent of (|max| + 104)
  const int et = static_cast<int>(__float_as_uint(__builtin_fabsf(m) + 104.0f) >> 23);
  int e_hi = et - ei + 128;  // last live binade
  if (e_hi > 254) e_hi = 254;
  if (e_hi < e_lo) return false;
  const int R = (e_hi - e_lo + 1) * 128;
  half = R + 2;
  top = R + 1;
  base1 = (e_lo << 7) - 1;
  if (2 * half > kLutCountWords || (COUNTERS ? kLutCountWords + 2 * half : 2 * half) > cap) return false;
  const int idx0 = static_cast<int>(threadIdx.x) - first_thread;
  for (int idx = idx0 < 0 ? 2 * half : idx0; idx < 2 * half; idx += kBlock - first_thread) {
    const int sgn = idx >= half ? 1 : 0;
    const int c = idx - sgn * half;
    float e;
    if (c == top) {
      e = sgn ? 0.0f : 1.0f;  // the positive one cannot occur; 1 keeps e falling along the table's logit order
    } else {
      float d;
      if (c == 0) {
        d = -m;
      } else {
        const uint32_t pattern = (static_cast<uint32_t>(sgn) << 15) | static_cast<uint32_t>(base1 + c);
        if (seen != nullptr && seen[pattern >> 3] == 0) continue;
        const float l = __uint_as_float(pattern << 16);
        d = l * inv - m;
      }
      d = __builtin_fminf(__builtin_fmaxf(d, -104.0f), 0.0f);  // positive only for patterns that cannot occur
      e = expf_core(d, tab);
    }
    lut[idx] = e;
    if (COUNTERS) lut[kLutCountWords + idx] = 0.0f;  // bit pattern of the integer 0
  }
  return true;
}

// The same table for a caller that has marked the patterns it will look up (`seen`: a byte per eight
// consecutive 16-bit patterns, 8192 bytes, 8-byte aligned) and builds with the waves from the second on:
// the table is cut into chunks of 64 consecutive patterns; every wave finds out which chunks hold a marked
// pattern (three reads of eight mark bytes per lane, three ballots: a table that fits has at most 192
// chunks) and the builders take those chunks in turn, so that each has the same number of them to work out,
// whatever the row looks like.  Unmarked chunks are left as they are.
__device__ bool build_exp_lut_marked(float* lut, int cap, float inv, float m, const uint64_t* tab, int& base1, int& top,
                                     int& half, const uint8_t* seen) {
  const float kInf = __uint_as_float(0x7f800000u);
  if (!(inv > 0.0f && inv < kInf && m > -kInf && m < kInf)) return false;
  const int ei = static_cast<int>(__float_as_uint(inv) >> 23);
  if (ei == 0) return false;
  const uint32_t mb = __float_as_uint(__builtin_fabsf(m));
  const int em = (mb >> 23) ? static_cast<int>(mb >> 23) : 1;
  int e_lo = em - ei + 100;  // (the bounds of build_exp_lut)
  if (e_lo < 0) e_lo = 0;
  const int et = static_cast<int>(__float_as_uint(__builtin_fabsf(m) + 104.0f) >> 23);
  int e_hi = et - ei + 128;
  if (e_hi > 254) e_hi = 254;
  if (e_hi < e_lo) return false;
  const int R = (e_hi - e_lo + 1) * 128;
  const int per_half = R >> 6, n_chunks = 2 * per_half;
  half = R + 2;
  top = R + 1;
  base1 = (e_lo << 7) - 1;
  if (2 * half > kLutCountWords || 2 * half > cap) return false;
  static_assert(kLutCountWords <= 192 * 64, "three ballots cover the chunks of a table that fits");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave == 0) return true;  // (takes no part: where the table lies)
  const int builders = kBlock / 64 - 1, me = wave - 1;
  auto first_pattern = [&](int k) -> uint32_t {
    const int sgn = k >= per_half ? 1 : 0;
    return (static_cast<uint32_t>(sgn) << 15) | static_cast<uint32_t>((e_lo << 7) + 64 * (k - sgn * per_half));
  };
  auto marked = [&](int k) -> bool {
    return k < n_chunks && *reinterpret_cast<const uint64_t*>(seen + (first_pattern(k) >> 3)) != 0ull;
  };
  const uint64_t need0 = __ballot(marked(lane)), need1 = __ballot(marked(lane + 64)), need2 = __ballot(marked(lane + 128));
  const uint64_t below = (1ull << lane) - 1ull;
  const int rank0 = __popcll(need0 & below), rank1 = __popcll(need0) + __popcll(need1 & below),
            rank2 = __popcll(need0) + __popcll(need1) + __popcll(need2 & below);
  uint64_t mine[3] = {__ballot(((need0 >> lane) & 1ull) && rank0 % builders == me),
                      __ballot(((need1 >> lane) & 1ull) && rank1 % builders == me),
                      __ballot(((need2 >> lane) & 1ull) && rank2 % builders == me)};
#pragma unroll
  for (int h = 0; h < 3; ++h) {
    while (mine[h] != 0ull) {
      const int k = 64 * h + __builtin_ctzll(mine[h]);
      mine[h] &= mine[h] - 1ull;
      const uint32_t pattern = first_pattern(k) + static_cast<uint32_t>(lane);
      const int sgn = static_cast<int>(pattern >> 15);
      const int c = static_cast<int>(pattern & 0x7fffu) - base1;
      const float l = __uint_as_float(pattern << 16);
      const float d = __builtin_fminf(__builtin_fmaxf(l * inv - m, -104.0f), 0.0f);  // positive only for patterns that cannot occur
      lut[sgn * half + c] = expf_core(d, tab);
    }
  }
  if (wave == 1 && lane < 4) {  // the two ends of each half: the patterns below and beyond the table's
    const int sgn = lane >> 1;
    const bool beyond = (lane & 1) != 0;
    const float tiny = expf_core(__builtin_fminf(__builtin_fmaxf(-m, -104.0f), 0.0f), tab);
    lut[sgn * half + (beyond ? top : 0)] = beyond ? (sgn ? 0.0f : 1.0f) : tiny;
  }
  return true;
}

// Table slot of one bf16 pattern (16 bits: sign, 8 exponent bits, 7 mantissa bits).
__device__ __forceinline__ int lut_slot(uint32_t mag15, uint32_t sgn, int base1, int top, int half) {
  const int c = min(max(static_cast<int>(mag15), base1), base1 + top);
  return static_cast<int>(__umul24(sgn, static_cast<uint32_t>(half))) + c - base1;
}

// The same as the LDS byte address of the entry's e (4 bytes per entry), in three instructions:
// clamp, sign * half + bias, shift-add.  lo = base1, hi = base1 + top, half4 = 4 * half,
// bias = (LDS address of the table) - 4 * base1 (mod 2^32), all loop-invariant.
typedef __attribute__((address_space(3))) float* LdsF32;
typedef __attribute__((address_space(3))) uint32_t* LdsU32;
struct LutAddr {
  int lo, hi;
  uint32_t half4, bias;
};
__device__ __forceinline__ LutAddr lut_addr_of(float* lut, int base1, int top, int half) {
  const uint32_t table = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsF32)lut));
  return {base1, base1 + top, static_cast<uint32_t>(half) * 4u, table - static_cast<uint32_t>(base1) * 4u};
}
__device__ __forceinline__ uint32_t lut_entry_address(uint32_t mag15, uint32_t sgn, const LutAddr& t) {
  int c;
  uint32_t side, addr;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(c) : "v"(mag15), "v"(t.lo), "v"(t.hi));
  asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(side) : "v"(sgn), "v"(t.half4), "v"(t.bias));
  asm("v_lshl_add_u32 %0, %1, 2, %2" : "=v"(addr) : "v"(c), "v"(side));
  return addr;
}

constexpr int kGroup = 2;  // 16-byte vectors per lane between two barriers of the main loop

// What a kScanSum pass records for the top-p draw.
//   kListNone    nothing
//   kListAppend  entries whose exp could still reach the cutoff once the normaliser is known
//                (exp >= cutoff * max(1, running sum), with slack) are appended to the candidate
//                list and counted in sm.counter
//   kListHist    (table rows) entries that pass the same test add one to their table entry's
//                counter
constexpr int kListNone = 0, kListAppend = 1, kListHist = 2;

// Smallest exp a listing pass records while the running sum is s.
template <int LIST, bool FLOOR>
__device__ __forceinline__ float list_cut(const ScanArgs& a, float s) {
  if (LIST == kListNone) return 0.0f;
  if (FLOOR) return a.list_floor;  // top-k rows: the cutoff is 0
  return a.cutoff * __builtin_fmaxf(s, 1.0f) * 0.999f;
}

// One pass over the row in index order.  The main loop handles kGroup * kBlock full vectors per
// iteration without bounds checks (loads for the next iteration are issued before the current one
// is processed); the remainder goes through a bounds-checked loop.  Returns true if the threshold
// was crossed.
template <int DT, bool ALIGNED, int MODE, int LIST, bool LUT, bool FLOOR = false>
__device__ __forceinline__ bool scan_row(const ScanArgs& a, SeqSum& st, BlockScratch& sm) {
  static_assert(!LUT || DT == kDtypeBFloat16, "the expf table is indexed by bf16 bit patterns");
  static_assert(LIST != kListHist || LUT, "the histogram lives in the expf table");
  constexpr int VE = VecElems<DT>::value;
  const int tid = threadIdx.x;
  const int V = a.V;
  const float inv = a.inv, m = a.m;
  const uint64_t* tab = sm.exp2tab;
  int done_elems = 0;
  auto value_of = [&](float l) -> float {
    if (MODE == kScanWalkCached) return div_row(l, a.div);  // l is e_i
    const float x = l * inv;
    float d = x - m;
    d = __builtin_fmaxf(d, -104.0f);  // expf is 0 below ln(2^-150); the core gives 0 at -104 too
    const float e = expf_core(d, tab);
    return MODE == kScanWalk ? div_row(e, a.div) : e;  // sampler.cpp:205-207: a true division
  };
  // table rows: e of one bf16 pattern (and the histogram update)
  const LutAddr lut_addr = lut_addr_of(a.lut, a.lut_base1, a.lut_top, a.lut_half);
  auto table_count = [&](uint32_t entry_address, float e, float cut_lo) {
    if (LIST == kListHist && e >= cut_lo) {
      __hip_atomic_fetch_add((LdsU32)static_cast<uintptr_t>(entry_address + 4u * kLutCountWords), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
  };
  auto table_value = [&](uint32_t mag15, uint32_t sgn, float cut_lo) -> float {
    const uint32_t address = lut_entry_address(mag15, sgn, lut_addr);
    const float e = *(LdsF32)static_cast<uintptr_t>(address);
    table_count(address, e, cut_lo);
    return e;  // a walk's table already holds the probabilities
  };
  auto append = [&](uint32_t e_bits, int index) {
    const uint32_t slot = atomicAdd(&sm.counter, 1u);
    const uint64_t ent = (static_cast<uint64_t>(e_bits) << 32) | static_cast<uint32_t>(index);
    if (slot < static_cast<uint32_t>(a.lds_list_cap)) {
      a.lds_list[slot] = ent;
    } else {
      a.list[slot] = ent;
    }
  };
  if (ALIGNED && V >= VE) {  // (a row shorter than one vector has no vector to prefetch)
    const int nvec = V / VE;
    const uint4* vec = reinterpret_cast<const uint4*>(a.logits);
    constexpr int per_iter = kBlock * kGroup;
    // The last group of a row may be partial.  Its missing vectors are replaced by logits of
    // -inf * sign(inv): x = -inf, whose exp is 0 on every path, so they add nothing.
    const uint32_t filler1 = MODE == kScanWalkCached ? 0u : (inv < 0.0f ? InfPattern<DT>::plus : InfPattern<DT>::minus);
    const uint4 filler = {filler1, filler1, filler1, filler1};
    uint4 raw[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) raw[u] = vec[min(u * kBlock + tid, nvec - 1)];
    for (int vbase = 0; vbase < nvec; vbase += per_iter) {
      if (vbase + per_iter > nvec) {
#pragma unroll
        for (int u = 0; u < kGroup; ++u) {
          if (vbase + u * kBlock + tid >= nvec) raw[u] = filler;
        }
      }
      const float scale = fast_scale(st.s);
      const float cut_lo = list_cut<LIST, FLOOR>(a, st.s);
      FastAcc acc[kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) acc[u] = {0.0f, 0.0f};
      uint32_t bits[kGroup][VE];
      int first[kGroup];
      const bool more = vbase + per_iter < nvec;
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        float v[VE];
        if (LUT) {
          // all eight table reads are issued before the first use of one
          const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
          uint32_t address[VE];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            address[2 * k] = lut_entry_address(w[k] & 0x7fffu, (w[k] >> 15) & 1u, lut_addr);
            address[2 * k + 1] = lut_entry_address((w[k] >> 16) & 0x7fffu, w[k] >> 31, lut_addr);
          }
#pragma unroll
          for (int e = 0; e < VE; ++e) v[e] = *(LdsF32)static_cast<uintptr_t>(address[e]);
#pragma unroll
          for (int e = 0; e < VE; ++e) {
            table_count(address[e], v[e], cut_lo);  // (a walk's table already holds the probabilities)
          }
        } else {
          decode_vec<DT>(raw[u], v);
        }
        if (more) raw[u] = vec[min(vbase + per_iter + u * kBlock + tid, nvec - 1)];
        first[u] = (vbase + u * kBlock + tid) * VE;
        uint32_t cmask = 0;
#pragma unroll
        for (int e = 0; e < VE; ++e) {
          const float val = LUT ? v[e] : value_of(v[e]);
          bits[u][e] = __float_as_uint(val);
          fast_fold(acc[u], val, scale);
          if (LIST == kListAppend && val >= cut_lo) cmask |= 1u << e;
        }
        if (LIST == kListAppend) {
          while (cmask) {
            const int e = __ffs(static_cast<int>(cmask)) - 1;
            cmask &= cmask - 1u;
            uint32_t eb = bits[u][0];
#pragma unroll
            for (int q = 1; q < VE; ++q) eb = (e == q) ? bits[u][q] : eb;
            append(eb, first[u] + e);
          }
        }
        if (!LUT && MODE == kScanSum && a.keep_e != nullptr && vbase + u * kBlock + tid < nvec) {
          uint4* kept = reinterpret_cast<uint4*>(a.keep_e + first[u]);
#pragma unroll
          for (int q = 0; q < VE / 4; ++q) kept[q] = {bits[u][4 * q], bits[u][4 * q + 1], bits[u][4 * q + 2], bits[u][4 * q + 3]};
        }
      }
      if (seq_sum_group<kGroup, VE, MODE == kScanSum>(st, bits, acc, scale, first, V, a.threshold, sm)) return true;
    }
    done_elems = nvec * VE;
  }
  // remainder (and rows whose base or pitch is not 16-byte aligned)
  for (int base = done_elems; base < V; base += kBlock * VE) {
    const int first = base + tid * VE;
    const float cut_lo = list_cut<LIST, FLOOR>(a, st.s);
    uint32_t bits[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) {
      const int i = first + e;
      float val = 0.0f;
      if (i < V) {
        const float l = load_elem<DT>(a.logits, i);
        if (LUT) {
          const uint32_t pattern = __float_as_uint(l) >> 16;
          val = table_value(pattern & 0x7fffu, pattern >> 15, cut_lo);
        } else {
          val = value_of(l);
        }
        if (LIST == kListAppend && val >= cut_lo) append(__float_as_uint(val), i);
        if (!LUT && MODE == kScanSum && a.keep_e != nullptr) a.keep_e[i] = val;
      }
      bits[e] = __float_as_uint(val);
    }
    if (seq_sum_chunk<VE>(st, bits, first, V, a.threshold, sm)) return true;
  }
  return false;
}

// Stable radix sort of n entries by their upper 32 bits, least significant byte first, by one
// workgroup; `a` holds the entries, `b` is a second buffer of n entries (both global memory), `table`
// is LDS for 3 * kWaves * 256 words.  Every wave owns a contiguous chunk of the input: it counts its
// chunk's digits into its own row of the table, the rows become write positions (digit-major, then
// wave), and the wave moves its chunk 64 entries at a time -- lanes with equal digits find each
// other through a 64-bit word per digit in which each sets its bit, and take consecutive positions
// in lane order -- so equal digits keep their input
// order and the scatter needs no synchronisation between waves.  A byte that is the same in every
// entry costs only its counting pass.  Returns the buffer that holds the sorted entries.
__device__ uint64_t* radix_sort_block(uint64_t* a, uint64_t* b, int n, LdsU32 table, BlockScratch& sm) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int chunk = (((n + kWaves - 1) / kWaves) + 63) & ~63;
  const int c0 = min(n, wave * chunk), c1 = min(n, c0 + chunk);
  LdsU32 mine = table + wave * 256;
  LdsKeys board = (LdsKeys)(table + kWaves * 256) + wave * 256;
  for (int d = lane; d < 256; d += 64) board[d] = 0ull;  // left clear by every use
  for (int shift = 32; shift < 64; shift += 8) {
    // ---- count
    for (int d = lane; d < 256; d += 64) mine[d] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
    for (int base = c0; base < c1; base += 64 * 8) {  // eight loads in flight
      uint64_t entry[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int i = base + k * 64 + lane;
        entry[k] = a[i < c1 ? i : c0];
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (base + k * 64 + lane < c1) {
          const uint32_t digit = static_cast<uint32_t>(entry[k] >> shift) & 255u;
          __hip_atomic_fetch_add(&mine[digit], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
        }
      }
    }
    __syncthreads();
    // ---- positions: exclusive prefix over (digit, wave); lane t holds digit t / 4, waves 4 * (t % 4) ...
    const int digit0 = tid >> 2, wave0 = (tid & 3) * 4;
    uint32_t c[4];
    uint32_t sum = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      c[k] = table[(wave0 + k) * 256 + digit0];
      sum += c[k];
    }
    // digits are spread over groups of four lanes: a digit's total is the sum over its group
    uint32_t digit_total = sum + __shfl_xor(sum, 1);
    digit_total += __shfl_xor(digit_total, 2);
    const bool one_digit = __ballot(digit_total == static_cast<uint32_t>(n)) != 0ull;
    const float upto = wave_scan_inclusive_f32(static_cast<float>(sum), lane);  // exact: n is below 2^24
    if (lane == 63) sm.red_f[wave] = upto;
    if (lane == 0) sm.red_u[wave] = one_digit ? 1u : 0u;
    __syncthreads();
    float before = 0.0f;
    uint32_t any_one = 0u;
    for (int w = 0; w < kWaves; ++w) {
      if (w < wave) before += sm.red_f[w];
      any_one |= sm.red_u[w];
    }
    uint32_t start = static_cast<uint32_t>(before + upto) - sum;
    if (!any_one) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        table[(wave0 + k) * 256 + digit0] = start;
        start += c[k];
      }
    }
    __syncthreads();
    if (any_one) continue;  // every entry has the same byte here
    // ---- move
    for (int base4 = c0; base4 < c1; base4 += 64 * 4) {  // four loads in flight
      uint64_t entry4[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int i = base4 + k * 64 + lane;
        entry4[k] = a[i < c1 ? i : c0];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
      const int base = base4 + k * 64;
      if (base >= c1) break;
      const int i = base + lane;
      const bool valid = i < c1;
      const uint64_t entry = entry4[k];
      const uint32_t digit = static_cast<uint32_t>(entry >> shift) & 255u;
      // the lanes with this digit: every lane sets its bit in the digit's word, then reads the word
      if (valid) __hip_atomic_fetch_or(&board[digit], 1ull << lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");  // (waits for the wave's own LDS accesses)
      const uint64_t peers = valid ? board[digit] : 0ull;
      const uint32_t rank = static_cast<uint32_t>(__popcll(peers & ((1ull << lane) - 1ull)));
      uint32_t position = 0u;
      if (valid) {
        position = mine[digit];
        b[position + rank] = entry;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");  // every peer has read the position
      if (valid && rank == 0u) {
        mine[digit] = position + static_cast<uint32_t>(__popcll(peers));
        board[digit] = 0ull;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
      }
    }
    __syncthreads();
    uint64_t* t = a;
    a = b;
    b = t;
  }
  return a;
}

// General path: every candidate (top-p: p >= cutoff; top-k: the whole row, sampler.cpp:87-100)
// becomes a sort key and the full list is sorted: in LDS when it fits (bitonic network), otherwise
// by the radix sort above over the whole row in index order, with keys that sort last in place of
// the entries that are no candidates (a candidate's probability is positive in top-p, and in top-k
// every entry is one, so no candidate ties with them).  Used by large top-k and by top-p rows
// whose candidates do not fit in LDS.  `scratch` holds `scratch_cap` entries.
template <int DT>
__device__ int32_t draw_general(const char* logits, int V, float inv, float m, float S, bool use_topk,
                                             int topk, float topp, float cutoff, float coin, uint64_t* scratch,
                                             int64_t scratch_cap, uint64_t* lds_keys, int cap, RowDebug& dbg,
                                             BlockScratch& sm, const FusedOps* fused = nullptr) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const float cut = use_topk ? 0.0f : cutoff;
  const RowDivisor div = row_divisor(S);
  if (tid == 0) sm.counter = 0u;
  __syncthreads();
  uint32_t kept = 0u;
  for (int base = 0; base < V; base += kBlock) {
    const int i = base + tid;
    if (i < V) {
      const float x = (fused ? load_logit<DT>(logits, i, *fused) : load_elem<DT>(logits, i)) * inv;
      const float pi = div_row(expf_nonpositive(x - m, sm.exp2tab), div);
      const bool keep = pi >= cut;
      scratch[i] = keep ? cand_key(pi, i) : ~0ull;
      kept += keep ? 1u : 0u;
    }
  }
  kept = wave_sum_u32(kept);
  if (lane == 0 && kept != 0u) atomicAdd(&sm.counter, kept);
  __syncthreads();
  const int n0 = static_cast<int>(sm.counter);
  dbg.n_candidates = n0;
  if (n0 == 0) return -1;  // the reference reads probindex[-1] here
  const int N = pow2_ceil(n0);
  if (N <= cap) {
    __syncthreads();
    if (tid == 0) sm.counter = 0u;
    __syncthreads();
    for (int base = 0; base < V; base += kBlock) {
      const int i = base + tid;
      const uint64_t key = i < V ? scratch[i] : ~0ull;
      const bool keep = key != ~0ull;
      const uint32_t slot = wave_append_slot(keep, &sm.counter, lane);
      if (keep) lds_keys[slot] = key;
    }
    for (int i = n0 + tid; i < N; i += kBlock) lds_keys[i] = ~0ull;
    __syncthreads();
    sort_keys_lds((LdsKeys)lds_keys, N);
    // (keys in LDS are walked through an LDS-typed pointer, keys in global memory through a global
    // one: no generic pointer that could stand for either)
    const int pos = draw_from_sorted((LdsKeys)lds_keys, n0, n0, use_topk, topk, topp, coin, dbg, sm);
    return static_cast<int32_t>(static_cast<uint32_t>(lds_keys[pos]));
  }
  // the host sizes the scratch for two buffers of V entries and the key buffer for the sort's table
  const uint64_t* keys = radix_sort_block(scratch, scratch + scratch_cap / 2, V, (LdsU32)lds_keys, sm);
  const int pos = draw_from_sorted(keys, n0, n0, use_topk, topk, topp, coin, dbg, sm);
  return static_cast<int32_t>(static_cast<uint32_t>(keys[pos]));
}

// Workgroup sum of two floats per lane (DPP inside the wave, LDS across waves, one barrier).
__device__ __forceinline__ void block_sum2(float& x, float& y, BlockScratch& sm, uint32_t& buf) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  x = wave_sum_f32(x);
  y = wave_sum_f32(y);
  if (lane == 0) {
    sm.group_total[buf][wave] = x;
    sm.aux_total[buf][wave] = y;
  }
  __syncthreads();
  x = 0.0f;
  y = 0.0f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    x += sm.group_total[buf][w];
    y += sm.aux_total[buf][w];
  }
  buf ^= 1u;
}

// Sort and both CDF walks (sampler.cpp:150-170) for n <= 64 candidate keys at lds[0, n), done by
// the first wave in registers: rank by counting, ds_permute into place, then the two scalar loops
// with the probabilities read lane by lane.  Same contract as draw_from_sorted (returns the sorted
// position or -2) but `token` is returned directly, since the sorted keys never go back to LDS.
// With topk > 0 (n >= topk) the walks are top-k's (sampler.cpp:103-119): the mass of the first topk
// keys, no threshold.  `p_floor`: entries that are not among the keys may have probabilities up to
// p_floor; the last key walked must have a larger one for the prefix to be the reference's (else -2).
// The wave's part of draw_small_wave(): `key` is the lane's candidate key (all ones in lanes from n on).
// Returns the sorted position (-2: undecided) and, with it, the last index walked, the mass, r and the token.
__device__ __forceinline__ int small_wave_core(uint64_t key, int n, int n_total, float topp, float coin, int topk, float p_floor,
                                               int& last_idx_out, float& mass_out, float& r_out, uint32_t& token_out) {
  int rank = 0;
  const int lane = threadIdx.x & 63;
  const uint32_t key_hi = static_cast<uint32_t>(key >> 32), key_lo = static_cast<uint32_t>(key);
  for (int j = 0; j < n; ++j) {
    const uint64_t other = (static_cast<uint64_t>(readlane_u32(key_hi, j)) << 32) | readlane_u32(key_lo, j);
    rank += other < key ? 1 : 0;
  }
  if (lane >= n) rank = lane;  // padding stays where it is; ranks of real keys are < n
  const uint32_t hi = __builtin_amdgcn_ds_permute(rank * 4, static_cast<int>(key >> 32));
  const uint32_t lo = __builtin_amdgcn_ds_permute(rank * 4, static_cast<int>(static_cast<uint32_t>(key)));
  const float prob = __uint_as_float(0xffffffffu - hi);  // cand_prob
  float s = 0.0f;
  int found = -1;
  if (topk > 0) {
    for (int i = 0; i < topk; ++i) s = s + readlane_f32(prob, i);
    found = topk - 1;
  } else {
    for (int i = 0; i < n; ++i) {
      s = s + readlane_f32(prob, i);
      if (s > topp) {
        found = i;
        break;
      }
    }
  }
  int pos = -2;
  if ((found >= 0 || n == n_total) && readlane_f32(prob, found >= 0 ? found : n - 1) > p_floor) {
    const int last_idx = found >= 0 ? found : n - 1;
    const float r = coin * s;  // sampler.cpp:162
    float c = 0.0f;
    pos = last_idx;
    for (int i = 0; i <= last_idx; ++i) {
      c = c + readlane_f32(prob, i);
      if (c > r) {
        pos = i;
        break;
      }
    }
    last_idx_out = last_idx;
    mass_out = s;
    r_out = r;
    token_out = readlane_u32(lo, pos);
  }
  return pos;
}

__device__ int draw_small_wave(LdsKeys lds, int n, int n_total, float topp, float coin, RowDebug& dbg,
                               int32_t& token, BlockScratch& sm, int topk = 0, float p_floor = -1.0f) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    const uint64_t key = lane < n ? lds[lane] : ~0ull;
    int last_idx = 0;
    float mass = 0.0f, r = 0.0f;
    uint32_t tok = 0u;
    const int pos = small_wave_core(key, n, n_total, topp, coin, topk, p_floor, last_idx, mass, r, tok);
    if (lane == 0) {
      if (pos != -2) {
        sm.flag = last_idx;
        sm.bc_sum = mass;
        sm.red_f[1] = r;
        sm.counter = tok;
      }
      sm.bc_found = pos;
    }
  }
  __syncthreads();
  const int pos = sm.bc_found;
  if (pos != -2) {
    dbg.last_idx = sm.flag;
    dbg.cumulative = sm.bc_sum;
    dbg.r = sm.red_f[1];
    dbg.position = pos;
    token = static_cast<int32_t>(sm.counter);
  }
  __syncthreads();
  return pos;
}

// Ascending sort of n distinct candidate keys in LDS by buckets: the keys go into 2048 buckets by
// the size of their probability (64 per binade below the largest one, like the histogram of the
// candidates; one counting pass, one scan, one scatter into `work`), then every key counts the keys
// of its own bucket that are below it (its neighbours read the same keys, which LDS broadcasts) and
// goes back to `keys` at that rank.  A few passes over the keys instead of the bitonic network's
// log2(N)^2 / 2, as long as no bucket is long: a nucleus of 4234 fp32 probabilities has about ten
// keys to a bucket.  `work`: room for n keys and, behind them, 4096 32-bit words.
// Returns false, with `keys` as they were, when a bucket holds more than kBucketMax keys (many equal
// probabilities: the caller sorts by the network).  Ends with a barrier.
constexpr int kSortBuckets = 2048;
constexpr int kBucketMax = 192;
__device__ bool sort_keys_bucketed(LdsKeys keys, int n, LdsKeys work, BlockScratch& sm) {
  static_assert(kSortBuckets == 2 * kBlock, "two buckets per lane");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  LdsU32 cursor = (LdsU32)(work + n);
  LdsU32 start = cursor + kSortBuckets;
  cursor[2 * tid] = 0u;
  cursor[2 * tid + 1] = 0u;
  // the largest probability has the smallest key
  uint32_t top = 0u;
  for (int i = tid; i < n; i += kBlock) {
    const uint32_t inv = ~static_cast<uint32_t>(keys[i] >> 32);
    top = inv > top ? inv : top;
  }
  top = wave_max_u32(top);
  if (lane == 0) sm.red_u[wave] = top;
  __syncthreads();
  top = sm.red_u[0];
  for (int w = 1; w < kWaves; ++w) top = sm.red_u[w] > top ? sm.red_u[w] : top;
  const uint32_t hi_min = ~top;
  auto bucket_of = [&](uint64_t key) -> uint32_t {
    const uint32_t b = (static_cast<uint32_t>(key >> 32) - hi_min) >> 17;
    return b < static_cast<uint32_t>(kSortBuckets - 1) ? b : static_cast<uint32_t>(kSortBuckets - 1);
  };
  for (int i = tid; i < n; i += kBlock)
    __hip_atomic_fetch_add(&cursor[bucket_of(keys[i])], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __syncthreads();
  const uint32_t c0 = cursor[2 * tid], c1 = cursor[2 * tid + 1];
  const uint32_t incl = wave_scan_inclusive_u32(c0 + c1);
  const uint32_t longest = wave_max_u32(c0 > c1 ? c0 : c1);
  __syncthreads();  // (red_u has been read by everybody)
  if (lane == 63) sm.red_u[wave] = incl;
  if (lane == 0) sm.red_f[wave] = __uint_as_float(longest);
  __syncthreads();
  uint32_t before = incl - (c0 + c1), worst = 0u;
  for (int w = 0; w < kWaves; ++w) {
    if (w < wave) before += sm.red_u[w];
    const uint32_t l = __float_as_uint(sm.red_f[w]);
    worst = l > worst ? l : worst;
  }
  __syncthreads();  // (red_u and red_f are free again)
  if (worst > static_cast<uint32_t>(kBucketMax)) return false;
  start[2 * tid] = before;
  start[2 * tid + 1] = before + c0;
  cursor[2 * tid] = before;
  cursor[2 * tid + 1] = before + c0;
  __syncthreads();
  for (int i = tid; i < n; i += kBlock) {
    const uint64_t key = keys[i];
    work[__hip_atomic_fetch_add(&cursor[bucket_of(key)], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)] = key;
  }
  __syncthreads();  // cursor[b] is now the end of bucket b
  for (int i = tid; i < n; i += kBlock) {
    const uint64_t key = work[i];
    const uint32_t b = bucket_of(key);
    const int first = static_cast<int>(start[b]), end = static_cast<int>(cursor[b]);
    int rank = first;
    for (int j = first; j < end; ++j) rank += work[j] < key ? 1 : 0;
    keys[rank] = key;
  }
  __syncthreads();
  return true;
}

// Top-p draw from the listed possible candidates (sampler.cpp:122-171).  Entry j of the list sits
// in lds_list[j] while j < lds_list_cap and in list[j] (global memory) beyond; lds_list is the
// upper part of the key buffer lds_keys[0, cap), starting at key index `list_base`.
//   A. exact filter p = fl(e / S) >= cutoff (sampler.cpp:137-143); the list is rewritten in place
//      as (p_bits << 32 | index), 0 for dropped entries;
//   B. a probability threshold tau = p_max / 4^k is lowered until the entries above it carry
//      safely more than topp (any-order float sums with a 0.4 % margin): the nucleus is among them;
//   C. only those entries are sorted (in LDS) and the reference's two CDF walks run over them.
// Returns false when the entries to sort do not fit in LDS or, against expectation, do not reach
// topp (the caller takes the general path).  more_exist: the list is the row's largest entries,
// not every candidate.  tau_hint: a threshold the caller expects to do for B (0: none).
__device__ bool draw_topp_listed(uint64_t* list, uint64_t* lds_list, int lds_list_cap, int list_base, int n_listed,
                                 float S, float cutoff, float topp, float coin, uint64_t* lds_keys, int cap,
                                 RowDebug& dbg, int32_t& token, BlockScratch& sm, bool more_exist = false,
                                 float tau_hint = 0.0f) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  uint32_t buf = 0u;
  const RowDivisor div = row_divisor(S);
  const int n_lds = n_listed < lds_list_cap ? n_listed : lds_list_cap;
  // Calls fn(p) for the probability field of every entry (dropped entries give 0).
  auto for_each_prob = [&](auto&& fn) {
    for (int j = tid; j < n_lds; j += kBlock) fn(__uint_as_float(static_cast<uint32_t>(lds_list[j] >> 32)));
    int j = n_lds + tid;
    for (; j + 3 * kBlock < n_listed; j += 4 * kBlock) {
      const uint64_t e0 = list[j], e1 = list[j + kBlock], e2 = list[j + 2 * kBlock], e3 = list[j + 3 * kBlock];
      fn(__uint_as_float(static_cast<uint32_t>(e0 >> 32)));
      fn(__uint_as_float(static_cast<uint32_t>(e1 >> 32)));
      fn(__uint_as_float(static_cast<uint32_t>(e2 >> 32)));
      fn(__uint_as_float(static_cast<uint32_t>(e3 >> 32)));
    }
    for (; j < n_listed; j += kBlock) fn(__uint_as_float(static_cast<uint32_t>(list[j] >> 32)));
  };
  // ---- A
  float cnt = 0.0f, mass = 0.0f;
  {
    auto filter = [&](uint64_t ent) -> uint64_t {
      const float pj = div_row(__uint_as_float(static_cast<uint32_t>(ent >> 32)), div);
      const bool keep = pj >= cutoff;
      cnt += keep ? 1.0f : 0.0f;
      mass += keep ? pj : 0.0f;
      return keep ? ((static_cast<uint64_t>(__float_as_uint(pj)) << 32) | static_cast<uint32_t>(ent)) : 0ull;
    };
    for (int j = tid; j < n_lds; j += kBlock) lds_list[j] = filter(lds_list[j]);
    int j = n_lds + tid;
    for (; j + 3 * kBlock < n_listed; j += 4 * kBlock) {
      const uint64_t e0 = list[j], e1 = list[j + kBlock], e2 = list[j + 2 * kBlock], e3 = list[j + 3 * kBlock];
      list[j] = filter(e0);
      list[j + kBlock] = filter(e1);
      list[j + 2 * kBlock] = filter(e2);
      list[j + 3 * kBlock] = filter(e3);
    }
    for (; j < n_listed; j += kBlock) list[j] = filter(list[j]);
  }
  block_sum2(cnt, mass, sm, buf);  // its barrier also orders the rewrites before the reads below
  const int n0 = static_cast<int>(cnt);
  dbg.n_candidates = n0;
  if (n0 == 0) {
    if (more_exist) return false;
    token = -1;  // the reference reads probindex[-1] here
    return true;
  }
  // more_exist: the list holds the row's largest entries only (every entry that is not listed is
  // smaller than every listed one), so the walks below must end inside it
  const int n_total = more_exist ? 0x7fffffff : n0;
  // ---- B
  const float target = topp * 1.004f + 1e-6f;
  float tau = 0.0f;  // select everything
  int n_sel = n0;
  // (a short list of the row's largest entries holds little but the nucleus: sorted as it is)
  bool hinted = false;
  if (mass >= target && n0 > 64 && !(more_exist && n0 <= 1024) && tau_hint > cutoff) {
    // the caller knows a threshold that should do (from a histogram of the candidates): one pass to check it
    float c = 0.0f, m = 0.0f;
    for_each_prob([&](float pj) {
      const bool in = pj >= tau_hint;
      c += in ? 1.0f : 0.0f;
      m += in ? pj : 0.0f;
    });
    block_sum2(c, m, sm, buf);
    if (m >= target) {
      tau = tau_hint;
      n_sel = static_cast<int>(c);
      hinted = true;
    }
  }
  if (!hinted && mass >= target && n0 > 64 && !(more_exist && n0 <= 1024)) {
    float t = (1.0f / S) * 0.25f;  // the largest probability is fl(1 / S)
    for (int step = 0; step < 24 && t > cutoff; ++step, t *= 0.25f) {
      float c = 0.0f, m = 0.0f;
      for_each_prob([&](float pj) {
        const bool in = pj >= t;
        c += in ? 1.0f : 0.0f;
        m += in ? pj : 0.0f;
      });
      block_sum2(c, m, sm, buf);
      if (m >= target) {
        tau = t;
        n_sel = static_cast<int>(c);
        break;
      }
    }
    // tighten between tau (enough mass) and 4 * tau (not enough): fewer keys to sort (three steps; up to
    // eight while the selection does not fit the key buffer)
    if (tau > 0.0f && n_sel > 256) {
      float hi = tau * 4.0f;
      for (int step = 0; step < 8 && (step < 3 || pow2_ceil(n_sel) > cap); ++step) {
        const float mid = sqrtf(tau * hi);
        float c = 0.0f, m = 0.0f;
        for_each_prob([&](float pj) {
          const bool in = pj >= mid;
          c += in ? 1.0f : 0.0f;
          m += in ? pj : 0.0f;
        });
        block_sum2(c, m, sm, buf);
        if (m >= target) {
          tau = mid;
          n_sel = static_cast<int>(c);
        } else {
          hi = mid;
        }
      }
    }
  }
  // ---- C
  const int N = pow2_ceil(n_sel);
  if (N > cap) return false;
  if (tid == 0) sm.counter2 = 0u;
  __syncthreads();
  // Selected entries move to lds_keys[0, n_sel).  While they fit below the list they are appended
  // directly; otherwise the move is in place, one barrier per kBlock entries between the reads of
  // a round and its stores (a round's stores land below the positions it read).
  const bool in_place = N > list_base;
  for (int base = 0; base < n_listed; base += kBlock) {
    const int j = base + tid;
    uint64_t ent = 0ull;
    if (j < n_listed) ent = j < lds_list_cap ? lds_list[j] : list[j];
    if (in_place) __syncthreads();
    const float pj = __uint_as_float(static_cast<uint32_t>(ent >> 32));
    const bool keep = ent != 0ull && pj >= tau;
    const uint32_t slot = wave_append_slot(keep, &sm.counter2, lane);
    if (keep) lds_keys[slot] = cand_key(pj, static_cast<int>(static_cast<uint32_t>(ent)));
  }
  __syncthreads();
  for (int i = n_sel + tid; i < N; i += kBlock) lds_keys[i] = ~0ull;
  __syncthreads();
  if (n_sel <= 64) return draw_small_wave((LdsKeys)lds_keys, n_sel, n_total, topp, coin, dbg, token, sm) != -2;
  // (the list is dead from here on: what lies behind the keys is free for the sort by buckets)
  bool sorted = false;
  if (n_sel > 512 && N + n_sel + kSortBuckets <= cap) sorted = sort_keys_bucketed((LdsKeys)lds_keys, n_sel, (LdsKeys)lds_keys + N, sm);
  if (!sorted) sort_keys_lds((LdsKeys)lds_keys, N);
  const int pos = draw_from_sorted((LdsKeys)lds_keys, n_sel, n_total, false, 0, topp, coin, dbg, sm);
  if (pos == -2) return false;  // the pre-selection did not reach topp after all
  token = static_cast<int32_t>(static_cast<uint32_t>(lds_keys[pos]));
  return true;
}

// ---- top-p draw for rows scanned through the expf table ------------------------------------------
// After a kListHist scan every table entry holds e and the number of row entries with that bit
// pattern, counted at least wherever the entry can be a candidate (the scan skips entries whose e
// is below the cutoff times the running sum at the time, which only grows).  Walking the table in order of falling logit value gives, without touching the row,
// the candidate count (p = fl(e / S) >= cutoff, exact per pattern) and a probability threshold
// p_thr above which the entries carry safely more than topp.  One more pass over the row
// (L2-resident) gathers exactly the entries with p >= p_thr as sort keys; they are a prefix of the
// reference's sorted candidate array, and the two CDF walks run over them.

// Table index of position q in falling-logit order: positive patterns from the largest magnitude
// down, the positive "tiny" entry, then the negative half from "tiny" to "beyond".
__device__ __forceinline__ int hist_entry(int q, int top, int half) { return q < half ? top - q : q; }

typedef short short2v __attribute__((ext_vector_type(2)));

// Order key of a bf16 pattern: larger logit <=> larger key (-0 below +0).
__device__ __forceinline__ int pattern_order(uint32_t pattern16) {
  const int mag = static_cast<int>(pattern16 & 0x7fffu);
  return (pattern16 & 0x8000u) ? ~mag : mag;
}

// Returns false when the caller has to take the general path.
// Quotient used for comparisons: thresholds of a top-p row are far above 2^-126, those of a top-k
// row can be anything.
template <bool EXACT>
__device__ __forceinline__ float row_quotient(float e, const RowDivisor& div) {
  return EXACT ? div_row(e, div) : div_row_above(e, div);
}

// Third pass of the histogram draw: entries with order key >= k_star and p >= p_thr go to the key
// buffer.  Plain functions, not closures: a closure the compiler leaves out of line reads every
// captured value through memory.
struct GatherArgs {
  float inv, m, p_thr;
  int k_star, cap;
  RowDivisor div;
  uint64_t* lds_keys;
  BlockScratch* sm;
};

template <bool EXACT>
__device__ __forceinline__ void gather_take(uint32_t pattern16, int index, const GatherArgs& a) {
  if (pattern_order(pattern16) < a.k_star) return;
  const float x = __uint_as_float(pattern16 << 16) * a.inv;
  const float pj = row_quotient<EXACT>(expf_nonpositive(x - a.m, a.sm->exp2tab), a.div);
  if (pj >= a.p_thr) {
    const uint32_t slot = atomicAdd(&a.sm->counter2, 1u);
    if (slot < static_cast<uint32_t>(a.cap)) a.lds_keys[slot] = cand_key(pj, index);
  }
}

// Vectors are screened by their largest order key.  For a positive threshold the patterns
// themselves, read as signed 16-bit numbers, decide (negative logits are negative numbers).
template <bool POSITIVE>
__device__ __forceinline__ int best_order_key(const uint4& r) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  short2v best = {-32768, -32768};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const short2v h = __builtin_bit_cast(short2v, w[k]);
    const short2v key = POSITIVE ? h : h ^ ((h >> 15) & static_cast<short>(0x7fff));
    best = __builtin_elementwise_max(best, key);
  }
  return max(static_cast<int>(best.x), static_cast<int>(best.y));
}

template <bool POSITIVE, bool EXACT>
__device__ __forceinline__ void gather_sweep(const uint4* vec, int nvec, const GatherArgs& a) {
  const int tid = threadIdx.x;
  for (int j = tid; j < nvec; j += 16 * kBlock) {  // 16 loads in flight; out-of-range ones re-read vec[j]
    uint4 r[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int jk = j + k * kBlock;
      r[k] = vec[jk < nvec ? jk : j];
    }
    // screen first, take afterwards: the screening code stays compact (the rare take, with its
    // expf, exists once and reads its vector again)
    uint32_t hits = 0u;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int jk = j + k * kBlock;
      if (jk < nvec && best_order_key<POSITIVE>(r[k]) >= a.k_star) hits |= 1u << k;
    }
    while (hits) {
      const int k = __ffs(static_cast<int>(hits)) - 1;
      hits &= hits - 1u;
      const int jk = j + k * kBlock;
      const uint4 v = vec[jk];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll 1
      for (int h = 0; h < 8; ++h) {
        uint32_t word = w[0];
        word = (h >> 1) == 1 ? w[1] : word;
        word = (h >> 1) == 2 ? w[2] : word;
        word = (h >> 1) == 3 ? w[3] : word;
        gather_take<EXACT>((word >> ((h & 1) * 16)) & 0xffffu, jk * 8 + h, a);
      }
    }
  }
}

// With TOPK the same walk selects by COUNT instead of mass: the entries with the `topk` largest
// probabilities and everything tied with the last of them (sampler.cpp:87-100 sorts all entries;
// the walks of :103-119 only read the first topk).  The caller passes cutoff = 0 and a scan that
// counted every entry.
template <bool ALIGNED, bool TOPK>
__device__ __noinline__ bool draw_topp_hist(const char* logits, int V, float inv, float m, float S, float cutoff, float topp,
                               int topk, float coin, float* lut, int base1, int top, int half, uint64_t* lds_keys,
                               int cap, RowDebug& dbg, int32_t& token, BlockScratch& sm) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const RowDivisor div = row_divisor(S);
  const uint32_t* lut_u = reinterpret_cast<const uint32_t*>(lut);
  if (TOPK && V > (1 << 24)) return false;  // counts are summed in float
  const float target = TOPK ? static_cast<float>(topk) : topp * 1.004f + 1e-6f;

  constexpr int kMaxRun = 16;  // table positions per lane; the key buffer bounds them by 16 * kBlock
  // Every threshold below is at least the cutoff, and the cutoff is far above 2^-126 (1 - topp is
  // at least 2^-24 and the vocabulary below 2^31): div_row_above is exact wherever it matters.
  // ---- how far down the table candidates can sit: e falls along q (up to last-bit wobble of
  //      expf, far inside the 0.1 % margin), and p >= cutoff needs e >= cutoff * S * (1 - 2^-23)
  int Q = 2 * half;
  {
    const int coarse = (Q + kBlock - 1) / kBlock;
    if (coarse > kMaxRun) return false;
    const float e_min = cutoff * S * 0.999f;
    const int q = tid * coarse;
    const bool live = q < Q && lut[hist_entry(min(q, Q - 1), top, half)] >= e_min;
    const uint64_t ballot = __ballot(live);
    if (lane == 0) sm.red_u[wave] = static_cast<uint32_t>(__popcll(ballot));
    __syncthreads();
    uint32_t live_lanes = 0u;
    for (int w = 0; w < kWaves; ++w) live_lanes += sm.red_u[w];
    __syncthreads();
    Q = min(Q, static_cast<int>(live_lanes) * coarse);  // the first position of every later run is below e_min
  }
  const int run = (Q + kBlock - 1) / kBlock;
  const int q0 = min(Q, tid * run), q1 = min(Q, q0 + run);
  if (Q == 0) {
    dbg.n_candidates = 0;
    token = -1;  // the reference reads probindex[-1] here
    return true;
  }

  // ---- this lane's run of table positions: p and count of each, candidate mass and count
  float pq[kMaxRun];
  uint32_t cq[kMaxRun];
#pragma unroll
  for (int k = 0; k < kMaxRun; ++k) {
    pq[k] = 0.0f;
    cq[k] = 0u;
    if (k < run) {  // uniform
      const int q = q0 + k;
      const int idx = hist_entry(min(q, Q - 1), top, half);  // always a valid entry: no branch around the load
      const float e = lut[idx];
      const uint32_t c = lut_u[kLutCountWords + idx];
      pq[k] = q < q1 ? e : 0.0f;
      cq[k] = q < q1 ? c : 0u;
    }
  }
  float mass = 0.0f;
  uint32_t cnt = 0u;
  int last_cand = -1;
#pragma unroll
  for (int k = 0; k < kMaxRun; ++k) {
    if (k < run) {
      pq[k] = row_quotient<TOPK>(pq[k], div);
      if (pq[k] >= cutoff && cq[k] != 0u) {  // positions past the run hold count 0
        mass += TOPK ? static_cast<float>(cq[k]) : static_cast<float>(cq[k]) * pq[k];
        cnt += cq[k];
        last_cand = q0 + k;
      }
    }
  }
  const float upto = wave_scan_inclusive_f32(mass, lane);
  const uint32_t cnt_w = wave_sum_u32(cnt);
  const int last_w = wave_max_i32(last_cand);
  if (lane == 63) {
    sm.group_total[0][wave] = upto;
    sm.red_u[wave] = cnt_w;
  }
  if (lane == 0) sm.first_flag[wave] = last_w;
  if (tid == 0) {
    sm.bc_found = -1;
    sm.counter2 = 0u;
  }
  __syncthreads();
  float mass_before = 0.0f, mass_all = 0.0f;
  uint32_t n0 = 0u;
  int q_cut = -1, wave_star = -1;
  for (int w = 0; w < kWaves; ++w) {
    if (w == wave) mass_before = mass_all;
    mass_all += sm.group_total[0][w];
    n0 += sm.red_u[w];
    q_cut = max(q_cut, sm.first_flag[w]);
    if (wave_star < 0 && mass_all >= target) wave_star = w;
  }
  dbg.n_candidates = static_cast<int>(n0);
  if (n0 == 0u) {
    token = -1;  // the reference reads probindex[-1] here
    return true;
  }
  // ---- the lane whose run takes the mass past the target fixes p_thr and how far the table
  //      positions with p >= p_thr reach (q_ext); without such a lane every candidate is taken
  const bool take_all = wave_star < 0 || (!TOPK && n0 <= 64u);
  if (!take_all && wave == wave_star) {
    const float hi = mass_before + upto;  // any-order float sums: the margin in `target` covers them
    const uint64_t ballot = __ballot(hi >= target);
    const int lane_star = __ffsll(static_cast<long long>(ballot)) - 1;  // lane 63 reaches it at the latest
    const float lo = mass_before + lane_before_f32(upto);
    if (lane == lane_star) {
      float running = lo;
      int q_star = -1;
      float p_thr = 0.0f;
      bool reached = false;
#pragma unroll
      for (int k = 0; k < kMaxRun; ++k) {
        if (k < run && !reached && pq[k] >= cutoff && cq[k] != 0u) {
          running += TOPK ? static_cast<float>(cq[k]) : static_cast<float>(cq[k]) * pq[k];
          q_star = q0 + k;
          p_thr = pq[k];
          reached = running >= target;
        }
      }
      int q_ext = q_star;
      for (int q = q_star + 1; q_star >= 0 && q < Q; ++q) {
        const int idx = hist_entry(q, top, half);
        if (!(row_quotient<TOPK>(lut[idx], div) >= p_thr)) break;
        q_ext = q;
      }
      if (q_star >= 0) {
        sm.bc_found = q_ext;
        sm.bc_sum = p_thr;
      }
    }
  }
  __syncthreads();
  int q_ext = sm.bc_found;
  float p_thr = sm.bc_sum;
  if (take_all || q_ext < 0) {
    q_ext = q_cut;
    p_thr = cutoff;
  }
  // ---- nothing behind q_ext may reach p_thr (expf need not be monotone to the last bit); count
  //      what will be gathered
  uint32_t n_take = 0u;
  bool straggler = false;
#pragma unroll
  for (int k = 0; k < kMaxRun; ++k) {
    if (k < run) {
      const bool in = cq[k] != 0u && pq[k] >= p_thr;
      if (in && q0 + k > q_ext) straggler = true;
      if (in) n_take += cq[k];
    }
  }
  n_take = wave_sum_u32(n_take);
  const bool wave_straggler = __ballot(straggler) != 0ull;
  if (lane == 0) {
    sm.red_u[wave] = n_take;
    sm.first_flag[wave] = wave_straggler ? 1 : 0;
  }
  __syncthreads();
  uint32_t n_sel = 0u;
  bool any_straggler = false;
  for (int w = 0; w < kWaves; ++w) {
    n_sel += sm.red_u[w];
    any_straggler = any_straggler || sm.first_flag[w] != 0;
  }
  __syncthreads();  // the table is dead from here on: its memory becomes the key buffer
  if (any_straggler || n_sel > static_cast<uint32_t>(cap) || n_sel == 0u) return false;

  // ---- order key of the last table position taken
  int k_star;
  if (q_ext < half) {
    const int c = top - q_ext;
    k_star = c >= 1 ? base1 + c : 0;
  } else {
    const int c = q_ext - half;
    const int mag = base1 + c;
    k_star = c >= top ? -32768 : (mag >= 0 ? -mag - 1 : 0);
  }
  // ---- gather: entries with order key >= k_star and p >= p_thr
  const GatherArgs ga = {inv, m, p_thr, k_star, cap, div, lds_keys, &sm};
  int done = 0;
  if (ALIGNED) {
    const int nvec = V / 8;
    const uint4* vec = reinterpret_cast<const uint4*>(logits);
    if (k_star > 0) {
      gather_sweep<true, TOPK>(vec, nvec, ga);
    } else {
      gather_sweep<false, TOPK>(vec, nvec, ga);
    }
    done = nvec * 8;
  }
  for (int i = done + tid; i < V; i += kBlock) {
    gather_take<TOPK>(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(logits)[i]), i, ga);
  }
  __syncthreads();
  const int n_got = static_cast<int>(sm.counter2);
  if (n_got > cap || n_got == 0) return false;
  if (TOPK) {
    if (n_got < topk) return false;
    dbg.n_candidates = V;  // every entry is a candidate of a top-k draw
  } else if (n_got <= 64) {
    return draw_small_wave((LdsKeys)lds_keys, n_got, static_cast<int>(n0), topp, coin, dbg, token, sm) != -2;
  }
  const int N = pow2_ceil(n_got);
  for (int i = n_got + tid; i < N; i += kBlock) lds_keys[i] = ~0ull;
  __syncthreads();
  sort_keys_lds((LdsKeys)lds_keys, N);
  const int pos = draw_from_sorted((LdsKeys)lds_keys, n_got, static_cast<int>(n0), TOPK, topk, topp, coin, dbg, sm);
  if (pos == -2) return false;  // the pre-selection did not reach topp after all
  token = static_cast<int32_t>(static_cast<uint32_t>(lds_keys[pos]));
  return true;
}

// A lower bound of the k-th largest of the workgroup's kBlock values (one per lane, never NaN),
// exact in the upper 20 bits of the float order.  Every wave holds all values in registers; the
// bound is fixed four bits at a time: wave w counts the values at or above the bound with w in the
// next four bits, and the largest w that still leaves k values wins.  `buf` is LDS for kBlock
// words.  Ends with a barrier.
__device__ __forceinline__ float kth_largest_lane_value(float v, int k, uint32_t* buf, BlockScratch& sm) {
  static_assert(kBlock == 1024 && kWaves == 16, "sixteen values per lane, sixteen trials per step");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  buf[tid] = order_key(v);
  __syncthreads();
  const uint4* rows = reinterpret_cast<const uint4*>(buf);
  uint32_t key[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4 r = rows[j * 64 + lane];
    key[4 * j] = r.x;
    key[4 * j + 1] = r.y;
    key[4 * j + 2] = r.z;
    key[4 * j + 3] = r.w;
  }
  uint32_t bound = 0u;
  uint32_t hand = 0u;
  for (int shift = 28; shift >= 12; shift -= 4) {
    const uint32_t trial = bound | (static_cast<uint32_t>(wave) << shift);
    int count = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) count += __popcll(__ballot(key[j] >= trial));
    if (lane == 0) sm.aux_total[hand][wave] = static_cast<float>(count);  // at most kBlock: exact
    __syncthreads();
    uint32_t best = 0u;  // trial 0 is the bound itself: at least k values reach it
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      if (sm.aux_total[hand][w] >= static_cast<float>(k)) best = static_cast<uint32_t>(w);  // counts fall with w
    }
    bound |= best << shift;
    hand ^= 1u;
  }
  __syncthreads();
  // back from the order key to the float (order_key maps NaN to 0, which no value here has)
  return __uint_as_float((bound & 0x80000000u) ? (bound & 0x7fffffffu) : ~bound);
}

// Top-k draw of a row whose scan listed every entry with exp >= list_floor (at least topk of them
// by construction): sorts the listed entries and walks the first topk (sampler.cpp:87-119).
// Entries that were not listed have a smaller exp than every listed one; they could only tie with
// the topk-th probability where the division loses resolution, which the check against the
// floor's own quotient rules out.  Returns false when the caller has to take the general path.
// The list sits `list_base` keys above the start of the key buffer; the sort keys are written from
// the start of the buffer, so that the sort and the walks run on the buffer itself like every
// other caller's.
constexpr int kTopkListMax = 256;
__device__ __noinline__ bool draw_topk_listed(uint64_t* lds_keys, int cap, int list_base, int n_listed, float S,
                                              float list_floor, int topk, float topp, float coin, int V, RowDebug& dbg,
                                              int32_t& token, BlockScratch& sm) {
  const int tid = threadIdx.x;
  if (n_listed < topk || n_listed > cap - list_base) return false;
  const int N = pow2_ceil(n_listed);
  if (N > cap || (list_base != kBlock && list_base < N)) return false;
  const RowDivisor div = row_divisor(S);
  // with the list kBlock keys up, key i replaces list entry i - kBlock: the slot a lane writes is
  // the one it read one step earlier; a list further up is clear of the keys
  for (int i = tid; i < N; i += kBlock) {
    uint64_t key = ~0ull;
    if (i < n_listed) {
      const uint64_t ent = lds_keys[list_base + i];
      key = cand_key(div_row(__uint_as_float(static_cast<uint32_t>(ent >> 32)), div), static_cast<int>(static_cast<uint32_t>(ent)));
    }
    lds_keys[i] = key;
  }
  __syncthreads();
  dbg.n_candidates = V;  // every entry is a candidate of a top-k draw
  if (n_listed <= 64) {
    return draw_small_wave((LdsKeys)lds_keys, n_listed, n_listed, topp, coin, dbg, token, sm, topk,
                           div_row(list_floor, div)) != -2;
  }
  sort_keys_lds((LdsKeys)lds_keys, N);
  if (!(cand_prob(lds_keys[topk - 1]) > div_row(list_floor, div))) return false;
  const int pos = draw_from_sorted((LdsKeys)lds_keys, n_listed, n_listed, true, topk, topp, coin, dbg, sm);
  token = static_cast<int32_t>(static_cast<uint32_t>(lds_keys[pos]));
  return true;
}

// ---- the stochastic path: one workgroup per row -------------------------------------------------
// Pass 1 reads the row from HBM: maximum of x = logit * inv_temperature and whether any x is NaN.
// Pass 2 re-reads it (L2 / Infinity Cache): exact expf, the sequential sum in index order, and
// the list of possible top-p candidates.  Then the coin and the draw.
constexpr int kDrawTopP = 0, kDrawMultinomial = 1, kDrawTopK = 2;  // sampler.cpp:238-249, chosen by the host
constexpr int kDrawAny = 3;  // chosen per row from its top-k and top-p (rows with parameters of their own)

// LOOP: fewer workgroups than rows, a workgroup takes one row after the other (the loop costs
// registers, so a launch with a workgroup per row uses the instantiation without it).
template <int DT, bool ALIGNED, int DRAW, bool LOOP>
__global__ void __launch_bounds__(kBlock) sample_rows_kernel(RowParams p) {
  extern __shared__ __align__(16) uint64_t lds_keys[];
  __shared__ BlockScratch sm;
  __shared__ int next_lrow;
  constexpr int VE = VecElems<DT>::value;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int V = p.vocab;
  uint64_t* scratch = p.scratch + static_cast<int64_t>(blockIdx.x) * p.scratch_stride;
  const float kInf = __uint_as_float(0x7f800000u);
  const float kNaN = __uint_as_float(0x7fc00000u);
  for (int lrow = blockIdx.x; lrow < p.rows; lrow = LOOP ? take_row(p, &next_lrow) : p.rows) {
  if (LOOP) request_row(p, &next_lrow);
  const int row = p.row_map ? p.row_map[lrow] : lrow;
  const float inv = p.row_cfg ? p.row_cfg[row].inv_temperature : p.inv_temperature;
  const float topp = p.row_cfg ? p.row_cfg[row].topp : p.topp;
  const int32_t topk = p.row_cfg ? p.row_cfg[row].topk : p.topk;
  const char* logits = static_cast<const char*>(p.logits) + static_cast<int64_t>(row) * p.row_stride * ElemSize<DT>::value;

  if (tid < 32) sm.exp2tab[tid] = kExp2Table[tid];
  if (tid == 0) sm.counter = 0u;

  // (compile-time constants but for kDrawAny, where the row's parameters decide: sampler.cpp:238-249)
  const int draw = DRAW != kDrawAny ? DRAW
                                    : ((topk > 0 && topk < V) ? kDrawTopK : ((topp <= 0.0f || topp >= 1.0f) ? kDrawMultinomial : kDrawTopP));
  const bool use_topk = draw == kDrawTopK;
  const bool use_mult = draw == kDrawMultinomial;
  const bool use_topp = draw == kDrawTopP;

  // ---- pass 1: row maximum (sampler.cpp:231-233, 191-197)
  float m = -kInf;
  bool any_nan = false;
  {
    auto visit = [&](float l) {
      const float x = l * inv;
      m = __builtin_fmaxf(m, x);  // ignores NaN, like `if (x > max)`
      any_nan = any_nan || (x != x);
    };
    bool vectors_done = false;
    if constexpr (ALIGNED && (DT == kDtypeBFloat16 || DT == kDtypeHalf)) {
      // 16-bit rows with a positive finite 1/temperature: fl(l * inv) does not decrease as l grows,
      // so the maximum of x is the x of the largest logit, and that one is found on the raw bit
      // patterns, two per instruction.  As signed 16-bit integers the non-negative patterns order
      // like their values and every negative one is below them; among negative patterns the
      // smallest integer is the value nearest to zero.  NaN patterns lie above +inf's in signed
      // order (positive NaN) or above -inf's in unsigned order (negative NaN).
      if (inv > 0.0f && inv < kInf) {
        typedef short Short2 __attribute__((ext_vector_type(2)));
        typedef unsigned short UShort2 __attribute__((ext_vector_type(2)));
        union Word {
          uint32_t u;
          Short2 s;
          UShort2 us;
        };
        Word hi_s, lo_s, hi_u;
        hi_s.u = 0x80008000u;
        lo_s.u = 0x7fff7fffu;
        hi_u.u = 0u;
        const int nvec = V / VE;
        const uint4* vec = reinterpret_cast<const uint4*>(logits);
        for (int j = tid; j < nvec; j += 8 * kBlock) {
          uint4 r[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const int jk = j + k * kBlock;
            r[k] = vec[jk < nvec ? jk : j];
          }
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const uint32_t w[4] = {r[k].x, r[k].y, r[k].z, r[k].w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              Word x;
              x.u = w[q];
              hi_s.s = __builtin_elementwise_max(hi_s.s, x.s);
              lo_s.s = __builtin_elementwise_min(lo_s.s, x.s);
              hi_u.us = __builtin_elementwise_max(hi_u.us, x.us);
            }
          }
        }
        const int top = max(static_cast<int>(hi_s.s.x), static_cast<int>(hi_s.s.y));
        const int low = min(static_cast<int>(lo_s.s.x), static_cast<int>(lo_s.s.y));
        const uint32_t utop = max(static_cast<uint32_t>(hi_u.us.x), static_cast<uint32_t>(hi_u.us.y));
        constexpr uint32_t kInf16 = DT == kDtypeBFloat16 ? 0x7f80u : 0x7c00u;
        const bool nan_seen = top > static_cast<int>(kInf16) || utop > (0x8000u | kInf16);
        if (!nan_seen && tid < nvec) {  // (a lane with a NaN redoes its entries below, value by value)
          const uint32_t pattern = static_cast<uint32_t>(top >= 0 ? top : low) & 0xffffu;
          const float l = DT == kDtypeBFloat16 ? __uint_as_float(pattern << 16) : half_bits_to_float(pattern);
          m = l * inv;
        }
        vectors_done = !nan_seen;
      }
    }
    if (ALIGNED && vectors_done) {
      const int nvec = V / VE;
      for (int i = nvec * VE + tid; i < V; i += kBlock) visit(load_elem<DT>(logits, i));
    } else if (ALIGNED) {
      const int nvec = V / VE;
      const uint4* vec = reinterpret_cast<const uint4*>(logits);
      // eight 16-byte loads in flight per lane; out-of-range ones re-read the lane's first vector
      for (int j = tid; j < nvec; j += 8 * kBlock) {
        uint4 r[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const int jk = j + k * kBlock;
          r[k] = vec[jk < nvec ? jk : j];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          float v[VE];
          decode_vec<DT>(r[k], v);
#pragma unroll
          for (int e = 0; e < VE; ++e) visit(v[e]);
        }
      }
      for (int i = nvec * VE + tid; i < V; i += kBlock) visit(load_elem<DT>(logits, i));
    } else {
      for (int i = tid; i < V; i += kBlock) visit(load_elem<DT>(logits, i));
    }
  }
  const float lane_max = m;  // of the entries this lane read
  bool row_nan;
  {
    m = wave_max_ignoring_nan(m);
    const uint64_t nan_ballot = __ballot(any_nan);
    if (lane == 0) {
      sm.red_f[wave] = m;
      sm.red_u[wave] = nan_ballot ? 1u : 0u;
    }
    __syncthreads();
    m = sm.red_f[0];
    uint32_t nan_any = sm.red_u[0];
    for (int w = 1; w < kWaves; ++w) {
      m = (sm.red_f[w] > m) ? sm.red_f[w] : m;
      nan_any |= sm.red_u[w];
    }
    const float x0 = load_elem<DT>(logits, 0) * inv;
    if (x0 != x0) m = x0;  // max_val starts at x[0]; nothing compares greater than NaN
    // expf(x - m) is NaN for some entry exactly when an x is NaN or m is not finite (then the
    // maximal entry itself gives inf - inf); one NaN addend poisons the running sum for good
    row_nan = nan_any != 0u || !(m > -kInf && m < kInf);
    __syncthreads();
  }

  // ---- pass 2: softmax normaliser, sequential in index order (sampler.cpp:199-203)
  const float cutoff = use_topp ? (1.0f - topp) / static_cast<float>(V - 1) : 0.0f;  // sampler.cpp:136
  float S = kNaN;
  // Top-k rows (k up to kTopkListMax) list the entries that can be among the k largest.  At least k
  // entries are >= the k-th largest of the lanes' maxima, so everything clearly below the exp of
  // that value is out.
  float list_floor = 0.0f;
  bool topk_listed = false;
  if (use_topk && !row_nan && topk >= 1 && topk <= kTopkListMax && p.lds_keys >= 2 * kBlock) {
    const float t = kth_largest_lane_value(lane_max, topk, reinterpret_cast<uint32_t*>(lds_keys), sm);
    list_floor = expf_nonpositive(t - m, sm.exp2tab) * 0.998f;
    topk_listed = list_floor > 0.0f;
    if (!topk_listed) list_floor = kInf;  // nothing is listed; the draw sorts the row
  }
  bool use_lut = false;
  int lut_base1 = 0, lut_top = 0, lut_half = 0;
  float* lut = reinterpret_cast<float*>(lds_keys);  // the key buffer is free until the draw
  if (DT == kDtypeBFloat16 && ALIGNED && !row_nan && V >= 4 * kBlock) {
    use_lut = build_exp_lut(lut, p.lds_keys * 2, inv, m, sm.exp2tab, lut_base1, lut_top, lut_half);
    __syncthreads();
  }
  // Candidate lists live in the key buffer: above room for a short sorted selection, or above
  // the table and its counters; what does not fit goes to the row's scratch in global memory.
  // (Top-p rows with a table count bit patterns in the table instead.)
  int list_base = use_lut ? kLutCountWords : kBlock;  // 2 * kLutCountWords words of table = kLutCountWords keys
  if (list_base > p.lds_keys) list_base = p.lds_keys;
  uint64_t* lds_list = lds_keys + list_base;
  const int lds_list_cap = p.lds_keys - list_base;
  if (!row_nan) {
    ScanArgs a = {logits, V,        inv,       m,       row_divisor(1.0f), kInf, cutoff, scratch, lut,
                  lut_base1, lut_top, lut_half, lds_list, lds_list_cap, list_floor,
                  (use_mult && !use_lut) ? reinterpret_cast<float*>(scratch) : nullptr};
    SeqSum st = {0.0f, -1, 0u};
    bool scanned = false;
    if constexpr (DT == kDtypeBFloat16 && ALIGNED) {
      if (use_lut) {
        if (use_topk && topk_listed) {
          scan_row<DT, ALIGNED, kScanSum, kListAppend, true, true>(a, st, sm);
        } else if (use_topp || use_topk) {  // top-k beyond the listed sizes: the cutoff is 0, every entry is counted
          scan_row<DT, ALIGNED, kScanSum, kListHist, true>(a, st, sm);
        } else {
          scan_row<DT, ALIGNED, kScanSum, kListNone, true>(a, st, sm);
        }
        scanned = true;
      }
    }
    if (!scanned) {
      if (use_topk && topk_listed) {
        scan_row<DT, ALIGNED, kScanSum, kListAppend, false, true>(a, st, sm);
      } else if (use_topp) {
        scan_row<DT, ALIGNED, kScanSum, kListAppend, false>(a, st, sm);
      } else {
        scan_row<DT, ALIGNED, kScanSum, kListNone, false>(a, st, sm);
      }
    }
    S = st.s;
  }

  // ---- one coin per call (sampler.cpp:237, 210-220)
  if (tid == 0) {
    uint64_t rs = p.rng[row];
    rs ^= rs >> 12;
    rs ^= rs << 25;
    rs ^= rs >> 27;
    p.rng[row] = rs;
    const uint32_t u = static_cast<uint32_t>((rs * 0x2545F4914F6CDD1Dull) >> 32);
    sm.red_f[0] = static_cast<float>(u >> 8) / 16777216.0f;
  }
  __syncthreads();
  const float coin = sm.red_f[0];
  const int n_listed = static_cast<int>(sm.counter);
  __syncthreads();

  if (p.probs) {
    float* probs = p.probs + static_cast<int64_t>(row) * V;
    if (row_nan) {
      for (int i = tid; i < V; i += kBlock) {
        const float x = load_elem<DT>(logits, i) * inv;
        probs[i] = expf_nonpositive(x - m, sm.exp2tab) / S;
      }
    } else {
      const RowDivisor div = row_divisor(S);
      for (int i = tid; i < V; i += kBlock) {
        const float x = load_elem<DT>(logits, i) * inv;
        probs[i] = div_row(expf_nonpositive(x - m, sm.exp2tab), div);
      }
    }
  }

  // The draw's results live in LDS: the draw functions are calls, and a result in a lane's own
  // variable would be passed by address, which puts it (and every lane's copy) in private memory.
  // Every lane stores the same values.
  __shared__ RowDebug dbg;
  __shared__ int32_t token;
  if (tid == 0) {
    dbg = RowDebug{m, S, coin, 0.0f, 0.0f, 0, 0, 0};
    token = -1;
  }
  __syncthreads();
  if (row_nan) {
    // Every probability is NaN.  The multinomial walk never fires and returns the last index
    // (sampler.cpp:58-70); top-p keeps no candidate, where the reference reads probindex[-1]:
    // report -1; top-k's comparisons are all false, so every entry ties with every other: in
    // index order the first topk are entries 0 .. topk-1, their mass is NaN, the walk never fires
    // and the fallback is the last of them (sampler.cpp:103-119).
    token = use_mult ? V - 1 : (use_topk ? topk - 1 : -1);
  } else if (use_mult) {
    // ---- sampler.cpp:58-70: first index whose running sum of probabilities exceeds the coin
    ScanArgs a = {logits, V, inv, m, row_divisor(S), coin, 0.0f, nullptr, lut, lut_base1, lut_top, lut_half, nullptr, 0, 0.0f, nullptr};
    SeqSum walk = {0.0f, -1, 0u};
    bool walked = false;
    if constexpr (DT == kDtypeBFloat16 && ALIGNED) {
      if (use_lut) {
        // one division per bit pattern instead of one per entry: the table becomes p = fl(e / S)
        const RowDivisor div = row_divisor(S);
        for (int idx = tid; idx < 2 * lut_half; idx += kBlock) lut[idx] = div_row(lut[idx], div);
        __syncthreads();
        scan_row<DT, ALIGNED, kScanWalk, kListNone, true>(a, walk, sm);
        walked = true;
      }
    }
    if (!walked) {
      // pass 2 kept every e_i in the row's scratch: the walk divides them instead of redoing expf
      a.logits = reinterpret_cast<const char*>(scratch);
      scan_row<kDtypeFloat, true, kScanWalkCached, kListNone, false>(a, walk, sm);
    }
    token = walk.stop_index >= 0 ? walk.stop_index : V - 1;
    dbg.cumulative = walk.s;
    dbg.position = token;
  } else {
    bool done = false, tried = false;
    if constexpr (DT == kDtypeBFloat16 && ALIGNED) {
      if (use_topp && use_lut) {
        done = draw_topp_hist<ALIGNED, false>(logits, V, inv, m, S, cutoff, topp, 0, coin, lut, lut_base1, lut_top,
                                              lut_half, lds_keys, p.lds_keys, dbg, token, sm);
        tried = true;
      }
      if (use_topk && use_lut && !topk_listed) {
        done = draw_topp_hist<ALIGNED, true>(logits, V, inv, m, S, 0.0f, topp, topk, coin, lut, lut_base1, lut_top,
                                             lut_half, lds_keys, p.lds_keys, dbg, token, sm);
      }
    }
    if (use_topk && topk_listed) {
      done = draw_topk_listed(lds_keys, p.lds_keys, list_base, n_listed, S, list_floor, topk, topp, coin, V, dbg, token, sm);
    }
    if (use_topp && !tried) {
      done = draw_topp_listed(scratch, lds_list, lds_list_cap, list_base, n_listed, S, cutoff, topp, coin, lds_keys,
                              p.lds_keys, dbg, token, sm);
    }
    if (!done) {
      token = draw_general<DT>(logits, V, inv, m, S, use_topk, topk, topp, cutoff, coin, scratch, p.scratch_stride,
                               lds_keys, p.lds_keys, dbg, sm);
    }
  }
  if (tid == 0) {
    p.tokens[row] = token;
    if (p.debug) p.debug[row] = dbg;
  }
  }  // rows of this workgroup
}

}  // namespace ets
