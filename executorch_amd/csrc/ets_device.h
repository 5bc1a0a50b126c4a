// Device-side building blocks of the gfx950 token sampler: exact fp32 conversions, a
// bit-faithful expf, and the "sequential float sum" emulation that lets a 1024-lane
// workgroup reproduce a scalar `s += a[i]` loop bit for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ETS_HD __host__ __device__ __forceinline__
#include "ets_seqsum_math.h"

namespace ets {

constexpr int kBlock = 1024;           // lanes per workgroup in the row kernels
constexpr int kWaves = kBlock / 64;    // wave64 wavefronts per workgroup
constexpr int kRun = 4;                // consecutive elements owned by one lane per chunk
constexpr int kChunk = kBlock * kRun;  // elements a workgroup consumes per step

constexpr int kDtypeHalf = 5, kDtypeFloat = 6, kDtypeBFloat16 = 15, kDtypeUInt16 = 27;

// ---- element loads: every storage type converts to fp32 exactly -----------------------------
template <int DT>
__device__ __forceinline__ float load_elem(const void* row, int64_t i);

template <>
__device__ __forceinline__ float load_elem<kDtypeFloat>(const void* row, int64_t i) {
  return static_cast<const float*>(row)[i];
}
template <>
__device__ __forceinline__ float load_elem<kDtypeHalf>(const void* row, int64_t i) {
  return static_cast<float>(static_cast<const _Float16*>(row)[i]);
}
template <>
__device__ __forceinline__ float load_elem<kDtypeBFloat16>(const void* row, int64_t i) {
  return __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(row)[i]) << 16);
}
template <>
__device__ __forceinline__ float load_elem<kDtypeUInt16>(const void* row, int64_t i) {
  return static_cast<float>(static_cast<const uint16_t*>(row)[i]);
}

template <int DT>
struct ElemSize {
  static constexpr int value = (DT == kDtypeFloat) ? 4 : 2;
};

// ---- expf, bit-identical to glibc's (sysdeps/ieee754/flt-32/e_expf.c, FMA build) ------------
// exp(x) = 2^(k/32) * 2^(r/32), k = round(x * 32/ln2): 2^(k/32) from a 32-entry table of
// doubles, 2^(r/32) from a cubic in r, all in double with one final rounding to float.  The
// reference sampler calls libm expf once per vocabulary entry (sampler.cpp:201); matching its
// last bit is what makes the sequential softmax sum reproducible.
__device__ __constant__ uint64_t kExp2Table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

// `tab` is a copy of kExp2Table in LDS (lanes index it divergently).
__device__ __forceinline__ float expf_exact(float x, const uint64_t* tab) {
  const uint32_t ux = __float_as_uint(x);
  const uint32_t abstop = (ux >> 20) & 0x7ffu;
  if (abstop >= 0x42bu) {  // |x| >= 88, inf or NaN
    if (ux == 0xff800000u) return 0.0f;
    if (abstop >= 0x7f8u) return x + x;
    if (x > 0x1.62e42ep6f) return __uint_as_float(0x7f800000u);
    if (x < -0x1.9fe368p6f) return 0.0f;
  }
  const double kInvLn2N = 0x1.71547652b82fep+0 * 32.0;
  const double kShift = 0x1.8p+52;
  const double kC0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
  const double kC1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
  const double kC2 = 0x1.62e42ff0c52d6p-1 / 32.0;
  const double xd = static_cast<double>(x);
  double kd = __builtin_fma(kInvLn2N, xd, kShift);
  const uint64_t ki = static_cast<uint64_t>(__double_as_longlong(kd));
  kd -= kShift;
  const double r = __builtin_fma(kInvLn2N, xd, -kd);
  const uint64_t t = tab[ki & 31u] + (ki << 47);
  const double s = __longlong_as_double(static_cast<long long>(t));
  const double z = __builtin_fma(kC0, r, kC1);
  const double r2 = r * r;
  double y = __builtin_fma(kC2, r, 1.0);
  y = __builtin_fma(z, r2, y);
  y = y * s;
  return static_cast<float>(y);
}

__device__ __forceinline__ ParityInc wave_scan_inclusive(ParityInc v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    ParityInc o;
    o.even = __shfl_up(v.even, d);
    o.odd = __shfl_up(v.odd, d);
    if (lane >= d) v = compose(o, v);
  }
  return v;
}

// LDS scratch shared by the workgroup-wide primitives.
struct BlockScratch {
  uint64_t exp2tab[32];
  ParityInc wave_total[kWaves];
  int first_flag[kWaves];
  float red_f[kWaves];
  uint32_t red_u[kWaves];
  float bc_sum;
  int bc_found;
  uint32_t counter;
  int flag;
};

struct SeqSumResult {
  float sum;      // value of s after the last element consumed
  int stop_index; // first i with s > threshold after adding a[i]; -1 if none
};

// Emulates, with all kBlock lanes of the workgroup,
//     s = s0; for (i = 0; i < n; ++i) { s += a(i); if (s > threshold) return {s, i}; }
// bit for bit in fp32.  `a(i)` must return a finite, non-negative float and is evaluated once
// per element; pass threshold = +inf to sum everything.  Must be called by every lane.
template <typename Fetch>
__device__ SeqSumResult seq_sum_block(Fetch a, int n, float s0, float threshold, BlockScratch& sm) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  float s = s0;
  for (int base = 0; base < n; base += kChunk) {
    uint32_t bits[kRun];
    const int first = base + tid * kRun;
#pragma unroll
    for (int e = 0; e < kRun; ++e) {
      const int i = first + e;
      bits[e] = (i < n) ? __float_as_uint(a(i)) : 0u;
    }
    int resume = 0;  // chunk-relative lane index from which elements are still unconsumed
    while (true) {
      const SumState st = sum_state(s);
      ParityInc mine = {0u, 0u};
      if (tid >= resume) {
#pragma unroll
        for (int e = 0; e < kRun; ++e) fold_elem(mine, bits[e], st.kb);
      }
      const ParityInc incl_w = wave_scan_inclusive(mine, lane);
      if (lane == 63) sm.wave_total[wave] = incl_w;
      __syncthreads();
      ParityInc prefix = {0u, 0u};
      ParityInc total = {0u, 0u};
      for (int w = 0; w < kWaves; ++w) {
        if (w == wave) prefix = total;
        total = compose(total, sm.wave_total[w]);
      }
      ParityInc excl_w;
      excl_w.even = __shfl_up(incl_w.even, 1);
      excl_w.odd = __shfl_up(incl_w.odd, 1);
      if (lane == 0) excl_w = {0u, 0u};
      const ParityInc excl = compose(prefix, excl_w);
      const ParityInc incl = compose(excl, mine);
      const bool odd = st.S & 1u;
      const uint32_t S_excl = st.S + (odd ? excl.odd : excl.even);
      const uint32_t S_incl = st.S + (odd ? incl.odd : incl.even);
      // A lane needs scalar treatment if its run leaves the binade or crosses the threshold.
      bool special = S_incl >= (1u << 24);
      if (!special) special = sum_value(S_incl, st.kb) > threshold;
      const uint64_t ballot = __ballot(special);
      if (lane == 0) sm.first_flag[wave] = ballot ? (wave * 64 + __ffsll(static_cast<long long>(ballot)) - 1) : kBlock;
      __syncthreads();
      int j = kBlock;
      for (int w = 0; w < kWaves; ++w) {
        const int f = sm.first_flag[w];
        if (f < kBlock) {
          j = f;
          break;
        }
      }
      if (j == kBlock) {  // whole chunk consumed inside the binade
        s = sum_value(st.S + (odd ? total.odd : total.even), st.kb);
        break;
      }
      if (tid == j) {
        float sj = sum_value(S_excl, st.kb);
        int found = -1;
#pragma unroll
        for (int e = 0; e < kRun; ++e) {
          const int i = first + e;
          if (i < n && found < 0) {
            sj = sj + __uint_as_float(bits[e]);
            if (sj > threshold) found = i;
          }
        }
        sm.bc_sum = sj;
        sm.bc_found = found;
      }
      __syncthreads();
      s = sm.bc_sum;
      const int found = sm.bc_found;
      if (found >= 0) return {s, found};
      resume = j + 1;
    }
  }
  return {s, -1};
}

// ---- small workgroup reductions ----------------------------------------------------------------
__device__ __forceinline__ float wave_max_ignoring_nan(float v) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    const float o = __shfl_xor(v, d);
    v = (o > v) ? o : v;
  }
  return v;
}

}  // namespace ets
