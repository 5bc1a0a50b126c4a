// Device-side building blocks of the gfx950 token sampler: exact fp32 conversions, a
// bit-faithful expf, and the "sequential float sum" emulation that lets a 1024-lane
// workgroup reproduce a scalar `s += a[i]` loop bit for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ETS_HD __host__ __device__ __forceinline__
#include "ets_seqsum_math.h"

namespace ets {

constexpr int kBlock = 1024;         // lanes per workgroup in the row kernels
constexpr int kWaves = kBlock / 64;  // wave64 wavefronts per workgroup

constexpr int kDtypeHalf = 5, kDtypeFloat = 6, kDtypeBFloat16 = 15, kDtypeUInt16 = 27;

template <int DT>
struct ElemSize {
  static constexpr int value = (DT == kDtypeFloat) ? 4 : 2;
};
// Elements per 16-byte vector load.
template <int DT>
struct VecElems {
  static constexpr int value = 16 / ElemSize<DT>::value;
};

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

__device__ __forceinline__ float half_bits_to_float(uint32_t h16) {
  union {
    uint16_t u;
    _Float16 f;
  } cvt;
  cvt.u = static_cast<uint16_t>(h16);
  return static_cast<float>(cvt.f);
}

// Decode one 16-byte vector into VecElems<DT> floats.
template <int DT>
__device__ __forceinline__ void decode_vec(const uint4& raw, float* out) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  if (DT == kDtypeFloat) {
#pragma unroll
    for (int k = 0; k < 4; ++k) out[k] = __uint_as_float(w[k]);
  } else if (DT == kDtypeBFloat16) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      out[2 * k] = __uint_as_float(w[k] << 16);
      out[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
    }
  } else if (DT == kDtypeHalf) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      out[2 * k] = half_bits_to_float(w[k] & 0xffffu);
      out[2 * k + 1] = half_bits_to_float(w[k] >> 16);
    }
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      out[2 * k] = static_cast<float>(w[k] & 0xffffu);
      out[2 * k + 1] = static_cast<float>(w[k] >> 16);
    }
  }
}

// Elements [first, first + VecElems) of a row as floats; positions >= n read as `fill`.
// ALIGNED rows (16-byte aligned base and pitch) use one 128-bit load for interior vectors.
template <int DT, bool ALIGNED>
__device__ __forceinline__ void load_run(const void* row, int first, int n, float fill, float* out) {
  constexpr int VE = VecElems<DT>::value;
  if (ALIGNED && first + VE <= n) {
    const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const char*>(row) +
                                                      static_cast<int64_t>(first) * ElemSize<DT>::value);
    decode_vec<DT>(raw, out);
  } else {
#pragma unroll
    for (int e = 0; e < VE; ++e) out[e] = (first + e < n) ? load_elem<DT>(row, first + e) : fill;
  }
}

// ---- expf, bit-identical to glibc's (sysdeps/ieee754/flt-32/e_expf.c, FMA build) ------------
// exp(x) = 2^(k/32) * 2^(r/32), k = round(x * 32/ln2): 2^(k/32) from a 32-entry table of
// doubles, 2^(r/32) from a cubic in r, all in double with one final rounding to float.  The
// reference sampler calls libm expf once per vocabulary entry (sampler.cpp:201); matching its
// last bit is what makes the sequential softmax sum reproducible.
static __device__ __constant__ uint64_t kExp2Table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

// The table-and-cubic core for |x| < 104 (no special cases).  `tab` is a copy of kExp2Table in
// LDS (lanes index it divergently).
__device__ __forceinline__ float expf_core(float x, const uint64_t* tab) {
  const double kInvLn2N = 0x1.71547652b82fep+0 * 32.0;
  const double kShift = 0x1.8p+52;
  const double kC0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
  const double kC1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
  const double kC2 = 0x1.62e42ff0c52d6p-1 / 32.0;
  const double xd = static_cast<double>(x);
  double kd = __builtin_fma(kInvLn2N, xd, kShift);
  const uint32_t ki_lo = static_cast<uint32_t>(__double_as_longlong(kd));  // round(x*32/ln2) mod 2^32
  kd -= kShift;
  const double r = __builtin_fma(kInvLn2N, xd, -kd);
  // t = tab[k % 32] + (k << 47): the shifted term only touches the high word
  const uint64_t te = tab[ki_lo & 31u];
  const uint32_t t_hi = static_cast<uint32_t>(te >> 32) + (ki_lo << 15);
  const double s = __hiloint2double(static_cast<int>(t_hi), static_cast<int>(static_cast<uint32_t>(te)));
  const double z = __builtin_fma(kC0, r, kC1);
  const double r2 = r * r;
  double y = __builtin_fma(kC2, r, 1.0);
  y = __builtin_fma(z, r2, y);
  y = y * s;
  return static_cast<float>(y);
}

// Full expf (every float input).
__device__ __forceinline__ float expf_exact(float x, const uint64_t* tab) {
  const uint32_t ux = __float_as_uint(x);
  const uint32_t abstop = (ux >> 20) & 0x7ffu;
  if (abstop >= 0x42bu) {  // |x| >= 88, inf or NaN
    if (ux == 0xff800000u) return 0.0f;
    if (abstop >= 0x7f8u) return x + x;
    if (x > 0x1.62e42ep6f) return __uint_as_float(0x7f800000u);
    if (x < -0x1.9fe368p6f) return 0.0f;
  }
  return expf_core(x, tab);
}

// expf for the softmax argument d = x - max, i.e. d <= 0 or NaN.  Branch-free: below
// ln(2^-150) = -103.972 the result is 0, which is also what the core returns at -104, so
// clamping there is exact.  A NaN argument comes back as NaN.
__device__ __forceinline__ float expf_nonpositive(float d, const uint64_t* tab) {
  const float dc = (d > -104.0f) ? d : -104.0f;  // also maps NaN to -104
  const float e = expf_core(dc, tab);
  return (d != d) ? d : e;
}

// ---- workgroup-wide primitives ------------------------------------------------------------------
// Reductions over the 64 lanes, result in every lane.  Six DPP steps (a VALU operand taken from
// another lane: shifts inside each row of 16, then two row broadcasts) leave the total in lane 63;
// a butterfly of shuffles would cost six round trips through the LDS crossbar.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_u32_or(uint32_t fallback, uint32_t v) {
  // lanes without a source under CTRL (or masked off) read `fallback`
  return __builtin_amdgcn_update_dpp(fallback, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
  v += dpp_u32_or<0x111, 0xf>(0u, v);
  v += dpp_u32_or<0x112, 0xf>(0u, v);
  v += dpp_u32_or<0x114, 0xf>(0u, v);
  v += dpp_u32_or<0x118, 0xf>(0u, v);
  v += dpp_u32_or<0x142, 0xa>(0u, v);
  v += dpp_u32_or<0x143, 0xc>(0u, v);
  return __builtin_amdgcn_readlane(v, 63);
}
// Inclusive prefix sums of a 32-bit value over the 64 lanes (wraps like the type).
__device__ __forceinline__ uint32_t wave_scan_inclusive_u32(uint32_t v) {
  v += dpp_u32_or<0x111, 0xf>(0u, v);
  v += dpp_u32_or<0x112, 0xf>(0u, v);
  v += dpp_u32_or<0x114, 0xf>(0u, v);
  v += dpp_u32_or<0x118, 0xf>(0u, v);
  v += dpp_u32_or<0x142, 0xa>(0u, v);
  v += dpp_u32_or<0x143, 0xc>(0u, v);
  return v;
}
__device__ __forceinline__ int wave_max_i32(int v) {
#define ETS_MAX_STEP(CTRL, MASK)                                                                      \
  {                                                                                                   \
    const int o = static_cast<int>(dpp_u32_or<CTRL, MASK>(static_cast<uint32_t>(v), static_cast<uint32_t>(v))); \
    v = o > v ? o : v;                                                                                \
  }
  ETS_MAX_STEP(0x111, 0xf) ETS_MAX_STEP(0x112, 0xf) ETS_MAX_STEP(0x114, 0xf) ETS_MAX_STEP(0x118, 0xf)
  ETS_MAX_STEP(0x142, 0xa) ETS_MAX_STEP(0x143, 0xc)
#undef ETS_MAX_STEP
  return static_cast<int>(__builtin_amdgcn_readlane(static_cast<uint32_t>(v), 63));
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  // (lanes without a source read 0, the identity of the maximum: one instruction per step)
#define ETS_MAX_STEP(CTRL, MASK)                      \
  {                                                   \
    const uint32_t o = dpp_u32_or<CTRL, MASK>(0u, v); \
    v = o > v ? o : v;                                \
  }
  ETS_MAX_STEP(0x111, 0xf) ETS_MAX_STEP(0x112, 0xf) ETS_MAX_STEP(0x114, 0xf) ETS_MAX_STEP(0x118, 0xf)
  ETS_MAX_STEP(0x142, 0xa) ETS_MAX_STEP(0x143, 0xc)
#undef ETS_MAX_STEP
  return __builtin_amdgcn_readlane(v, 63);
}

// Unsigned key of a float: a larger value has a larger key (-0 below +0; a NaN with the sign bit
// clear above +inf), and back.
__device__ __forceinline__ uint32_t float_max_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return u ^ (static_cast<uint32_t>(static_cast<int32_t>(u) >> 31) | 0x80000000u);
}
__device__ __forceinline__ float float_of_max_key(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

__device__ __forceinline__ float wave_max_ignoring_nan(float v) {
#define ETS_MAX_STEP(CTRL, MASK)                                                                      \
  {                                                                                                   \
    const float o = __uint_as_float(dpp_u32_or<CTRL, MASK>(__float_as_uint(v), __float_as_uint(v)));    \
    v = (o > v) ? o : v;                                                                              \
  }
  ETS_MAX_STEP(0x111, 0xf) ETS_MAX_STEP(0x112, 0xf) ETS_MAX_STEP(0x114, 0xf) ETS_MAX_STEP(0x118, 0xf)
  ETS_MAX_STEP(0x142, 0xa) ETS_MAX_STEP(0x143, 0xc)
#undef ETS_MAX_STEP
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 63));
}

// LDS scratch shared by the workgroup-wide primitives.
struct BlockScratch {
  uint64_t exp2tab[32];
  ParityInc wave_total[2][64];      // per (chunk, wave) slot; double-buffered, like group_total
  int first_flag[kWaves];
  float group_total[2][kWaves];    // same, for block_sum2
  float slot_total[2][2 * kWaves];  // same, for seq_sum_group: one entry per (chunk, wave) slot
  uint32_t slot_tie[2][2 * kWaves];  //   whether the slot holds a half-ulp tie
  uint32_t tie_fix[2 * kWaves];     //   what a slot's ties add to its increments (see seq_sum_group)
  float slot_sum[64];               // plain float sums per slot (seq_sum_predicted)
  float chain_s[2];                 // running sum handed from one serial slot to the next
  int chain_found[2];               //   and where the threshold was crossed, if it was
  float aux_total[2][kWaves];      // second value of block_sum2
  float red_f[kWaves];
  uint32_t red_u[kWaves];
  float bc_sum;
  int bc_found;
  uint32_t counter;
  uint32_t counter2;
  int flag;
};

struct SeqSumResult {
  float sum;       // value of s after the last element consumed
  int stop_index;  // first i with s > threshold after adding a[i]; -1 if none
};

// Running state of a sequential sum that a workgroup advances chunk by chunk.
struct SeqSum {
  float s;
  int stop_index;
  uint32_t parity_buf;  // which half of the double-buffered LDS totals the next round uses
};

// Lane-local summary of the order-free shortcut, accumulated in float while the elements are
// produced: inc = sum of rne(a / ulp(s)) (exact while below 2^24), tie = max |t - rne(t)|, which is
// 0.5 exactly when some element sits on a half-ulp tie.
struct FastAcc {
  float inc;
  float tie;
};

// Scale that maps an addend to units of ulp(s); 0 when s is too small for the shortcut.
__device__ __forceinline__ float fast_scale(float s) {
  const SumState ss = sum_state(s);
  return ss.kb >= 64 ? __uint_as_float(static_cast<uint32_t>(277 - ss.kb) << 23) : 0.0f;
}

__device__ __forceinline__ void fast_fold(FastAcc& a, float e, float scale) {
  const float t = e * scale;
  const float r = __builtin_rintf(t);
  a.inc += r;
  a.tie = __builtin_fmaxf(a.tie, __builtin_fabsf(t - r));
}

// ---- wave64 cross-lane helpers on DPP (data-parallel primitives: a VALU operand taken from another
// lane of the same row of 16, or a row broadcast).  A DPP step costs one VALU issue; a shuffle
// through ds_bpermute costs an LDS round trip, which dominates single-wave code.
template <int CTRL, int ROW_MASK, int BANK_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {
  // lanes without a source under CTRL (or masked off) read 0
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, ROW_MASK, BANK_MASK, false));
}

// Inclusive prefix sum over the 64 lanes: Hillis-Steele inside each row of 16 (row_shr 1, 2, 4, 8),
// then row_bcast:15 into rows 1 and 3 and row_bcast:31 into rows 2 and 3.
__device__ __forceinline__ float wave_scan_inclusive_f32(float v, int /*lane*/) {
  v += dpp_or_zero<0x111, 0xf, 0xf>(v);
  v += dpp_or_zero<0x112, 0xf, 0xf>(v);
  v += dpp_or_zero<0x114, 0xf, 0xf>(v);
  v += dpp_or_zero<0x118, 0xf, 0xf>(v);
  v += dpp_or_zero<0x142, 0xa, 0xf>(v);
  v += dpp_or_zero<0x143, 0xc, 0xf>(v);
  return v;
}

// The same scan for parity summaries (compose() is associative, not commutative: the earlier lanes
// go on the left).  Lanes without a source read the identity {0, 0}.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ ParityInc dpp_parity_or_identity(ParityInc v) {
  ParityInc r;
  r.even = __builtin_amdgcn_update_dpp(0u, v.even, CTRL, ROW_MASK, 0xf, false);
  r.odd = __builtin_amdgcn_update_dpp(0u, v.odd, CTRL, ROW_MASK, 0xf, false);
  return r;
}
__device__ __forceinline__ ParityInc wave_scan_inclusive(ParityInc v, int /*lane*/) {
  v = compose(dpp_parity_or_identity<0x111, 0xf>(v), v);
  v = compose(dpp_parity_or_identity<0x112, 0xf>(v), v);
  v = compose(dpp_parity_or_identity<0x114, 0xf>(v), v);
  v = compose(dpp_parity_or_identity<0x118, 0xf>(v), v);
  v = compose(dpp_parity_or_identity<0x142, 0xa>(v), v);
  v = compose(dpp_parity_or_identity<0x143, 0xc>(v), v);
  return v;
}

// Value of lane `l` (wave-uniform index) in every lane.
__device__ __forceinline__ float readlane_f32(float v, int l) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), l));
}
__device__ __forceinline__ uint32_t readlane_u32(uint32_t v, int l) { return __builtin_amdgcn_readlane(v, l); }

// A value that is the same in every lane, moved to a scalar register: what is computed from it
// (exponent, mantissa, branches) then runs on the scalar unit.
__device__ __forceinline__ float uniform_f32(float v) {
  return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v)));
}

// Sum over the 64 lanes, in every lane.
__device__ __forceinline__ float wave_sum_f32(float v) { return readlane_f32(wave_scan_inclusive_f32(v, 0), 63); }

// Value of the previous lane (0 in lane 0): wave_shr:1.
__device__ __forceinline__ float lane_before_f32(float v) { return dpp_or_zero<0x138, 0xf, 0xf>(v); }

// Summary of a lane's run of R elements for the running sum s (see ets_seqsum_math.h).
template <int R>
__device__ __forceinline__ ParityInc fold_run(const uint32_t (&bits)[R], float s) {
  const SumState ss = sum_state(s);
  ParityInc acc = {0u, 0u};
  if (ss.kb >= 64) {
    const float scale = __uint_as_float(static_cast<uint32_t>(277 - ss.kb) << 23);  // 2^(150 - kb)
#pragma unroll
    for (int e = 0; e < R; ++e) fold_elem_scaled(acc, __uint_as_float(bits[e]), scale);
  } else {
#pragma unroll
    for (int e = 0; e < R; ++e) fold_elem(acc, bits[e], ss.kb);
  }
  return acc;
}

// One wavefront consumes its own 64 runs exactly, starting from running sum s.  No barriers: only
// this wave takes part.  On return s is the running sum after the wave's last element, or `found`
// is the position where the threshold was crossed.
//
// Common case (s >= 2^-63): the lanes' increments rne(a / ulp(s)) are summed in float (exact below
// 2^24).  A lane is an "event" if one of its elements sits on a half-ulp tie (the only case in
// which an increment depends on the order), or if the prefix sum up to and including it leaves
// the binade of s or crosses the threshold.  The first event lane adds its elements natively and
// the scan restarts behind it with the new ulp.  Tiny running sums use the two-hypothesis parity
// summaries instead (integer arithmetic, any magnitude).
// (The ordered paths are forced inline: left out of line they take the group's entries by
// reference, which puts that array -- written for every entry of the row -- into private memory.)
template <int R>
__device__ __forceinline__ void wave_resolve(float& s, int& found, const uint32_t (&bits)[R], int first, int n, float threshold,
                             int consumed = 0) {  // lanes below `consumed` have been consumed
  const int lane = threadIdx.x & 63;
  found = -1;
  s = uniform_f32(s);
  if (s == 0.0f && consumed == 0) {
    // The start of a row: while the running sum is of the order of its addends it leaves a binade
    // or meets a half-ulp tie every few elements (about ln(k) times in the first k), and every
    // such event costs the loop below a round.  The first lanes add their elements natively, one
    // lane after the other.
    constexpr int kNativeLanes = 8;
#pragma unroll 1
    for (int l = 0; l < kNativeLanes; ++l) {
      float sl = s;
      int fl = -1;
      if (lane == l) {
#pragma unroll
        for (int e = 0; e < R; ++e) {
          const int i = first + e;
          if (i < n && fl < 0) {
            sl = sl + __uint_as_float(bits[e]);
            if (sl > threshold) fl = i;
          }
        }
      }
      s = readlane_f32(sl, l);
      fl = static_cast<int>(readlane_u32(static_cast<uint32_t>(fl), l));
      if (fl >= 0) {
        found = fl;
        return;
      }
    }
    consumed = kNativeLanes;
  }
  while (consumed < 64) {
    const float scale = fast_scale(s);
    const SumState ss = sum_state(s);
    uint64_t ballot;
    uint32_t S_excl, S_end;
    if (scale != 0.0f) {
      FastAcc acc = {0.0f, 0.0f};
      if (lane >= consumed) {
#pragma unroll
        for (int e = 0; e < R; ++e) fast_fold(acc, __uint_as_float(bits[e]), scale);
      }
      const float incl = wave_scan_inclusive_f32(acc.inc, lane);
      const float room = static_cast<float>((1u << 24) - ss.S);
      bool special = acc.tie == 0.5f || !(incl < room);
      if (!special) special = sum_value(ss.S + static_cast<uint32_t>(incl), ss.kb) > threshold;
      ballot = __ballot(special);
      // exact for every lane up to the first event (all prefix sums in front of it are below `room`)
      const float excl = lane_before_f32(incl);
      S_excl = ss.S + static_cast<uint32_t>(excl < room ? excl : 0.0f);
      const float total = readlane_f32(incl, 63);
      S_end = ss.S + static_cast<uint32_t>(total < room ? total : 0.0f);
    } else {
      ParityInc mine = {0u, 0u};
      if (lane >= consumed) mine = fold_run<R>(bits, s);
      const ParityInc incl = wave_scan_inclusive(mine, lane);
      ParityInc excl;
      excl.even = __shfl_up(incl.even, 1);
      excl.odd = __shfl_up(incl.odd, 1);
      if (lane == 0) excl = {0u, 0u};
      const bool odd = ss.S & 1u;
      const uint32_t S_incl = ss.S + (odd ? incl.odd : incl.even);
      S_excl = ss.S + (odd ? excl.odd : excl.even);
      bool special = S_incl >= (1u << 24);
      if (!special) special = sum_value(S_incl, ss.kb) > threshold;
      ballot = __ballot(special);
      S_end = __shfl(S_incl, 63);
    }
    // (lanes already consumed hold no increment, but a running sum that is above the threshold
    // before anything is added flags them too: the walk only ever looks ahead)
    const int j = next_event(ballot, consumed, 64);
    if (j == 64) {
      s = sum_value(S_end, ss.kb);
      return;
    }
    float sj = 0.0f;
    int fj = -1;
    if (lane == j) {
      sj = sum_value(S_excl, ss.kb);
#pragma unroll
      for (int e = 0; e < R; ++e) {
        const int i = first + e;
        if (i < n && fj < 0) {
          sj = sj + __uint_as_float(bits[e]);
          if (sj > threshold) fj = i;
        }
      }
    }
    s = readlane_f32(sj, j);
    fj = static_cast<int>(readlane_u32(static_cast<uint32_t>(fj), j));
    if (fj >= 0) {
      found = fj;
      return;
    }
    consumed = j + 1;
  }
}

// One wavefront consumes its 64 runs of a plain sum (no threshold) from prefix sums prepared in
// advance: incl_a / incl_b are the inclusive scans of the lanes' increments rne(a / ulp) for the
// binades with biased exponents kb_a (the one s is expected to be in) and kb_b > kb_a (the one the
// slot is expected to end in); the caller has checked that no element ties under either ulp and
// that the last entry of incl_b is below 2^24 (so every entry of it is exact).  If s is in binade
// kb_a, the first lane whose prefix under A reaches the end of the binade adds its elements
// natively; if that lands in binade kb_b and the increments of the lanes behind it stay inside, s
// is the sum after the slot and 64 is returned.  Otherwise s is the exact sum in front of the
// returned lane (0 .. 63), and the caller continues there with wave_resolve().
template <int R>
__device__ __forceinline__ int resolve_prepared(float& s, const uint32_t (&bits)[R], float incl_a, float incl_b,
                                                uint32_t kb_a, uint32_t kb_b) {
  const int lane = threadIdx.x & 63;
  s = uniform_f32(s);
  const SumState ss = sum_state(s);
  if (static_cast<uint32_t>(ss.kb) != kb_a) return 0;
  const float room = static_cast<float>((1u << 24) - ss.S);
  const uint64_t ballot = __ballot(!(incl_a < room));
  if (!ballot) {
    s = sum_value(ss.S + static_cast<uint32_t>(readlane_f32(incl_a, 63)), ss.kb);
    return 64;
  }
  const int j = __ffsll(static_cast<long long>(ballot)) - 1;
  const float excl_a = lane_before_f32(incl_a);  // exact in lane j: every prefix in front of it is below `room`
  float sj = 0.0f;
  if (lane == j) {
    sj = sum_value(ss.S + static_cast<uint32_t>(excl_a), ss.kb);
#pragma unroll
    for (int e = 0; e < R; ++e) sj = sj + __uint_as_float(bits[e]);
  }
  s = readlane_f32(sj, j);
  const SumState s2 = sum_state(s);
  if (static_cast<uint32_t>(s2.kb) != kb_b) return j + 1;
  const float rest = readlane_f32(incl_b, 63) - readlane_f32(incl_b, j);
  const uint32_t S_end = s2.S + static_cast<uint32_t>(rest);
  if (S_end >= (1u << 24)) return j + 1;
  s = sum_value(S_end, s2.kb);
  return 64;
}

// First attempt at a group of U * 16 slots: fold every slot ONCE, with the ulp it is predicted to
// see, instead of once per binade the running sum passes through.
//   1. plain float sums per slot give approximate running sums at the slot boundaries;
//   2. a slot whose two boundaries lie safely inside one binade is "stable" and is folded with that
//      binade's ulp into a parity summary; the others (a binade boundary or the threshold inside
//      or within 2^-13 of an end -- plain and sequential sums of a group's 16384 entries differ by
//      random rounding, some 1e-5 of the sum -- or sums too small for the float shortcut) are
//      "serial";
//   3. the slots are consumed in order from the exact running sum: a run of stable slots by
//      composing its summaries -- after checking that the exact sum entering it has the predicted
//      exponent and that the run neither leaves the binade nor crosses the threshold, which is
//      all their validity needs -- and a serial slot by wave_resolve() in its own wave, one barrier
//      each.
// The predictions steer only which work is done; every committed step is exact.  Returns the
// number of slots consumed (st.s is the exact sum behind them): a failed check stops in front of
// the offending run, and the caller continues from there with the general rounds.  When the
// threshold is crossed st.stop_index is set and `stopped` is true.
// PLAIN: the threshold is known to be +inf at compile time (a plain sum).
template <int U, int R, bool PLAIN>
__device__ __forceinline__ int seq_sum_predicted(SeqSum& st, const uint32_t (&bits)[U][R], const int (&first)[U], int n, float threshold,
                                 bool& stopped, BlockScratch& sm) {
  if (PLAIN) threshold = __uint_as_float(0x7f800000u);
  stopped = false;
  static_assert(U * kWaves <= 32, "the serial-slot mask is 32 bits");
  constexpr int kSlots = U * kWaves;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const float kBig = 67108864.0f;
  // ---- 1
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float a = 0.0f;
#pragma unroll
    for (int e = 0; e < R; ++e) a += __uint_as_float(bits[u][e]);
    a = wave_sum_f32(a);
    if (lane == 0) sm.slot_sum[u * kWaves + wave] = a;
  }
  __syncthreads();
  // ---- 2 (every wave, one slot per lane)
  const float incl = wave_scan_inclusive_f32(lane < kSlots ? sm.slot_sum[lane] : 0.0f, lane);
  const float s_in = st.s + lane_before_f32(incl);
  const float s_out = st.s + incl;
  const uint32_t kb_in = __float_as_uint(s_in) >> 23, kb_out = __float_as_uint(s_out) >> 23;
  const float edge = __uint_as_float(kb_in << 23);  // 2^(kb_in - 127) <= s_in
  const bool serial = kb_in != kb_out || kb_in < 70u || kb_in > 250u || s_in < edge * 1.0001220703125f ||
                      s_out > edge * 1.999755859375f || (!PLAIN && !(s_out < threshold * 0.9998779296875f));
  const uint32_t serial_mask = static_cast<uint32_t>(__ballot(serial && lane < kSlots));
  const uint32_t buf = st.parity_buf;
  st.parity_buf ^= 1u;
  // A serial slot of a plain sum is prepared by its wave while the others fold theirs: prefix sums
  // of the lanes' increments with the ulp of the binade it is predicted to be entered in (A) and of
  // the one it is predicted to be left in (B).  With them, and no tie under either ulp, the slot
  // costs step 3 one comparison, the crossing lane's native adds and one subtraction instead of
  // two folds (see resolve_prepared).
  float prep_a[U], prep_b[U];
  uint32_t prep_kb_a[U], prep_kb_b[U];
  bool prepared[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int slot_index = u * kWaves + wave;
    ParityInc slot = {0u, 0u};
    prepared[u] = false;
    prep_a[u] = prep_b[u] = 0.0f;
    prep_kb_a[u] = prep_kb_b[u] = 0u;
    if (PLAIN && ((serial_mask >> slot_index) & 1u)) {
      const uint32_t kba = readlane_u32(kb_in, slot_index);
      const uint32_t kbo = readlane_u32(kb_out, slot_index);
      const uint32_t kbb = kbo > kba ? kbo : kba + 1u;
      if (kba >= 70u && kbb <= 250u) {
        const float scale_a = __uint_as_float((277u - kba) << 23), scale_b = __uint_as_float((277u - kbb) << 23);
        FastAcc fa = {0.0f, 0.0f}, fb = {0.0f, 0.0f};
#pragma unroll
        for (int e = 0; e < R; ++e) {
          fast_fold(fa, __uint_as_float(bits[u][e]), scale_a);
          fast_fold(fb, __uint_as_float(bits[u][e]), scale_b);
        }
        prep_a[u] = wave_scan_inclusive_f32(fa.inc, lane);
        prep_b[u] = wave_scan_inclusive_f32(fb.inc, lane);
        prep_kb_a[u] = kba;
        prep_kb_b[u] = kbb;
        prepared[u] = __ballot(fa.tie == 0.5f || fb.tie == 0.5f) == 0ull && readlane_f32(prep_b[u], 63) < 16777216.0f;
      }
    }
    if (!((serial_mask >> slot_index) & 1u)) {
      const uint32_t kb = readlane_u32(kb_in, slot_index);
      const float scale = __uint_as_float((277u - kb) << 23);  // 2^(150 - kb)
      FastAcc acc = {0.0f, 0.0f};
#pragma unroll
      for (int e = 0; e < R; ++e) fast_fold(acc, __uint_as_float(bits[u][e]), scale);
      if (__ballot(acc.tie == 0.5f) == 0ull) {
        const float inc = wave_sum_f32(acc.inc);
        const uint32_t v = inc < kBig ? static_cast<uint32_t>(inc) : kSat;
        slot.even = v;
        slot.odd = v;
      } else {
        const ParityInc upto = wave_scan_inclusive(fold_run<R>(bits[u], __uint_as_float(kb << 23)), lane);
        slot.even = readlane_u32(upto.even, 63);
        slot.odd = readlane_u32(upto.odd, 63);
      }
    }
    if (lane == 0) sm.wave_total[buf][slot_index] = slot;
  }
  __syncthreads();
  // ---- 3
  ParityInc mine = {0u, 0u};
  if (lane < kSlots) mine = sm.wave_total[buf][lane];
  // Without a tie in any stable slot (the usual case) a run's total is a difference of two plain
  // prefix sums (at most 32 summaries of at most 2^26 each: no overflow); serial slots hold 0.
  const bool no_ties = __ballot(mine.even != mine.odd) == 0ull;
  uint32_t plain_upto = mine.even;
  if (no_ties) {
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x111, 0xf, 0xf, false);
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x112, 0xf, 0xf, false);
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x114, 0xf, 0xf, false);
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x118, 0xf, 0xf, false);
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x142, 0xa, 0xf, false);
    plain_upto += __builtin_amdgcn_update_dpp(0u, plain_upto, 0x143, 0xc, 0xf, false);
  }
  float s = uniform_f32(st.s);
  int pos = 0;
  uint32_t hand = 0u;
  while (pos < kSlots) {
    const uint32_t ahead = serial_mask >> pos;
    const int next_serial = ahead ? pos + __ffs(static_cast<int>(ahead)) - 1 : kSlots;
    if (next_serial > pos) {
      const SumState ss = sum_state(s);
      if (static_cast<uint32_t>(ss.kb) != readlane_u32(kb_in, pos)) break;  // not the predicted binade
      uint32_t total;
      if (no_ties) {
        total = readlane_u32(plain_upto, next_serial - 1) - (pos ? readlane_u32(plain_upto, pos - 1) : 0u);
      } else {
        ParityInc in_run = {0u, 0u};
        if (lane >= pos && lane < next_serial) in_run = mine;
        const ParityInc upto = wave_scan_inclusive(in_run, lane);
        total = (ss.S & 1u) ? readlane_u32(upto.odd, 63) : readlane_u32(upto.even, 63);
      }
      if (ss.S + total >= (1u << 24)) break;  // the run would leave the binade
      const float s_run = sum_value(ss.S + total, ss.kb);
      if (!PLAIN && s_run > threshold) break;  // the crossing lies inside the run after all
      s = s_run;
      pos = next_serial;
    }
    if (pos == kSlots) break;
    if (wave == pos % kWaves) {
      const int ustar = pos / kWaves;
      float sw = s;
      int found = -1;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (u == ustar) {
          int from = 0;
          if (PLAIN && prepared[u]) from = resolve_prepared<R>(sw, bits[u], prep_a[u], prep_b[u], prep_kb_a[u], prep_kb_b[u]);
          if (from < 64) wave_resolve<R>(sw, found, bits[u], first[u], n, threshold, from);
        }
      }
      if (lane == 0) {
        sm.chain_s[hand] = sw;
        if (!PLAIN) sm.chain_found[hand] = found;
      }
    }
    __syncthreads();
    s = uniform_f32(sm.chain_s[hand]);
    const int found = PLAIN ? -1 : sm.chain_found[hand];
    hand ^= 1u;
    if (found >= 0) {
      st.s = s;
      st.stop_index = found;
      stopped = true;
      return pos;
    }
    ++pos;
  }
  st.s = s;
  return pos;
}

// Consumes U chunks: in chunk u lane `tid` owns elements first[u] .. first[u] + R - 1 (global
// positions; chunks in increasing position, lanes in order inside a chunk), given as float bit
// patterns in bits[u][] (finite, >= 0; positions >= n must hold 0).
// Emulates  for each element: s += a; if (s > threshold) stop  in fp32, bit for bit.
// The U * 16 (chunk, wave) runs are "slots" in position order.  Each round composes the slots'
// parity summaries in order and finds the first slot in which the running sum leaves its binade or
// crosses the threshold; the slots in front of it are committed, its wave resolves its own 64 runs
// with wave_resolve(), and the next round restarts behind it with the new ulp.  Two barriers per
// round, one when nothing happens.  Must be called by all lanes; returns true when the
// threshold was crossed (st.stop_index set).
template <int U, int R>
__device__ __forceinline__ bool seq_sum_rounds(SeqSum& st, const uint32_t (&bits)[U][R], const int (&first)[U], int n, float threshold,
                               BlockScratch& sm, int resume = 0) {
  static_assert(U * kWaves <= 64, "one lane per slot in the cross-wave scan");
  constexpr int kSlots = U * kWaves;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float kBig = 67108864.0f;  // 2^26 marks a slot that must be resolved (tie inside)
  // slots below `resume` have been consumed
  while (true) {
    const float scale = fast_scale(st.s);
    const SumState ss = sum_state(st.s);
    const uint32_t buf = st.parity_buf;
    st.parity_buf ^= 1u;
    int star;
    uint32_t S_front, S_all;
    // Every pending slot is summarised as a parity pair.  Without a half-ulp tie among its
    // elements both entries are the float-summed increment; a slot with ties takes the
    // two-hypothesis fold, so ties cost no round of their own.
#pragma unroll
    for (int u = 0; u < U; ++u) {
      ParityInc slot = {0u, 0u};
      if (u * kWaves + wave >= resume) {
        bool by_parity = scale == 0.0f;
        if (!by_parity) {
          FastAcc acc = {0.0f, 0.0f};
#pragma unroll
          for (int e = 0; e < R; ++e) fast_fold(acc, __uint_as_float(bits[u][e]), scale);
          by_parity = __ballot(acc.tie == 0.5f) != 0ull;
          if (!by_parity) {
            const float inc = wave_sum_f32(acc.inc);
            const uint32_t v = inc < kBig ? static_cast<uint32_t>(inc) : kSat;
            slot.even = v;
            slot.odd = v;
          }
        }
        if (by_parity) {
          const ParityInc incl = wave_scan_inclusive(fold_run<R>(bits[u], st.s), lane);
          slot.even = readlane_u32(incl.even, 63);
          slot.odd = readlane_u32(incl.odd, 63);
        }
      }
      if (lane == 0) sm.wave_total[buf][u * kWaves + wave] = slot;
    }
    __syncthreads();
    {
      // every wave redoes the small scan over the slot summaries in its first lanes
      ParityInc wt = {0u, 0u};
      if (lane < kSlots) wt = sm.wave_total[buf][lane];
      const ParityInc upto = wave_scan_inclusive(wt, lane);
      const bool odd = ss.S & 1u;
      const uint32_t S_upto = ss.S + (odd ? upto.odd : upto.even);
      bool event = S_upto >= (1u << 24);
      if (!event) event = sum_value(S_upto, ss.kb) > threshold;
      const uint64_t ballot = __ballot(event && lane < kSlots);
      star = next_event(ballot, resume, kSlots);  // never a slot that has been consumed: the rounds end
      S_front = star > 0 && star < kSlots ? readlane_u32(S_upto, star - 1) : ss.S;
      S_all = readlane_u32(S_upto, kSlots - 1);
    }
    if (star == kSlots) {
      st.s = sum_value(S_all, ss.kb);
      return false;
    }
    if (wave == star % kWaves) {
      const int ustar = star / kWaves;
      float s = sum_value(S_front, ss.kb);
      int found = -1;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (u == ustar) wave_resolve<R>(s, found, bits[u], first[u], n, threshold);
      }
      if (lane == 0) {
        sm.bc_sum = s;
        sm.bc_found = found;
      }
    }
    __syncthreads();
    st.s = sm.bc_sum;
    const int found = sm.bc_found;
    if (found >= 0) {
      st.stop_index = found;
      return true;
    }
    resume = star + 1;
  }
}

// Single-chunk form.
template <int R>
__device__ __forceinline__ bool seq_sum_chunk(SeqSum& st, const uint32_t (&bits)[R], int first, int n, float threshold,
                                              BlockScratch& sm) {
  uint32_t b[1][R];
#pragma unroll
  for (int e = 0; e < R; ++e) b[0][e] = bits[e];
  const int f[1] = {first};
  bool stopped = false;
  const int consumed = seq_sum_predicted<1, R, false>(st, b, f, n, threshold, stopped, sm);
  if (stopped) return true;
  if (consumed == kWaves) return false;
  return seq_sum_rounds<1, R>(st, b, f, n, threshold, sm, consumed);
}

// Consumes U chunks (chunk u: lane `tid` owns elements first[u] .. first[u] + R - 1, chunks in
// increasing position) with ONE barrier when all of them stay inside the binade of s, below the
// threshold and free of ties; `acc[u]` must have been folded over chunk u's elements with
// scale = fast_scale(st.s).
// A plain sum that leaves the binade in exactly one place of the group, again without ties, takes
// three barriers: the slots' increments under the old ulp are exact, so their prefix sums name
// the slot the sum leaves the binade in and the exact sum entering it; that slot's wave finds the
// lane the same way from its lanes' increments and lets it add its elements natively; every wave
// then folds what lies behind that lane with the ulp of the new sum, and the totals are added after
// checking that they hold no tie and stay inside the new binade.  Everything else (ties, a second
// change of binade, sums too small for float increments, threshold walks) goes through the
// predicted pass and the general rounds, from the sum the group was entered with.
template <int U, int R, bool PLAIN = false>
__device__ __forceinline__ bool seq_sum_group(SeqSum& st, const uint32_t (&bits)[U][R], const FastAcc (&acc)[U], float scale,
                              const int (&first)[U], int n, float threshold, BlockScratch& sm) {
  static_assert(U <= 2, "slot_total holds two chunks");
  if (PLAIN) threshold = __uint_as_float(0x7f800000u);  // a plain sum: the compiler drops the comparisons
  constexpr int kSlots = U * kWaves;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const float kBig = 67108864.0f;  // 2^26: "take the ordered path"
  bool slot_has_tie[U];
  bool wave_has_tie = false;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    slot_has_tie[u] = __ballot(acc[u].tie == 0.5f) != 0ull;
    wave_has_tie = wave_has_tie || slot_has_tie[u];
  }
  // (a threshold walk leaves every tie to the ordered paths; a plain sum corrects for them below)
  const bool ordered = scale == 0.0f || (!PLAIN && wave_has_tie);
  float inc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    inc[u] = wave_sum_f32(acc[u].inc);
    if (ordered || !(inc[u] < kBig)) inc[u] = kBig;
  }
  const uint32_t buf = st.parity_buf;
  st.parity_buf ^= 1u;
  if (lane == 0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      sm.slot_total[buf][u * kWaves + wave] = inc[u];
      if (PLAIN) sm.slot_tie[buf][u * kWaves + wave] = slot_has_tie[u] ? 1u : 0u;
    }
  }
  __syncthreads();
  const float mine = lane < kSlots ? sm.slot_total[buf][lane] : 0.0f;
  float upto = wave_scan_inclusive_f32(mine, lane);  // exact wherever it is below 2^24
  const float s_in = uniform_f32(st.s);
  const SumState ss = sum_state(s_in);
  const float room = static_cast<float>((1u << 24) - ss.S);
  const bool any_big = __ballot(mine >= kBig) != 0ull;
  uint32_t tie_slots = 0u;
  if (PLAIN) tie_slots = static_cast<uint32_t>(__ballot(lane < kSlots && sm.slot_tie[buf][lane] != 0u));
  float lane_fix[U];  // what this lane's ties add to its increments of chunk u (0 without ties)
#pragma unroll
  for (int u = 0; u < U; ++u) lane_fix[u] = 0.0f;
  const bool with_ties = PLAIN && tie_slots != 0u && !any_big;
  if (with_ties) {
    // ---- half-ulp ties in a plain sum.  The totals above count rint(t) for a tie t = n0 + 1/2, the
    // even one of its neighbours; the sequential sum adds n0 or n0 + 1, whichever makes the running
    // integer even: the same when the integer in front of the tie is even, the other neighbour
    // (+1 for even n0, -1 for odd n0) when it is odd.  Write a_i for the parity of the PROVISIONAL
    // integer in front of the i-th tie of the group (entering integer plus the counted increments
    // of everything before it) and x_i for the parity of the true one.  Every earlier correction is
    // odd exactly when its own x is, so x_i = a_i ^ x_1 ^ .. ^ x_(i-1), hence x_1 ^ .. ^ x_i = a_i
    // and x_i = a_i ^ a_(i-1): a tie needs the provisional parity in front of itself and in front
    // of the tie before it, nothing else.  A wave works out the ties of its slots, for both values
    // the a of the last tie of an earlier slot can have; after one more barrier everybody chains
    // the slots.  (All of this is exact up to the place where the sum leaves the binade, which is all
    // that is used of it.)
    int d0[U], d1[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      d0[u] = 0;
      d1[u] = 0;
      if (slot_has_tie[u]) {  // wave-uniform
        const int slot = u * kWaves + wave;
        const uint32_t entering = ss.S + static_cast<uint32_t>(readlane_f32(lane_before_f32(upto), slot));
        const uint32_t own = static_cast<uint32_t>(__builtin_fminf(acc[u].inc, kBig));
        uint32_t parity = (entering + wave_scan_inclusive_u32(own) - own) & 1u;  // in front of the lane's first element
        uint32_t has = 0u, a_first = 0u, a_last = 0u, odd_first = 0u;
        int rest = 0;  // corrections of the lane's ties after its first
#pragma unroll
        for (int e = 0; e < R; ++e) {
          const float t = __uint_as_float(bits[u][e]) * scale;
          const float r = __builtin_rintf(t);
          if (__builtin_fabsf(t - r) == 0.5f) {  // (then t < 2^23)
            const uint32_t odd = static_cast<uint32_t>(__builtin_floorf(t)) & 1u;
            if (has) {
              rest += (parity ^ a_last) ? 1 - 2 * static_cast<int>(odd) : 0;
            } else {
              has = 1u;
              a_first = parity;
              odd_first = odd;
            }
            a_last = parity;
          }
          parity ^= r < 16777216.0f ? (static_cast<uint32_t>(r) & 1u) : 0u;
        }
        const uint64_t has_mask = __ballot(has != 0u);
        const uint64_t last_mask = __ballot(has != 0u && a_last != 0u);
        if (has) {
          const uint64_t below = has_mask & ((1ull << lane) - 1ull);
          const int step = 1 - 2 * static_cast<int>(odd_first);
          if (below) {
            const uint32_t before = static_cast<uint32_t>(last_mask >> (63 - __clzll(static_cast<long long>(below)))) & 1u;
            d0[u] = d1[u] = rest + ((a_first ^ before) ? step : 0);
          } else {  // the slot's first tie: its predecessor is in an earlier slot, or there is none (a = 0)
            d0[u] = rest + (a_first ? step : 0);
            d1[u] = rest + (a_first ? 0 : step);
          }
        }
        const uint32_t D0 = wave_sum_u32(static_cast<uint32_t>(d0[u])) + 1024u;  // |D| <= 512
        const uint32_t D1 = wave_sum_u32(static_cast<uint32_t>(d1[u])) + 1024u;
        const uint32_t slot_last = static_cast<uint32_t>(last_mask >> (63 - __clzll(static_cast<long long>(has_mask)))) & 1u;
        if (lane == 0) sm.tie_fix[slot] = (D0 & 0xfffu) | ((D1 & 0xfffu) << 12) | (slot_last << 24);
      }
    }
    __syncthreads();
    const uint32_t my_fix = (lane < kSlots && ((tie_slots >> lane) & 1u)) ? sm.tie_fix[lane] : 0u;
    uint32_t before = 0u;  // a of the last tie so far
    int shift = 0;         // what the ties up to this lane's slot add
    uint32_t pending = tie_slots;
    while (pending) {  // uniform
      const int t = __ffs(static_cast<int>(pending)) - 1;
      pending &= pending - 1u;
      const uint32_t f = readlane_u32(my_fix, t);
      const int D = static_cast<int>((before ? (f >> 12) : f) & 0xfffu) - 1024;
      if (lane >= t) shift += D;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (t == u * kWaves + wave) lane_fix[u] = static_cast<float>(before ? d1[u] : d0[u]);
      }
      before = (f >> 24) & 1u;
    }
    upto += static_cast<float>(shift);
  }
  const bool countable = !any_big && (tie_slots == 0u || with_ties);  // `upto` holds the true prefix sums
  const uint64_t leaves = __ballot(lane < kSlots && !(upto < room));
  if (countable && !leaves) {  // stays inside the binade
    const float s_new = sum_value(ss.S + static_cast<uint32_t>(readlane_f32(upto, kSlots - 1)), ss.kb);
    if (!(s_new > threshold)) {
      st.s = s_new;
      return false;
    }
  }
  if (PLAIN && countable && leaves) {
    const int c = __ffsll(static_cast<long long>(leaves)) - 1;  // the slot the sum leaves the binade in
    const uint32_t S_c = ss.S + static_cast<uint32_t>(readlane_f32(lane_before_f32(upto), c));
    int j = 64;  // (in the slot's wave) the lane that added natively
    if (wave == c % kWaves) {
      float own = 0.0f;
#pragma unroll
      for (int u = 0; u < U; ++u) own = (u == c / kWaves) ? acc[u].inc + lane_fix[u] : own;
      const float lanes_upto = wave_scan_inclusive_f32(own, lane);
      const float room_c = static_cast<float>((1u << 24) - S_c);
      const uint64_t over = __ballot(!(lanes_upto < room_c));  // not empty: the slot's total is not below room_c
      j = __ffsll(static_cast<long long>(over)) - 1;
      const float before = lane_before_f32(lanes_upto);
      float sj = 0.0f;
      if (lane == j) {
        sj = sum_value(S_c + static_cast<uint32_t>(before), ss.kb);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u == c / kWaves) {
#pragma unroll
            for (int e = 0; e < R; ++e) sj = sj + __uint_as_float(bits[u][e]);  // (entries past n hold 0)
          }
        }
      }
      if (lane == 0) {
        sm.bc_sum = readlane_f32(sj, over ? j : 0);
        sm.bc_found = over ? 1 : 0;  // (always 1: the slot's total, the last of these prefix sums, is not below room_c)
      }
    }
    __syncthreads();
    const float s_mid = uniform_f32(sm.bc_sum);  // the exact sum behind lane j of slot c
    const SumState sb = sum_state(s_mid);
    const bool usable = sm.bc_found != 0 && sb.kb >= 64 && sb.kb < 250;
    if (usable) {
      const float scale_b = __uint_as_float(static_cast<uint32_t>(277 - sb.kb) << 23);  // 2^(150 - kb)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int slot = u * kWaves + wave;
        float v = 0.0f;
        if (slot >= c) {  // wave-uniform
          FastAcc fb = {0.0f, 0.0f};
          if (slot > c || lane > j) {
#pragma unroll
            for (int e = 0; e < R; ++e) fast_fold(fb, __uint_as_float(bits[u][e]), scale_b);
          }
          v = wave_sum_f32(fb.inc);
          if (__ballot(fb.tie == 0.5f) != 0ull || !(v < kBig)) v = kBig;
        }
        if (lane == 0) sm.slot_total[buf ^ 1u][slot] = v;
      }
    }
    __syncthreads();
    if (usable) {
      const float behind = lane < kSlots ? sm.slot_total[buf ^ 1u][lane] : 0.0f;
      if (__ballot(behind >= kBig) == 0ull) {
        const float total = wave_sum_f32(behind);
        if (total < static_cast<float>((1u << 24) - sb.S)) {
          st.s = sum_value(sb.S + static_cast<uint32_t>(total), sb.kb);
          st.parity_buf ^= 1u;  // the next group writes the half that was read before the last two barriers
          return false;
        }
      }
    }
    __syncthreads();  // the ordered paths below reuse bc_sum
  }
  int consumed = 0;
  if (U * kWaves <= 32) {
    bool stopped = false;
    consumed = seq_sum_predicted<U, R, PLAIN>(st, bits, first, n, threshold, stopped, sm);
    if (stopped) return true;
    if (consumed == U * kWaves) return false;
  }
  return seq_sum_rounds<U, R>(st, bits, first, n, threshold, sm, consumed);
}

// Whole-array form:  s = s0; for (i < n) { s += a(i); if (s > threshold) return {s, i}; }
// with lane `tid` owning R consecutive elements per chunk.  `a(i)` must return a finite,
// non-negative float; pass threshold = +inf to sum everything.  Must be called by every lane.
template <int R, typename Fetch>
__device__ SeqSumResult seq_sum_block(Fetch a, int n, float s0, float threshold, BlockScratch& sm) {
  SeqSum st = {s0, -1, 0u};
  for (int base = 0; base < n; base += kBlock * R) {
    uint32_t bits[R];
    const int first = base + static_cast<int>(threadIdx.x) * R;
#pragma unroll
    for (int e = 0; e < R; ++e) bits[e] = (first + e < n) ? __float_as_uint(a(first + e)) : 0u;
    if (seq_sum_chunk<R>(st, bits, first, n, threshold, sm)) break;
  }
  __syncthreads();  // callers reuse the scratch right away
  return {st.s, st.stop_index};
}

}  // namespace ets
