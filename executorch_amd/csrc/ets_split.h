// The stochastic path with every row spread over several workgroups: three launches.
//
//   split_pass1_kernel   (HBM read) per slot of 512 entries: the maximum of x = logit * inv_temperature
//                        and an approximate sum of exp(x - slot maximum)
//   split_pass2_kernel   (re-read, L2 / Infinity Cache) exact e = expf(x - row maximum) per entry; from
//                        the approximate running sums every slot learns the binade the sequential
//                        softmax sum will be in when it reaches the slot and folds its entries ONCE,
//                        with that binade's ulp, into a parity summary (ets_seqsum_math.h); slots that
//                        cannot be placed inside one binade keep their entries and prefix sums under
//                        the two candidate ulps instead; top-p candidates are listed
//   split_finish_kernel  one workgroup per row: composes the summaries in index order from the exact
//                        running sum, checks every prediction exactly, resolves the few slots in which
//                        the sum changes binade entry by entry, then draws the coin and the token
//
// Passes 1 and 2 hold no step that depends on another slot, so any number of workgroups share a
// row; what is inherently ordered (sampler.cpp:199-203 adds the entries one after the other) is
// reduced to one wave walking a few hundred 16-byte records.  Predictions only select the work:
// every value that reaches the result has been verified against the exact running sum.
#pragma once

#include "ets_kernels.h"

namespace ets {

// Phase clocks inside the kernels (device wall-clock reads around the phases of pass 2, of the
// finish kernel and of the chain) exist only in a profiling build: -DETS_PHASE_CLOCKS=1.
#ifndef ETS_PHASE_CLOCKS
#define ETS_PHASE_CLOCKS 0
#endif

constexpr int kSlot = 512;        // entries per slot: 64 lanes x 8 consecutive entries
constexpr int kMaxSlots = 2048;   // rows of up to 1048576 entries take this path
constexpr int kPrepCap = 40;      // prepared slots per row (a row of the usual kind needs 10 to 20)

constexpr uint32_t kSlotStable = 0u;  // even / odd hold the slot's parity summary for binade `kb`
constexpr uint32_t kSlotZero = 1u;    // every entry is 0: adds nothing whatever the running sum
constexpr uint32_t kSlotSerial = 2u;  // to be resolved in order (prepared data at index `prep`, if any)
constexpr uint32_t kSlotDual = 3u;    // no entry ties under the ulp of binade kb or of kb + 1: `even` is the slot's
                                      //   increment for a sum that passes it inside binade kb, `odd` inside kb + 1
constexpr uint32_t kSlotExact = 4u;   // slot 0 only: `even` holds the bits of the exact sum behind the slot

struct SlotRec {
  uint32_t meta;  // bits 0-7: biased exponent the summary was folded for; bits 8-10: kind; bits 16-23: the biased
                  //   exponent the sum is predicted to have when it reaches the slot (a serial slot: behind the
                  //   slot); serial slots, bit 24: "prepared, both binades in the range of the float shortcut" (the
                  //   chain's short form can serve it)
  uint32_t even, odd;
  uint32_t prep;  // index of the slot's PrepSlot, or 0xffffffff
};

// What pass 2 keeps of a slot that is resolved in order: its entries and the inclusive prefix sums
// over the lanes of the increments rne(e / ulp) of each lane's 8 entries, under the ulp of the
// binade the running sum is expected to enter the slot in (a) and of the one it is expected to
// leave it in (b), with the lanes in which an entry sits on a half-ulp tie (their increment
// depends on the order of the adds).  A lane's increment is capped at 2^24 (at least what any
// binade has room for), so the sums are exact integers wherever they matter and never wrap.
struct PrepSlot {
  float e[kSlot];
  uint32_t pre_a[64];
  uint32_t pre_b[64];
  uint32_t kb_a, kb_b;
  uint32_t tie_a_lo, tie_a_hi, tie_b_lo, tie_b_hi;
  uint32_t usable;  // both binades are in the range of the float shortcut
  uint32_t pad;
};
constexpr uint32_t kPrepTie = 0x80000000u;   // bit 31 of pre_a[l] / pre_b[l]: an entry of lane l ties under that binade's ulp
constexpr uint32_t kPrepSum = 0x7fffffffu;   //   (the prefix sums stay below 2^31: 64 lanes of at most 2^24)
static_assert(sizeof(PrepSlot) % 16 == 0, "prepared slots are copied as 16-byte vectors");

struct RowState {
  uint32_t prep_count;  // slots that pass 2 set aside to be resolved in order (may exceed the capacity)
  float m;              // row maximum of x (NaN when x[0] is NaN, like the reference's loop)
  uint32_t nan;         // some expf(x - m) is NaN
  float a_total;        // approximate softmax sum, in units of exp(-m)
  int32_t key_cut;      // 16-bit rows: order key of the first bin of the pattern histogram,
  int32_t n_bins;       //   how many bins it has (0: no pattern histogram)
  int32_t mag_min;      //   and the KeyMap's first magnitude with a key of its own
  uint32_t listed_buckets;  // 0: every possible candidate is listed; else only those of the histogram's
                            //   first `listed_buckets` buckets (which carry more than topp of the mass, or,
                            //   for a top-k row, hold at least topk entries); kNoLists: nothing usable is listed
};
constexpr uint32_t kNoLists = 0xffffffffu;

constexpr int kMaxRowWorkgroups = 64;  // workgroups of pass 2 per row
constexpr int kListRegion = 16384;     // candidates one workgroup of pass 2 can list

// Histogram of a row's candidates by the size of exp: 64 buckets per binade, from 1 downwards.
// Bucket b holds exp bit patterns in (0x3F800000 - (b + 1) * 2^17, 0x3F800000 - b * 2^17]; the last
// bucket also takes everything below.
constexpr int kHistBuckets = 2048;
__device__ __forceinline__ uint32_t hist_bucket(uint32_t e_bits) {
  const uint32_t b = (0x3F800000u - e_bits) >> 17;  // (exp <= 1)
  return b < static_cast<uint32_t>(kHistBuckets - 1) ? b : static_cast<uint32_t>(kHistBuckets - 1);
}
// Every exp in buckets 0 .. b - 1 is above hist_edge(b); every one in buckets b .. is at most that.
__device__ __forceinline__ float hist_edge(int b) {
  return b >= kHistBuckets ? 0.0f : __uint_as_float(0x3F800000u - (static_cast<uint32_t>(b) << 17));
}

// Order key of a 16-bit float pattern (fp16 or bf16): a larger value has a larger key.  Magnitudes
// below `mag_min` are so small that x = logit * inv_temperature vanishes against the row maximum
// (|x| under an eighth of its ulp), so all of them give the same exp as a logit of 0: they share one
// key per sign, which keeps the range of keys of a row short.  -0 sits just below +0.
struct KeyMap {
  int mag_min;  // first magnitude pattern with a key of its own
  int key_cut;  // key of the pattern histogram's first bin
  int n_bins;   // 0: no pattern histogram
};
__device__ __forceinline__ int pattern_key(uint32_t pattern16, int mag_min) {
  const int mag = static_cast<int>(pattern16 & 0x7fffu);
  const int cm = mag < mag_min ? 0 : mag - mag_min + 1;
  return (pattern16 & 0x8000u) ? 0x7fff - cm : 0x8000 + cm;
}
// A pattern with that key (the zero of its sign for the shared keys).
__device__ __forceinline__ uint32_t key_pattern(int key, int mag_min) {
  const int cm = key >= 0x8000 ? key - 0x8000 : 0x7fff - key;
  const uint32_t mag = cm == 0 ? 0u : static_cast<uint32_t>(cm - 1 + mag_min);
  return (key >= 0x8000 ? 0u : 0x8000u) | (mag & 0x7fffu);
}
template <int DT>
__device__ __forceinline__ float pattern_value(uint32_t pattern16) {
  return DT == kDtypeBFloat16 ? __uint_as_float(pattern16 << 16) : half_bits_to_float(pattern16);
}
// The 16-bit pattern of a value that was converted from one (exactly).
template <int DT>
__device__ __forceinline__ uint32_t value_pattern(float v) {
  if (DT == kDtypeBFloat16) return __float_as_uint(v) >> 16;
  union {
    _Float16 f;
    uint16_t u;
  } cvt;
  cvt.f = static_cast<_Float16>(v);
  return cvt.u;
}

struct SplitParams {
  RowParams row;        // what the one-workgroup kernel takes
  float* slot_max;      // [rows, ns_stride] largest x = logit * inv_temperature of the slot (NaN: the slot holds one)
  float* slot_max2;     // [rows, ns_stride] largest x among the other 63 lanes' entries
  float* slot_sum;      // [rows, ns_stride] sum of exp(x - slot_max), approximate
  float4* slot_pack;    // [rows, ns_stride] (slot_max, slot_max2, slot_sum, -) of a launch with pass 1 inside pass 2
  SlotRec* slot_rec;    // [rows, ns_stride]
  PrepSlot* prep;       // [rows, prep_cap]
  RowState* row_state;  // [rows]
  uint64_t* list;       // [rows, row_wgs, list_region] (exp bits << 32 | index) of possible top-p
                        //   candidates: every workgroup of pass 2 fills its own region
  uint32_t* list_count; // [rows, kMaxRowWorkgroups] candidates each workgroup found (may exceed its region)
  uint32_t* hist;       // [rows, row_wgs, kHistBuckets] the same candidates by size
  uint32_t* phist;      // [rows, row_wgs, phist_words] 16-bit rows: entries per bit pattern, two 16-bit
                        //   counters per word, from order key RowState::key_cut upwards
  int32_t phist_words;  // words per (row, workgroup) region; 0 disables the pattern histogram
  float2* walk;         // [rows] multinomial rows: the exact softmax sum and the coin, between the two chains
  uint32_t* arrive;     // the fused launch: word 0 numbers the launches on these buffers (the finish kernel adds one; see
                        //   coherent_store4)
  int32_t spin_limit;   // the fused launch: reads of the row's slot values after which a workgroup stops waiting for the others
  uint64_t* timers;     // phase clocks (profiling), or null
  int32_t list_region;  // entries per region
  int32_t short_lists;  // 1: pass 2 may list only the largest candidates of a peaked row (see RowState::listed_buckets)
  int32_t chain_rows;   // the looping finish kernel: rows a workgroup takes at a time (1 .. kChainRows); their sums are
                        //   composed side by side, one wave each
  int32_t row_wgs;      // workgroups of pass 2 per row
  int32_t ns;           // slots per row
  int32_t ns_stride;
  int32_t prep_cap;
};

// Relative distance between the exact sequential sum after i entries and the approximate sum of
// pass 1: every add rounds by at most half an ulp of a running sum that never decreases, so the
// sequential sum is within i * 2^-24 of the mathematical one; pass 1's exponentials and float
// additions are within 1e-4 of it.
__device__ __forceinline__ float split_eps(int entries) {
  return static_cast<float>(entries) * (1.02f / 16777216.0f) + 2e-4f;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr float kLog2e = 1.44269504088896340736f;

// The 8 entries of lane `lane` of slot `s` as floats; positions past the row read as `fill`.
template <int DT>
__device__ __forceinline__ void load_slot_lane(const char* logits, int s, int lane, int V, float fill, float* out,
                                               const FusedOps& f) {
  constexpr int VE = VecElems<DT>::value;
  const int first = s * kSlot + lane * 8;
  if ((s + 1) * kSlot <= V) {  // (the same for every lane) a slot inside the row: no position is tested
#pragma unroll
    for (int q = 0; q < 8 / VE; ++q) {
      const uint4 raw = *reinterpret_cast<const uint4*>(logits + static_cast<int64_t>(first + q * VE) * ElemSize<DT>::value);
      decode_vec<DT>(raw, out + q * VE);
    }
  } else {
#pragma unroll
    for (int q = 0; q < 8 / VE; ++q) load_run<DT, true>(logits, first + q * VE, V, fill, out + q * VE);
  }
  if (f.n > 0) {
    apply_fused<DT, 8>(out, f);
    if (first + 8 > V) {
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = first + e < V ? out[e] : fill;
    }
  }
}

// ---- pass 1 ---------------------------------------------------------------------------------------
// Slots of a row that workgroup x of `wgs` takes, in passes 1 and 2 alike: the two launches have
// the same grid, so a workgroup of pass 2 runs on the die (XCD) whose L2 already holds the entries
// its namesake of pass 1 read from HBM (workgroups go to the dies in turn, by their linear id).
__device__ __forceinline__ void split_range(int ns, int wgs, int x, int& s_begin, int& s_end) {
  const int per_wg = ((ns + wgs - 1) / wgs + kWaves - 1) / kWaves * kWaves;
  s_begin = x * per_wg;
  s_end = min(ns, s_begin + per_wg);
}

// Pass 1 for one slot, by one wave: `v` are the lane's 8 entries (logits; products with an
// infinite inv_temperature when `inv_u` is 1 for that reason).  Stores the slot's maximum of
// x = logit * inv_temperature (NaN when the slot holds one), the largest x of the other 63 lanes and
// the approximate sum of exp(x - slot maximum).
// Few instructions per entry (with a workgroup per row the kernel would otherwise be bound by
// them, not by HBM): the maximum is taken over the raw logits -- rounding is monotone, so the
// largest product l * inv is the product of the largest (smallest, for a negative inv) logit --
// and the exponent comes from one fused multiply-add per entry.
// COHERENT: the three values are read by other workgroups of the same launch (the fused kernel): they
// are stored with device-scope accesses that go through to memory, one by one, so that no workgroup
// has to write its die's whole L2 back (a release fence does, and costs microseconds per workgroup
// when every workgroup of a die issues one).
__device__ __forceinline__ void coherent_store(float* ptr, float v) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(ptr), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* ptr) {
  return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(ptr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// The same for a slot's three values at once: one 16-byte request through to memory instead of three
// of four bytes (every such store is charged a partial line behind L2).  The compiler does not count
// these accesses: the load waits for its own result, the stores are waited for where the others are.
typedef float ets_f32x4 __attribute__((ext_vector_type(4)));
// The fourth word is a tag by which the reader knows the three values of THIS launch from whatever the
// sixteen bytes held before: the launch's number (SplitParams::arrive[0] + 1, which the finish kernel
// advances, so no two launches on the same buffers share one) mixed with the values themselves.  A record
// of an earlier launch never carries this launch's tag, whatever its values; a record that is not there yet
// reads as that earlier record (or as the zeros the buffer starts with, whose tag would be 0 + the mix of
// zeros = 0, which no launch uses: next_launch_number).  The sixteen bytes travel as one request; were a read ever to see part
// of a store, the mix of the values would have to make up for the difference between two tags.
// The next launch's number, by the one thread of a launch that advances it.  The word never holds 2^32 - 1, so
// that no launch has the number 0, for which the zeros that the records start as would pass for a record.
// (After 2^32 - 1 launches on the same buffers the numbers come round.)
__device__ __forceinline__ void next_launch_number(uint32_t* word) {
  const uint32_t v = *word + 1u;
  *word = v == 0xffffffffu ? 0u : v;
}
__device__ __forceinline__ uint32_t pack_tag(uint32_t launch, float a, float b, float c) {
  const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b), uc = __float_as_uint(c);
  return launch ^ (ua * 0x9E3779B1u) ^ ((ub << 13) | (ub >> 19)) ^ (((uc << 7) | (uc >> 25)) * 0x85EBCA77u);
}
__device__ __forceinline__ void coherent_store4(float4* ptr, float a, float b, float c, uint32_t launch) {
  const ets_f32x4 v = {a, b, c, __uint_as_float(pack_tag(launch, a, b, c))};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ ets_f32x4 coherent_load4(const float4* ptr) {
  ets_f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(ptr) : "memory");
  return v;
}
// Four of them requested together (one trip to memory for a wave that reads four slots per lane).
__device__ __forceinline__ void coherent_load4x4(const float4* p0, const float4* p1, const float4* p2, const float4* p3,
                                                 ets_f32x4& v0, ets_f32x4& v1, ets_f32x4& v2, ets_f32x4& v3) {
  asm volatile(
      "global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %5, off sc1\n\t"
      "global_load_dwordx4 %2, %6, off sc1\n\tglobal_load_dwordx4 %3, %7, off sc1\n\ts_waitcnt vmcnt(0)"
      : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
      : "memory");
}
struct SlotMax {
  float M, M2;  // the slot's largest x = logit * inv_temperature (NaN entries ignored), and the largest of the other 63 lanes
};
__device__ __forceinline__ SlotMax split_pass1_max(const float (&v)[8], float inv_u) {
  const int lane = threadIdx.x & 63;
  const float kInf = __uint_as_float(0x7f800000u);
  float ext = inv_u < 0.0f ? kInf : -kInf;
  if (inv_u < 0.0f) {
#pragma unroll
    for (int e = 0; e < 8; ++e) ext = __builtin_fminf(ext, v[e]);  // ignores NaN
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) ext = __builtin_fmaxf(ext, v[e]);
  }
  // (a lane whose entries all lie past the row's end holds the fill value, whose product is -inf)
  // (reduced as integer keys: one instruction per step.  A NaN product -- the row is one then --
  // may come out as the maximum: the slot's maximum is stored as NaN in that case anyway.)
  const uint32_t xk = float_max_key(ext * inv_u);
  const uint32_t Mk = wave_max_u32(xk);
  // the largest entry of the other lanes (pass 2 bounds the mass of the row's largest entries
  // from below with the two)
  const uint64_t holds = __ballot(xk == Mk);
  const int holder = __ffsll(static_cast<long long>(holds)) - 1;  // (some lane holds the maximum)
  return {float_of_max_key(Mk), float_of_max_key(wave_max_u32(lane == holder ? float_max_key(-kInf) : xk))};
}
// COHERENT: the three values as one tagged record for the other workgroups of the launch (coherent_store4);
// PLAIN_TOO: and in the three arrays as well, for a later launch that reads them there.
template <bool COHERENT = false, bool PLAIN_TOO = false>
__device__ __forceinline__ void split_pass1_sum(const SplitParams& p, int row, int s, const float (&v)[8], float inv_u, SlotMax x,
                                                uint32_t launch = 0u) {
  const int lane = threadIdx.x & 63;
  const float kInf = __uint_as_float(0x7f800000u);
  const float c1 = inv_u * kLog2e;
  const float M = x.M;
  // With a finite maximum of ordinary size every entry's exponent below is finite or -inf unless
  // the entry is NaN, so the sum itself tells whether the slot holds a NaN; otherwise the
  // entries are tested one by one.
  const bool ordinary = M > -kInf && __builtin_fabsf(M) < 1e38f;
  float sum = 0.0f;
  bool nan = false;
  if (ordinary) {
    const float c2 = -M * kLog2e;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += fast_exp2(__builtin_fmaf(v[e], c1, c2));
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) nan = nan || (v[e] != v[e]);
    if (M > -kInf) {
      const float c2 = -M * kLog2e;
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += fast_exp2(__builtin_fmaf(v[e], c1, c2));  // (a NaN here: the row is one)
    }
  }
  sum = wave_sum_f32(sum);
  const bool any_nan = ordinary ? sum != sum : __ballot(nan) != 0ull;
  if (lane == 0) {
    const int64_t at = static_cast<int64_t>(row) * p.ns_stride + s;
    if (COHERENT) coherent_store4(p.slot_pack + at, any_nan ? __uint_as_float(0x7fc00000u) : M, x.M2, sum, launch);
    if (!COHERENT || PLAIN_TOO) {
      p.slot_max[at] = any_nan ? __uint_as_float(0x7fc00000u) : M;
      p.slot_max2[at] = x.M2;
      p.slot_sum[at] = sum;
    }
  }
}
template <bool COHERENT = false, bool PLAIN_TOO = false>
__device__ __forceinline__ void split_pass1_slot(const SplitParams& p, int row, int s, const float (&v)[8], float inv_u,
                                                 uint32_t launch = 0u) {
  split_pass1_sum<COHERENT, PLAIN_TOO>(p, row, s, v, inv_u, split_pass1_max(v, inv_u), launch);
}

// grid = (ceil(ns / (4 SLOTS)), rows), 256 lanes: every wave takes SLOTS slots, all loads issued first.
// (Small workgroups: many are resident per CU, which is what a kernel bound by HBM wants.)
constexpr int kPass1Block = 256;
// SLOTS: slots per wave (two when the launch is small: more, shorter waves end sooner; four when it
// fills the chip several times over).
template <int DT, int SLOTS>
__global__ void __launch_bounds__(kPass1Block) split_pass1_kernel(SplitParams p) {
  const int row = p.row.row_map ? p.row.row_map[blockIdx.y] : blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int V = p.row.vocab;
  const float inv = p.row.row_cfg ? p.row.row_cfg[row].inv_temperature : p.row.inv_temperature;
  const char* logits = static_cast<const char*>(p.row.logits) + static_cast<int64_t>(row) * p.row.row_stride * ElemSize<DT>::value;
  const float kInf = __uint_as_float(0x7f800000u);
  const float fill = inv < 0.0f ? kInf : -kInf;  // x = -inf: adds nothing
  const int s_end = p.ns;
  for (int slot0 = (blockIdx.x * (kPass1Block / 64) + wave) * SLOTS; slot0 < s_end; slot0 = s_end) {
    float v[SLOTS][8];
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
      if (slot0 + k < s_end) load_slot_lane<DT>(logits, slot0 + k, lane, V, fill, v[k], p.row.fused);
    }
    float inv_u = inv;
    if (!(__builtin_fabsf(inv) < kInf)) {
#pragma unroll
      for (int k = 0; k < SLOTS; ++k) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[k][e] = v[k][e] * inv;
      }
      inv_u = 1.0f;
    }
#pragma unroll
    for (int k = 0; k < SLOTS; ++k) {
      const int s = slot0 + k;
      if (s >= s_end) break;
      split_pass1_slot(p, row, s, v[k], inv_u);
    }
  }
}

// ---- pass 2 ---------------------------------------------------------------------------------------
// LDS of pass 2 beyond the expf table.
struct Pass2Shared {
  BlockScratch sm;
  float upto[kMaxSlots + 1];  // approximate running sum in front of every slot, in units of exp(-m)
  uint32_t cls[kMaxSlots];    // per slot: kb_lo | kb_hi << 8 | kind << 16 | prepared-slot index << 19 (11 bits) | bit 30: the
                              //   binade predicted at the slot's entry is the upper one
  float top[kMaxSlots];       // per slot: an upper bound of its largest exp (top-p: a slot below the listing cut is not searched)
  uint32_t hist[kHistBuckets];
  uint32_t list_count;        // candidates this workgroup has listed
  uint32_t top_mass[32];      // the slots' two largest exps, added up per binade (bin j: [2^-j, 2^(1-j))), in units of 2^-20
  uint32_t top_all[32];       // the whole mass of the slots, by the binade of their largest exp, in units of 2^-10 (rounded up)
  // what the first wave worked out on its own (FUSED): row maximum, approximate total, serial slots, NaN row, done
  float pro_m, pro_total;
  uint32_t pro_serial, pro_nan, pro_done;
  alignas(8) uint32_t seen[2048];  // (FUSED, bf16) a byte per eight consecutive 16-bit patterns: some entry of this workgroup has one of them
};

// One wave, one slot: e[] are the lane's 8 entries; `cls` is the slot's entry of Pass2Shared::cls.
template <bool TOPP, int DT>
__device__ __forceinline__ void split_fold_slot(const SplitParams& p, int row, int s, const float (&e)[8],
                                                const float (&logit)[8], uint32_t cls, float cut_lo, bool search, int V,
                                                uint64_t* region, Pass2Shared& sh, const KeyMap& km, uint32_t* ph) {
  const int lane = threadIdx.x & 63;
  const int64_t rec_at = static_cast<int64_t>(row) * p.ns_stride + s;
  // ---- candidates of the top-p draw (sampler.cpp:137-143), by a cut that is safely below the
  //      reference's once the exact normaliser is known
  if (TOPP && search) {
    // bit k: entry k is a candidate (two instructions per entry: compare, shift the outcome in)
    uint32_t cmask = 0u;
#pragma unroll
    for (int k = 7; k >= 0; --k)
      asm("v_cmp_le_f32 vcc, %2, %1\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(cmask) : "v"(e[k]), "s"(cut_lo) : "vcc");
    if (s == p.ns - 1) {  // entries past the row's end
      const int left = V - (s * kSlot + lane * 8);
      cmask &= left >= 8 ? 0xffu : (left > 0 ? (1u << left) - 1u : 0u);
    }
    const uint64_t has1 = __ballot(cmask != 0u);
    if (has1 != 0ull) {
      const int first = s * kSlot + lane * 8;
      uint32_t at = 0u;
      auto note = [&](float ek, float lk, int k) {
        const uint32_t eb = __float_as_uint(ek);
        atomicAdd(&sh.hist[hist_bucket(eb)], 1u);
        if constexpr (DT == kDtypeBFloat16 || DT == kDtypeHalf) {
          // 16-bit rows: the same candidates per bit pattern (one outside the range of bins is
          // missed there, which the totals give away)
          const int bin = pattern_key(value_pattern<DT>(lk), km.mag_min) - km.key_cut;
          if (bin >= 0 && bin < km.n_bins) atomicAdd(&ph[bin >> 1], 1u << ((bin & 1) << 4));
        }
        if (at < static_cast<uint32_t>(p.list_region)) region[at] = (static_cast<uint64_t>(eb) << 32) | static_cast<uint32_t>(first + k);
        ++at;
      };
      const uint32_t rest1 = cmask & (cmask - 1u);   // without the lane's first candidate
      const uint32_t rest2 = rest1 & (rest1 - 1u);   // without its second
      if (__ballot(rest2 != 0u) != 0ull) {
        // dense (some lane holds three or more): entry by entry, places from a scan over the lanes
        const uint32_t mine = static_cast<uint32_t>(__popc(cmask));
        const uint32_t incl = wave_scan_inclusive_u32(mine);
        const uint32_t total = readlane_u32(incl, 63);
        uint32_t base = 0u;
        if (lane == 0) base = atomicAdd(&sh.list_count, total);
        base = readlane_u32(base, 0);
        if (base >= static_cast<uint32_t>(p.list_region)) {
          // The workgroup's list is full already, so the finish kernel will find that the row's
          // lists do not hold every candidate and use neither them nor the histogram by size
          // (every use of the two is behind that check): only the count above and the count per
          // bit pattern, by which a 16-bit row with a long nucleus is drawn, are still needed.
          if constexpr (DT == kDtypeBFloat16 || DT == kDtypeHalf) {
            if (km.n_bins > 0) {
              const int shift = 0x8000 - km.key_cut, first_mag = km.mag_min - 1;
#pragma unroll
              for (int k = 0; k < 8; ++k) {
                // pattern_key() - key_cut (a negative value's key 0x7fff - cm is 0x8000 + ~cm)
                const uint32_t pat = value_pattern<DT>(logit[k]);
                const int mag = static_cast<int>(pat & 0x7fffu) - first_mag;
                const int cm = mag > 0 ? mag : 0;
                const int bin = (cm ^ (static_cast<int>(pat << 16) >> 31)) + shift;
                if (((cmask >> k) & 1u) && static_cast<uint32_t>(bin) < static_cast<uint32_t>(km.n_bins))
                  atomicAdd(&ph[bin >> 1], 1u << ((bin & 1) << 4));
              }
            }
          }
        } else {
          at = base + incl - mine;
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            if ((cmask >> k) & 1u) note(e[k], logit[k], k);
          }
        }
      } else {
        // sparse (the usual row: a few candidates in a slot, at most two in a lane): two rounds,
        // every lane taking its next candidate; places from the two ballots, no scan
        const uint64_t has2 = __ballot(rest1 != 0u);
        const uint32_t n1 = static_cast<uint32_t>(__popcll(has1)), n2 = static_cast<uint32_t>(__popcll(has2));
        uint32_t base = 0u;
        if (lane == 0) base = atomicAdd(&sh.list_count, n1 + n2);
        base = readlane_u32(base, 0);
        const uint64_t below = (1ull << lane) - 1ull;
        auto one = [&](uint32_t mask) {
          const int k = __ffs(static_cast<int>(mask)) - 1;
          // entry k of the lane's eight, by three levels of selects (kept in registers: indexing the
          // arrays with k would move them to private memory)
          const bool b0 = (k & 1) != 0, b1 = (k & 2) != 0, b2 = (k & 4) != 0;
          const float e01 = b0 ? e[1] : e[0], e23 = b0 ? e[3] : e[2], e45 = b0 ? e[5] : e[4], e67 = b0 ? e[7] : e[6];
          const float e03 = b1 ? e23 : e01, e47 = b1 ? e67 : e45;
          const float ek = b2 ? e47 : e03;
          float lk = 0.0f;
          if constexpr (DT == kDtypeBFloat16 || DT == kDtypeHalf) {
            const float l01 = b0 ? logit[1] : logit[0], l23 = b0 ? logit[3] : logit[2], l45 = b0 ? logit[5] : logit[4],
                        l67 = b0 ? logit[7] : logit[6];
            const float l03 = b1 ? l23 : l01, l47 = b1 ? l67 : l45;
            lk = b2 ? l47 : l03;
          }
          note(ek, lk, k);
        };
        if (cmask) {
          at = base + static_cast<uint32_t>(__popcll(has1 & below));
          one(cmask);
        }
        if (has2 != 0ull && rest1) {
          at = base + n1 + static_cast<uint32_t>(__popcll(has2 & below));
          one(rest1);
        }
      }
    }
  }
  uint32_t bits[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) bits[k] = __float_as_uint(e[k]);
  // ---- the row's first slot is entered with the sum 0: worked out here, entry by entry
  if (s == 0) {
    float sum = 0.0f;
    int found = -1;
    wave_resolve<8>(sum, found, bits, lane * 8, V, __uint_as_float(0x7f800000u));
    if (lane == 0) p.slot_rec[rec_at] = {kSlotExact << 8, __float_as_uint(sum), 0u, 0xffffffffu};
    return;
  }
  // ---- every entry 0: no effect on any running sum
  const uint32_t any_bits = bits[0] | bits[1] | bits[2] | bits[3] | bits[4] | bits[5] | bits[6] | bits[7];  // (no -0 among exps)
  const uint32_t kb_lo = cls & 255u, kb_hi = (cls >> 8) & 255u;
  const uint32_t kind = (cls >> 16) & 7u;
  // the binade the sum is predicted to be in when it reaches the slot (bits 16-23 of the record)
  const uint32_t kb_in = ((kb_lo + ((cls >> 30) & 1u)) & 255u) << 16;
  if (__ballot(any_bits != 0u) == 0ull) {
    if (lane == 0) p.slot_rec[rec_at] = {(kSlotZero << 8) | kb_in, 0u, 0u, 0xffffffffu};
    return;
  }
  if (kind == kSlotStable) {
    // ---- the sum stays in binade kb_lo throughout the slot
    const float scale = __uint_as_float((277u - kb_lo) << 23);  // 2^(150 - kb)
    FastAcc acc = {0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < 8; ++k) fast_fold(acc, e[k], scale);
    ParityInc slot;
    if (__ballot(acc.tie == 0.5f) == 0ull) {
      const float inc = wave_sum_f32(acc.inc);
      const uint32_t v = inc < 67108864.0f ? static_cast<uint32_t>(inc) : kSat;
      slot.even = v;
      slot.odd = v;
    } else {
      const ParityInc upto = wave_scan_inclusive(fold_run<8>(bits, __uint_as_float(kb_lo << 23)), lane);
      slot.even = readlane_u32(upto.even, 63);
      slot.odd = readlane_u32(upto.odd, 63);
    }
    if (lane == 0) p.slot_rec[rec_at] = {kb_lo | (kSlotStable << 8) | (kb_lo << 16), slot.even, slot.odd, 0xffffffffu};
    return;
  }
  if (kind == kSlotDual) {
    // ---- the sum passes the slot inside binade kb_lo or inside kb_lo + 1
    const float scale_a = __uint_as_float((277u - kb_lo) << 23), scale_b = __uint_as_float((276u - kb_lo) << 23);
    FastAcc fa = {0.0f, 0.0f}, fb = {0.0f, 0.0f};
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      fast_fold(fa, e[k], scale_a);
      fast_fold(fb, e[k], scale_b);
    }
    const bool ties = __ballot(fa.tie == 0.5f || fb.tie == 0.5f) != 0ull;
    const float inc_a = wave_sum_f32(fa.inc), inc_b = wave_sum_f32(fb.inc);
    if (lane == 0) {
      if (ties) {  // (rare) the finish kernel works the slot out from the logits
        p.slot_rec[rec_at] = {kb_lo | (kSlotSerial << 8) | ((kb_lo + 1u) << 16), 0u, 0u, 0xffffffffu};
      } else {
        p.slot_rec[rec_at] = {kb_lo | (kSlotDual << 8) | kb_in, inc_a < 67108864.0f ? static_cast<uint32_t>(inc_a) : kSat,
                              inc_b < 67108864.0f ? static_cast<uint32_t>(inc_b) : kSat, 0xffffffffu};
      }
    }
    return;
  }
  // ---- to be resolved in order: keep the entries and the lanes' increments under both candidate ulps
  const uint32_t idx = (cls >> 19) & 0x7ffu;
  const uint32_t kb_a = kb_lo, kb_b = kb_hi > kb_lo ? kb_hi : kb_lo + 1u;
  bool clean = false;  // prepared, both binades in the range of the float shortcut
  if (idx < static_cast<uint32_t>(p.prep_cap)) {
    PrepSlot& ps = p.prep[static_cast<int64_t>(row) * p.prep_cap + idx];
    float4* pe = reinterpret_cast<float4*>(ps.e + lane * 8);
    pe[0] = {e[0], e[1], e[2], e[3]};
    pe[1] = {e[4], e[5], e[6], e[7]};
    const bool usable = kb_a >= 70u && kb_b <= 250u;
    FastAcc fa = {0.0f, 0.0f}, fb = {0.0f, 0.0f};
    if (usable) {
      const float scale_a = __uint_as_float((277u - kb_a) << 23), scale_b = __uint_as_float((277u - kb_b) << 23);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        fast_fold(fa, e[k], scale_a);
        fast_fold(fb, e[k], scale_b);
      }
    }
    const float kCap = 16777216.0f;  // 2^24
    ps.pre_a[lane] = wave_scan_inclusive_u32(static_cast<uint32_t>(__builtin_fminf(fa.inc, kCap))) | (fa.tie == 0.5f ? kPrepTie : 0u);
    ps.pre_b[lane] = wave_scan_inclusive_u32(static_cast<uint32_t>(__builtin_fminf(fb.inc, kCap))) | (fb.tie == 0.5f ? kPrepTie : 0u);
    const uint64_t tie_a = __ballot(fa.tie == 0.5f), tie_b = __ballot(fb.tie == 0.5f);
    clean = usable && kb_b <= 255u;
    if (lane == 0) {
      ps.kb_a = kb_a;
      ps.kb_b = kb_b;
      ps.tie_a_lo = static_cast<uint32_t>(tie_a);
      ps.tie_a_hi = static_cast<uint32_t>(tie_a >> 32);
      ps.tie_b_lo = static_cast<uint32_t>(tie_b);
      ps.tie_b_hi = static_cast<uint32_t>(tie_b >> 32);
      ps.usable = usable ? 1u : 0u;
      ps.pad = 0u;
    }
  }
  if (lane == 0) {
    p.slot_rec[rec_at] = {kb_a | (kSlotSerial << 8) | ((kb_b & 255u) << 16) | (clean ? 1u << 24 : 0u), 0u, 0u,
                          idx < static_cast<uint32_t>(p.prep_cap) ? idx : 0xffffffffu};
  }
}

// grid = (workgroups per row, rows); dynamic LDS: the expf table of bf16 rows (kLutCountWords floats).
#ifndef ETS_PASS2_WAVES_PER_EU
#define ETS_PASS2_WAVES_PER_EU 4
#endif
// WALK: the second sum of a multinomial row (sampler.cpp:58-70): the entries are p = fl(e / S) with the exact
// softmax sum S that the first chain left in SplitParams::walk, and the records describe their running sum.
// TOPK: some row of the launch may be a top-k row (a launch without one runs the code without that case).
// FUSED: pass 1 inside this kernel, for launches whose workgroups are all resident at once (at most one per
// compute unit) and hold at most kFusedSlots slots per wave: a workgroup loads its slots ONCE, keeps them in
// registers, stores their maxima and approximate sums, and meets the other workgroups of its row at a counter
// in device memory before it goes on with what pass 2 does.  The wait is bounded: a workgroup that has polled
// `spin_limit` times works the other workgroups' slots out itself from the logits (the same values: whoever
// stores them stores the same bits), so every workgroup ends whatever the others do.  The grid is one-
// dimensional and the workgroups of a row are dealt so that they share a die (XCD) and its L2 when the number
// of rows is a multiple of eight (workgroups go to the eight dies in turn by their index).
constexpr int kFusedSlots = 4;
template <int DT, bool TOPP, bool WALK = false, bool TOPK = false, bool EXTRAS = true, bool FUSED = false>
__global__ void __launch_bounds__(kBlock, ETS_PASS2_WAVES_PER_EU) split_pass2_kernel(SplitParams p) {
  uint64_t* const timers = (ETS_PHASE_CLOCKS && EXTRAS) ? p.timers : nullptr;  // (EXTRAS: the launch may fill the phase clocks)
  extern __shared__ __align__(16) float lut_mem[];
  __shared__ Pass2Shared sh;
  BlockScratch& sm = sh.sm;
  int part = blockIdx.x, n_parts = gridDim.x;
  int lrow = blockIdx.y;  // row of this launch: indexes the buffers whose layout depends on the launch
  if (FUSED) {
    n_parts = p.row_wgs;
    const int rows = p.row.rows;
    if ((rows & 7) == 0) {
      const int die = blockIdx.x & 7, k = blockIdx.x >> 3;  // rows die, die + 8, ... on one die
      lrow = (k / n_parts) * 8 + die;
      part = k % n_parts;
    } else {
      lrow = blockIdx.x / n_parts;
      part = blockIdx.x % n_parts;
    }
  }
  const int row = p.row.row_map ? p.row.row_map[lrow] : lrow;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int V = p.row.vocab;
  const int ns = p.ns;
  const float inv = p.row.row_cfg ? p.row.row_cfg[row].inv_temperature : p.row.inv_temperature;
  const float topp = p.row.row_cfg ? p.row.row_cfg[row].topp : p.row.topp;
  const int32_t topk = !TOPK ? 0 : (p.row.row_cfg ? p.row.row_cfg[row].topk : p.row.topk);
  const bool row_topk = TOPK && topk > 0 && topk < p.row.vocab;  // sampler.cpp:239: top-k comes before top-p
  const char* logits = static_cast<const char*>(p.row.logits) + static_cast<int64_t>(row) * p.row.row_stride * ElemSize<DT>::value;
  const float* slot_max = p.slot_max + static_cast<int64_t>(row) * p.ns_stride;
  const float* slot_sum = p.slot_sum + static_cast<int64_t>(row) * p.ns_stride;
  const float* slot_max2 = p.slot_max2 + static_cast<int64_t>(row) * p.ns_stride;
  const float4* slot_pack = p.slot_pack + static_cast<int64_t>(row) * p.ns_stride;  // (FUSED)
  const float kInf = __uint_as_float(0x7f800000u);
  const float fill = inv < 0.0f ? kInf : -kInf;
  uint64_t c0 = 0, c1 = 0, c2 = 0, c3 = 0, cf0 = 0, cf1 = 0, cf2 = 0;
  if (timers) c0 = wall_clock64();
  if (tid < 32) sm.exp2tab[tid] = kExp2Table[tid];
  if (tid == 0) sh.list_count = 0u;
  if (TOPP && tid < 32) {
    sh.top_mass[tid] = 0u;
    sh.top_all[tid] = 0u;
  }
  if (FUSED && DT == kDtypeBFloat16) {
    sh.seen[tid] = 0u;
    sh.seen[tid + kBlock] = 0u;
  }
  // 16-bit rows: entries per bit pattern, behind the expf table
  constexpr bool kPatterns = TOPP && (DT == kDtypeBFloat16 || DT == kDtypeHalf);
  uint32_t* ph = reinterpret_cast<uint32_t*>(lut_mem + (DT == kDtypeBFloat16 ? kLutCountWords : 0));
  if (TOPP) {
    for (int b = tid; b < kHistBuckets; b += kBlock) sh.hist[b] = 0u;
    if (kPatterns) {
      for (int b = tid; b < p.phist_words; b += kBlock) ph[b] = 0u;
    }
  }

  // ---- this workgroup's slots: wave w takes s_begin + w, s_begin + w + 16, ...; the first one's
  //      entries are requested before anything else
  int s_begin, s_end;
  split_range(ns, n_parts, part, s_begin, s_end);
  float l[8];
  int s_mine = s_begin + wave;
  static_assert(kFusedSlots == 4, "four named register sets below");
  int lut_base1 = 0, lut_top = 0, lut_half = 0;
  int early_lut = -1;      // FUSED: the expf table was built for early_m already (1: usable, 0: not)
  float early_m = 0.0f;
  float held0[8], held1[8], held2[8], held3[8];  // FUSED: the wave's slots, read once (named one by one: they stay in registers)
  const uint32_t launch = FUSED ? p.arrive[0] + 1u : 0u;  // FUSED: the number this launch tags what it hands over with
  bool pro_early = false;  // FUSED: the first wave does the row-level work on its own while the others build the table
  float x_first = 0.0f;    // FUSED: x[0], asked for with the slots
  // (FUSED) Given up on the others: their slots from the logits (whoever stores a slot's three values stores the same bits).
  auto alone = [&]() {
    for (int s = wave; s < ns; s += kWaves) {
      if (s >= s_begin && s < s_end) continue;
      float v[8];
      load_slot_lane<DT>(logits, s, lane, V, fill, v, p.row.fused);
      split_pass1_slot<true>(p, row, s, v, inv, launch);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  if constexpr (FUSED) {
    if (s_mine < s_end) load_slot_lane<DT>(logits, s_mine, lane, V, fill, held0, p.row.fused);
    if (s_mine + kWaves < s_end) load_slot_lane<DT>(logits, s_mine + kWaves, lane, V, fill, held1, p.row.fused);
    if (s_mine + 2 * kWaves < s_end) load_slot_lane<DT>(logits, s_mine + 2 * kWaves, lane, V, fill, held2, p.row.fused);
    if (s_mine + 3 * kWaves < s_end) load_slot_lane<DT>(logits, s_mine + 3 * kWaves, lane, V, fill, held3, p.row.fused);
    x_first = load_logit<DT>(logits, 0, p.row.fused) * inv;  // (max_val starts at x[0]: a NaN there stays)
    // ---- pass 1 for these slots (the host sends no launch with an infinite inverse temperature here):
    //      every slot's maximum, second maximum and approximate sum, handed to the row's other
    //      workgroups: stored with device-scope accesses that go through to memory one by one (no
    //      fence of device scope, which would write back or discard the die's whole L2: microseconds,
    //      when every workgroup of the die does it), each with a tag that tells the reader that
    //      it is there (coherent_store4); no counter, and nobody waits for its own stores.  (A multinomial
    //      row's second sweep is a launch of its own, which reads the values where pass 1 leaves them.)
    if (s_mine < s_end) split_pass1_slot<true, !TOPP>(p, row, s_mine, held0, inv, launch);
    if (s_mine + kWaves < s_end) split_pass1_slot<true, !TOPP>(p, row, s_mine + kWaves, held1, inv, launch);
    if (s_mine + 2 * kWaves < s_end) split_pass1_slot<true, !TOPP>(p, row, s_mine + 2 * kWaves, held2, inv, launch);
    if (s_mine + 3 * kWaves < s_end) split_pass1_slot<true, !TOPP>(p, row, s_mine + 3 * kWaves, held3, inv, launch);
    if constexpr (DT == kDtypeBFloat16) {
      // the bit patterns among this workgroup's entries: the expf table is built for these alone (while
      // the other workgroups' values are on their way there is nothing else to do)
      __syncthreads();  // (the marks were cleared by other waves)
      auto mark = [&](const float (&v)[8]) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          reinterpret_cast<uint8_t*>(sh.seen)[__float_as_uint(v[k]) >> 19] = 1;
        }
      };
      if (s_mine < s_end) mark(held0);
      if (s_mine + kWaves < s_end) mark(held1);
      if (s_mine + 2 * kWaves < s_end) mark(held2);
      if (s_mine + 3 * kWaves < s_end) mark(held3);
    }
    if (timers) cf0 = wall_clock64();
    pro_early = true;
  } else {
    if (s_mine < s_end) load_slot_lane<DT>(logits, s_mine, lane, V, fill, l, p.row.fused);
  }

  // ---- The row-level work of every workgroup of the row: the row maximum from the slots' maxima
  //      (sampler.cpp:191-197), the approximate running sums in front of every slot and, from them,
  //      the binades the sequential sum can be in at the two ends of each slot.  A slot that cannot be
  //      placed inside one binade (or one of two neighbours) is resolved in order by the finish kernel
  //      and gets a prepared-slot index.  Two forms of it, the same arithmetic in the same order (all
  //      workgroups of a row must arrive at the same classes and indices, whichever form each takes):
  //      by the whole workgroup, a slot per lane; and (FUSED) by the first wave alone, sixty-four
  //      slots at a time, with no barrier, while the other waves build the expf table.
  RowDivisor walk_div = {};
  float walk_scale = 1.0f;
  if (WALK) {
    const float S = p.walk[row].x;
    walk_div = row_divisor(S);
    walk_scale = 1.0f / S;  // (the approximate sums only place the running sum in a binade)
  }
  // a slot's approximate mass in units of exp(-m); notes the bound of its largest exp and, for top-p
  // rows, lower bounds of its two largest exps by binade
  auto slot_mass = [&](int s, float sum, float smax, float smax2, float m_row) -> float {
    const float f = sum > 0.0f ? fast_exp2((smax - m_row) * kLog2e) : 0.0f;  // exp of the slot's largest entry
    float a = sum > 0.0f ? sum * f : 0.0f;
    if (WALK) a *= walk_scale;
    if (TOPP) sh.top[s] = f * 1.0001f;  // (the hardware's exp2 is within 1e-5 of the exact exp)
    if (TOPP && f > 0.0f) {
      // lower bounds of the exact exps of the slot's two largest entries, into the bins of their
      // binades (integers: every workgroup of the row arrives at the same totals)
      const float f2 = smax2 > -kInf ? fast_exp2((smax2 - m_row) * kLog2e) : 0.0f;
      const float below[2] = {f * 0.9999f, f2 * 0.9999f};
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int j = 127 - static_cast<int>(__float_as_uint(below[q]) >> 23);
        if (below[q] > 0.0f && j >= 0 && j < 32) atomicAdd(&sh.top_mass[j], static_cast<uint32_t>(below[q] * 1048576.0f));
        // a top-k row counts them by histogram bucket (the histogram is not in use yet)
        if (row_topk && below[q] > 0.0f) atomicAdd(&sh.hist[hist_bucket(__float_as_uint(below[q]))], 1u);
      }
      // the slot's whole mass (at most 512), rounded up: what bounds how many of its entries reach a cut
      const int j0 = 127 - static_cast<int>(__float_as_uint(below[0]) >> 23);
      if (j0 >= 0 && j0 < 32) atomicAdd(&sh.top_all[j0], static_cast<uint32_t>(a * 1024.0f) + 1u);
    }
    return a;
  };
  // the class of slot s from the approximate sums at its two ends: kb_lo | kb_hi << 8 | kind << 16 | bit 30
  auto slot_class = [&](int s, float a_in, float a_out) -> uint32_t {
    const float lo = a_in * (1.0f - split_eps(s * kSlot));
    const float hi = a_out * (1.0f + split_eps((s + 1) * kSlot));
    const uint32_t kb_lo = __float_as_uint(lo > 0.0f ? lo : 0.0f) >> 23, kb_hi = __float_as_uint(hi) >> 23;
    // inside one binade for certain; or inside one of two neighbours, the sums themselves
    // pointing at no change inside the slot (kept as one increment per binade); or in order
    uint32_t kind = kSlotSerial;
    if (lo > 0.0f && kb_lo >= 70u && kb_hi <= 250u) {
      if (kb_lo == kb_hi) {
        kind = kSlotStable;
      } else if (kb_hi == kb_lo + 1u && (__float_as_uint(a_in) >> 23) == (__float_as_uint(a_out) >> 23)) {
        kind = kSlotDual;
      }
    }
    // (bit 30: the approximate sum in front of the slot lies in the upper of the two binades)
    const uint32_t in_hi = (__float_as_uint(a_in) >> 23) > kb_lo ? 1u << 30 : 0u;
    return (kb_lo & 255u) | ((kb_hi > 255u ? 255u : kb_hi) << 8) | (kind << 16) | in_hi;
  };

  float m = -kInf;
  float a_total = 0.0f;
  uint32_t serial_before = 0u;
  bool row_nan = false;
  bool pro_done = false;
  if constexpr (FUSED) {
    if (pro_early) {
      if (wave == 0) {
        // (the hand-over: the slots' values are read until every one carries this launch's tag, a bounded
        // number of times; they are parked in LDS where the results will go, four slots of a lane per
        // trip to memory)
        int met = 0;
        float mm = -kInf;
        bool nanf = false;
        for (int spin = 0; spin < p.spin_limit && !met; ++spin) {
          if (spin != 0) __builtin_amdgcn_s_sleep(2);
          mm = -kInf;
          nanf = false;
          bool missing = false;
          for (int base = 0; base < ns; base += 256) {
            ets_f32x4 v[4];
            const int s0 = base + lane;
            coherent_load4x4(slot_pack + min(s0, ns - 1), slot_pack + min(s0 + 64, ns - 1), slot_pack + min(s0 + 128, ns - 1),
                             slot_pack + min(s0 + 192, ns - 1), v[0], v[1], v[2], v[3]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int s = s0 + 64 * k;
              if (s < ns) {
                missing = missing || __float_as_uint(v[k].w) != pack_tag(launch, v[k].x, v[k].y, v[k].z);
                sh.top[s] = v[k].x;
                sh.cls[s] = __float_as_uint(v[k].y);
                sh.upto[s + 1] = v[k].z;
                nanf = nanf || (v[k].x != v[k].x);
                mm = __builtin_fmaxf(mm, v[k].x);
              }
            }
          }
          met = __ballot(missing) == 0ull ? 1 : 0;
        }
        if (met) {
          mm = wave_max_ignoring_nan(mm);
          const bool nan_any = __ballot(nanf) != 0ull;
          if (x_first != x_first) mm = x_first;  // max_val starts at x[0]; nothing compares greater than NaN
          if (lane == 0) {
            sh.pro_m = mm;
            sh.pro_nan = (nan_any || !(mm > -kInf && mm < kInf)) ? 1u : 0u;
          }
        }
        if (lane == 0) sh.pro_done = met ? 1u : 0u;
      }
      __syncthreads();
      if (timers) cf1 = wall_clock64();
      pro_done = sh.pro_done != 0u;
      if (pro_done) {
        m = sh.pro_m;
        row_nan = sh.pro_nan != 0u;
        if (!row_nan) {
          if (wave == 0) {
            float run = 0.0f;
            uint32_t serials = 0u;
            for (int c0 = 0; c0 < ns; c0 += 64) {
              const int s = c0 + lane;
              float a = 0.0f;
              if (s < ns) a = slot_mass(s, sh.upto[s + 1], sh.top[s], __uint_as_float(sh.cls[s]), m);
              const float incl = wave_scan_inclusive_f32(a, lane);
              const float before = run;
              run = run + readlane_f32(incl, 63);
              const float a_out = before + incl;
              const float a_in = before + lane_before_f32(incl);
              const uint32_t cls = slot_class(s, a_in, a_out);
              const bool serial = s < ns && s > 0 && ((cls >> 16) & 7u) == kSlotSerial;  // (slot 0 is worked out in this kernel)
              const uint64_t serial_ballot = __ballot(serial);
              const uint32_t rank = serials + static_cast<uint32_t>(__popcll(serial_ballot & ((1ull << lane) - 1ull)));
              if (s < ns) {
                sh.upto[s + 1] = a_out;
                sh.cls[s] = cls | ((rank & 0x7ffu) << 19);
              }
              serials += static_cast<uint32_t>(__popcll(serial_ballot));
            }
            if (lane == 0) {
              sh.pro_total = run;
              sh.pro_serial = serials;
            }
          }
          if constexpr (DT == kDtypeBFloat16) {
            // (the table's entries are dealt to the other waves; the first one only works out where it lies)
            early_m = m;
            early_lut = build_exp_lut_marked(lut_mem, kLutCountWords, inv, m, sm.exp2tab, lut_base1, lut_top, lut_half,
                                             reinterpret_cast<const uint8_t*>(sh.seen)) ? 1 : 0;
          }
          __syncthreads();
          a_total = sh.pro_total;
          serial_before = sh.pro_serial;
        }
      } else {
        alone();  // (given up on the others: their slots from the logits, then the form below)
      }
      if (timers) cf2 = wall_clock64();
    }
  }
  float first_max = 0.0f, first_sum = 0.0f, first_max2 = -kInf;  // the scan below starts with the same slots
  // (FUSED: other workgroups of this launch stored these) a slot's maximum, second maximum and sum
  auto slot_values = [&](int s, float& mx, float& mx2, float& sum) {
    if constexpr (FUSED) {
      const ets_f32x4 v = coherent_load4(slot_pack + s);
      mx = v.x;
      mx2 = v.y;
      sum = v.z;
    } else {
      mx = slot_max[s];
      sum = slot_sum[s];
      mx2 = TOPP ? slot_max2[s] : -kInf;
    }
  };
  if (!pro_done) {
    bool any_nan = false;
    for (int s = tid; s < ns; s += kBlock) {
      float v, v2, vs;
      slot_values(s, v, v2, vs);
      if (s == tid) {
        first_max = v;
        first_sum = vs;
        first_max2 = v2;
      }
      any_nan = any_nan || (v != v);
      m = __builtin_fmaxf(m, v);
    }
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
    const float x0 = load_logit<DT>(logits, 0, p.row.fused) * inv;
    if (x0 != x0) m = x0;  // max_val starts at x[0]; nothing compares greater than NaN
    row_nan = nan_any != 0u || !(m > -kInf && m < kInf);
  }
  if (row_nan) {  // one NaN addend poisons the sum: the finish kernel needs nothing else
    if (part == 0 && tid == 0) p.row_state[row] = {0u, m, 1u, 0.0f, 0, 0, 0, 0u};
    return;
  }
  __syncthreads();
  if (timers) c1 = wall_clock64();
  if (!pro_done) {
    float carry = 0.0f;
    for (int base = 0; base < ns; base += kBlock) {
      const int s = base + tid;
      float a = 0.0f;
      if (s < ns) {
        float sum = first_sum, smax = first_max, smax2 = first_max2;
        if (base != 0) slot_values(s, smax, smax2, sum);
        a = slot_mass(s, sum, smax, smax2, m);
      }
      const float incl = wave_scan_inclusive_f32(a, lane);
      if (lane == 63) sm.group_total[0][wave] = incl;
      __syncthreads();
      float before = carry, all = carry;
      for (int w = 0; w < kWaves; ++w) {
        if (w == wave) before = all;
        all += sm.group_total[0][w];
      }
      const float a_out = before + incl;
      const float a_in = before + lane_before_f32(incl);
      if (s < ns) sh.upto[s + 1] = a_out;
      carry = all;
      const uint32_t cls = slot_class(s, a_in, a_out);
      const bool serial = s < ns && s > 0 && ((cls >> 16) & 7u) == kSlotSerial;  // (slot 0 is worked out in this kernel)
      const uint64_t serial_ballot = __ballot(serial);
      if (lane == 0) sm.red_u[wave] = static_cast<uint32_t>(__popcll(serial_ballot));
      __syncthreads();
      uint32_t rank = serial_before;
      uint32_t chunk_total = 0u;
      for (int w = 0; w < kWaves; ++w) {
        if (w < wave) rank += sm.red_u[w];
        chunk_total += sm.red_u[w];
      }
      rank += static_cast<uint32_t>(__popcll(serial_ballot & ((1ull << lane) - 1ull)));
      if (s < ns) sh.cls[s] = cls | ((rank & 0x7ffu) << 19);
      serial_before += chunk_total;
    }
    a_total = carry;
  }
  if (timers) c2 = wall_clock64();

  // ---- bf16 rows: expf by bit pattern
  bool use_lut = false;
  if constexpr (DT == kDtypeBFloat16) {
    if (FUSED && early_lut >= 0 && __float_as_uint(early_m) == __float_as_uint(m)) {
      use_lut = early_lut != 0;  // (built while the slots' sums were on their way)
    } else {
      use_lut = build_exp_lut<false>(lut_mem, kLutCountWords, inv, m, sm.exp2tab, lut_base1, lut_top, lut_half);
    }
    if (WALK && use_lut) {  // one division per bit pattern: the table becomes p = fl(e / S)
      __syncthreads();
      for (int idx = tid; idx < 2 * lut_half; idx += kBlock) lut_mem[idx] = div_row(lut_mem[idx], walk_div);
    }
  }
  __syncthreads();
  if (timers) c3 = wall_clock64();
  const LutAddr lut_addr = lut_addr_of(lut_mem, lut_base1, lut_top, lut_half);

  const float cutoff = TOPP ? (1.0f - topp) / static_cast<float>(V - 1) : 0.0f;  // sampler.cpp:136
  const float cut_lo = cutoff * a_total * (1.0f - split_eps(V)) * 0.999f;
  // ---- a peaked row: when the largest entries of the slots alone carry safely more than topp of
  //      the mass, the nucleus lies among the entries of their binades, and only those are listed
  //      (whole buckets of the histogram, so that the finish kernel knows what the lists hold).  The
  //      count of all candidates is lost then, which only the debug record reports: a launch that
  //      asks for debug records lists everything.
  float list_cut = cut_lo;
  uint32_t listed_buckets = 0u;
  if (TOPP && row_topk) {
    // ---- a top-k row (sampler.cpp:72-120): the k largest entries are among those of the histogram
    //      buckets in which the slots' two largest exps first number k (lower bounds of the exps of
    //      distinct entries: at least k entries lie in those buckets), so those buckets are listed, whole.
    //      (How many more entries they hold is not known here: the finish kernel sorts the row when
    //      they do not fit its LDS.)  Fewer than k such exps above the last bucket: nothing is listed.
    static_assert(kHistBuckets == 2 * kBlock, "two buckets per lane");
    const uint32_t c0 = sh.hist[2 * tid], c1 = sh.hist[2 * tid + 1];
    const uint32_t incl_c = wave_scan_inclusive_u32(c0 + c1);
    if (lane == 63) sm.red_u[wave] = incl_c;
    if (tid == 0) sm.flag = -1;
    __syncthreads();
    uint32_t upto = incl_c;
    for (int w = 0; w < wave; ++w) upto += sm.red_u[w];
    const uint32_t before = upto - (c0 + c1);
    const uint32_t k = static_cast<uint32_t>(topk);
    if (upto >= k && before < k) sm.flag = before + c0 >= k ? 2 * tid : 2 * tid + 1;  // (one lane)
    __syncthreads();
    const int b_k = sm.flag;
    sh.hist[2 * tid] = 0u;  // (the sweep counts the listed candidates here)
    sh.hist[2 * tid + 1] = 0u;
    __syncthreads();
    list_cut = kInf;
    listed_buckets = kNoLists;
    if (b_k >= 0 && b_k < kHistBuckets - 1) {
      list_cut = __uint_as_float(0x3F800000u - (static_cast<uint32_t>(b_k + 1) << 17) + 1u);
      listed_buckets = static_cast<uint32_t>(b_k) + 1u;
    }
  } else if (TOPP && p.short_lists != 0 && p.row.debug == nullptr) {
    const uint32_t mine = lane < 32 ? sh.top_mass[lane] : 0u;
    const uint32_t incl = wave_scan_inclusive_u32(mine);
    const float need = topp * a_total * 1.04f * 1048576.0f;
    const uint64_t reach = __ballot(lane < 32 && static_cast<float>(incl) >= need);
    const uint32_t incl_all = wave_scan_inclusive_u32(lane < 32 ? sh.top_all[lane] : 0u);
    if (reach != 0ull) {
      const uint32_t j = static_cast<uint32_t>(__ffsll(static_cast<long long>(reach)) - 1);  // binades 1 .. j are enough
      // buckets 0 .. 64 j hold every exp from 2^-j up (bucket 64 j starts with 2^-j itself and is listed whole)
      const float whole = __uint_as_float(0x3F800000u - ((64u * j + 1u) << 17) + 1u);
      // How many entries that can list: an entry that reaches the cut adds at least the cut to its
      // slot's mass, and only slots whose largest exp is in binades 1 .. j + 1 hold any.  Beyond a
      // few thousand the full lists (and, for 16-bit rows, the draw by runs) serve better.
      const float listed_mass = static_cast<float>(readlane_u32(incl_all, j < 30u ? static_cast<int>(j) + 1 : 31)) * (1.0f / 1024.0f);
      const bool few = listed_mass <= 4096.0f * (whole * 0.97f);
      if (few && whole > cut_lo) {
        list_cut = whole;
        listed_buckets = 64u * j + 1u;
      }
    }
  }
  uint64_t* region = p.list + (static_cast<int64_t>(lrow) * p.row_wgs + part) * p.list_region;
  // ---- the pattern histogram's range of order keys: from safely below the smallest logit whose exp
  //      can reach cut_lo up to the row's largest logit (every workgroup of the row arrives at the
  //      same two numbers).  Too many bins for the LDS set aside: no pattern histogram.
  KeyMap km = {0, 0, 0};
  // (short lists are drawn from directly: no pattern histogram then)
  if (kPatterns && !row_topk && listed_buckets == 0u && p.phist_words > 0 && inv > 0.0f && inv < kInf && cut_lo > 0.0f &&
      (__float_as_uint(inv) >> 23) != 0u) {
    // magnitudes below 2^(em - ei - 27) vanish against m (em, ei: biased exponents of |m| and inv)
    const uint32_t mb = __float_as_uint(__builtin_fabsf(m));
    const int em = (mb >> 23) ? static_cast<int>(mb >> 23) : 1;
    const int et = em - static_cast<int>(__float_as_uint(inv) >> 23) - 27 + 127;
    if (et >= 1) km.mag_min = static_cast<int>(value_pattern<DT>(__uint_as_float(static_cast<uint32_t>(et > 254 ? 254 : et) << 23)) & 0x7fffu);
    const float x_cut = m + (__logf(cut_lo) - 0.01f);
    const float l_cut = x_cut / inv;
    const float l_top = m / inv;
    const float l_lo = l_cut - __builtin_fabsf(l_cut) * 1e-5f, l_hi = l_top + __builtin_fabsf(l_top) * 1e-5f;
    constexpr float kMaxFinite = DT == kDtypeBFloat16 ? 3.3895313892515355e38f : 65504.0f;
    const float l_lo_c = __builtin_fminf(__builtin_fmaxf(l_lo, -kMaxFinite), kMaxFinite);
    const float l_hi_c = __builtin_fminf(__builtin_fmaxf(l_hi, -kMaxFinite), kMaxFinite);
    km.key_cut = pattern_key(value_pattern<DT>(l_lo_c), km.mag_min) - 2;
    const int key_top = pattern_key(value_pattern<DT>(l_hi_c), km.mag_min) + 2;
    if (km.key_cut < 0) km.key_cut = 0;
    km.n_bins = key_top - km.key_cut + 1;
    if (km.n_bins < 1 || km.n_bins > 2 * p.phist_words) km.n_bins = 0;
  }
  if (part == 0 && tid == 0) p.row_state[row] = {serial_before, m, 0u, a_total, km.key_cut, km.n_bins, km.mag_min, listed_buckets};

  // ---- the slots, no barriers.  Two buffers take turns, so that the entries of the slot after this
  //      one are on their way while this one is worked on (a copy from one buffer to the other
  //      would have to wait for them).
  const uint64_t* tab = sm.exp2tab;
  auto work = [&](int s, const float (&in)[8]) {
    float e[8];
    bool done = false;
    if constexpr (DT == kDtypeBFloat16) {
      if (use_lut) {
        uint32_t address[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t fb = __float_as_uint(in[k]);
          address[k] = lut_entry_address((fb >> 16) & 0x7fffu, fb >> 31, lut_addr);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] = *(LdsF32)static_cast<uintptr_t>(address[k]);
        done = true;
      }
    }
    if (!done) {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float d = __builtin_fmaxf(in[k] * inv - m, -104.0f);  // expf is 0 below ln(2^-150); the core gives 0 at -104 too
        e[k] = expf_core(d, tab);
        if (WALK) e[k] = div_row(e[k], walk_div);
      }
    }
    const bool search = TOPP && __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(sh.top[s]))) >= list_cut;
    split_fold_slot<TOPP, DT>(p, row, s, e, in, sh.cls[s], list_cut, search, V, region, sh, km, ph);
  };
  if constexpr (FUSED) {
    if (s_mine < s_end) work(s_mine, held0);
    if (s_mine + kWaves < s_end) work(s_mine + kWaves, held1);
    if (s_mine + 2 * kWaves < s_end) work(s_mine + 2 * kWaves, held2);
    if (s_mine + 3 * kWaves < s_end) work(s_mine + 3 * kWaves, held3);
  } else {
    float l2[8];
    while (s_mine < s_end) {
      if (s_mine + kWaves < s_end) load_slot_lane<DT>(logits, s_mine + kWaves, lane, V, fill, l2, p.row.fused);
      work(s_mine, l);
      s_mine += kWaves;
      if (s_mine >= s_end) break;
      if (s_mine + kWaves < s_end) load_slot_lane<DT>(logits, s_mine + kWaves, lane, V, fill, l, p.row.fused);
      work(s_mine, l2);
      s_mine += kWaves;
    }
  }
  if (TOPP) {
    __syncthreads();
    if (tid == 0) p.list_count[static_cast<int64_t>(lrow) * kMaxRowWorkgroups + part] = sh.list_count;
    uint32_t* hist_out = p.hist + (static_cast<int64_t>(lrow) * p.row_wgs + part) * kHistBuckets;
    // (short lists: the buckets behind the listed ones are empty, and the finish kernel does not read them)
    const int n_hist = listed_buckets == kNoLists ? 0 : (listed_buckets != 0u ? static_cast<int>(listed_buckets) : kHistBuckets);
    for (int b = tid; b < n_hist; b += kBlock) hist_out[b] = sh.hist[b];
    if (kPatterns && km.n_bins > 0) {
      uint32_t* ph_out = p.phist + (static_cast<int64_t>(lrow) * p.row_wgs + part) * p.phist_words;
      for (int b = tid; b < (km.n_bins + 1) / 2; b += kBlock) ph_out[b] = ph[b];
    }
  }
  if (timers && part == 0 && tid == 0) {
    uint64_t* t = timers + static_cast<int64_t>(p.row.rows) * 8 + static_cast<int64_t>(lrow) * 4;
    t[0] = (c1 - c0) | (FUSED ? ((cf0 - c0) << 16) | ((cf1 - cf0) << 32) | ((cf2 - cf1) << 48) : 0ull);
    t[1] = c2 - c1;
    t[2] = c3 - c2;
    t[3] = wall_clock64() - c3;
  }
}

// After a fused launch that was not followed by its finish kernel: the next one gets a number of its own.
template <int DT>
__global__ void split_launch_number_kernel(uint32_t* arrive) {
  if (threadIdx.x == 0 && blockIdx.x == 0) next_launch_number(arrive);
}

// ---- finish ---------------------------------------------------------------------------------------
// One wave works a slot out from what pass 2 prepared: `bits` are the lane's 8 entries, pre_a /
// pre_b the inclusive prefix sums over the lanes of their increments under the ulp of binade kb_a /
// kb_b, tie_a / tie_b the lanes that hold a half-ulp tie under either.  While the running sum is in
// one of the two binades, differences of prefix sums commit every lane in front of the first one
// that holds a tie or behind which the sum would leave the binade; that lane adds its entries
// natively, and the walk goes on behind it (with the other binade's sums if the sum has moved
// there).  A sum in any other binade hands the remaining lanes to wave_resolve().  Returns with s
// the exact sum behind the slot.
__device__ __forceinline__ void resolve_lanes(float& s, const uint32_t (&bits)[8], uint32_t pre_a, uint32_t pre_b,
                                              uint64_t tie_a, uint64_t tie_b, uint32_t kb_a, uint32_t kb_b, int first, int V,
                                              uint32_t* inner = nullptr) {
  const int lane = threadIdx.x & 63;
  int cur = 0;
  // ---- the usual slot, in one go: the sum enters in binade a, no tie in front of the lane in which
  //      it leaves a, that lane's native adds land in binade b, nothing ties behind it and the rest
  //      stays inside b.  Anything else: the general rounds below, from the lane reached.
  {
    s = uniform_f32(s);
    const SumState ss = sum_state(s);
    if (static_cast<uint32_t>(ss.kb) == kb_a) {
      const uint32_t room = (1u << 24) - ss.S;
      const uint64_t over = __ballot(pre_a >= room);  // (prefix sums rise: the lanes from the crossing one on)
      if (over == 0ull) {
        if (tie_a == 0ull) {
          s = sum_value(ss.S + readlane_u32(pre_a, 63), ss.kb);
          return;
        }
      } else {
        const int j = __ffsll(static_cast<long long>(over)) - 1;
        if ((tie_a & ((1ull << j) - 1ull)) == 0ull) {
          const uint32_t S_j = ss.S + (j > 0 ? readlane_u32(pre_a, j - 1) : 0u);
          float sj = 0.0f;
          if (lane == j) {
            sj = sum_value(S_j, ss.kb);
#pragma unroll
            for (int k = 0; k < 8; ++k) sj = sj + __uint_as_float(bits[k]);  // (entries past the row hold 0)
          }
          s = readlane_f32(sj, j);
          cur = j + 1;
          if (cur == 64) return;
          const SumState s2 = sum_state(s);
          if (static_cast<uint32_t>(s2.kb) == kb_b && (tie_b >> cur) == 0ull) {
            const uint32_t rest = readlane_u32(pre_b, 63) - readlane_u32(pre_b, j);
            if (s2.S + rest < (1u << 24)) {
              s = sum_value(s2.S + rest, s2.kb);
              return;
            }
          }
        }
      }
    }
  }
  while (cur < 64) {
    if (inner) ++*inner;
    s = uniform_f32(s);
    const SumState ss = sum_state(s);
    const uint32_t K = static_cast<uint32_t>(ss.kb);
    if (K != kb_a && K != kb_b) {
      int found = -1;
      wave_resolve<8>(s, found, bits, first, V, __uint_as_float(0x7f800000u), cur);
      return;
    }
    const uint32_t pre = K == kb_a ? pre_a : pre_b;
    const uint64_t tie = K == kb_a ? tie_a : tie_b;
    const uint32_t done_before = cur > 0 ? readlane_u32(pre, cur - 1) : 0u;
    const uint32_t room = (1u << 24) - ss.S;
    const uint64_t over = __ballot(lane >= cur && pre - done_before >= room);
    const int j = next_event(tie | over, cur, 64);
    uint32_t S_j = ss.S;
    if (j > cur) S_j += readlane_u32(pre, j - 1) - done_before;
    if (j == 64) {
      s = sum_value(S_j, ss.kb);
      return;
    }
    float sj = 0.0f;
    if (lane == j) {
      sj = sum_value(S_j, ss.kb);
#pragma unroll
      for (int k = 0; k < 8; ++k) sj = sj + __uint_as_float(bits[k]);  // (entries past the row hold 0)
    }
    s = readlane_f32(sj, j);
    cur = j + 1;
  }
}

// A value every lane holds alike (loaded from one address, say), as a scalar: what is decided by it
// then runs on the scalar unit, and branches on it do not touch the execution mask.
__device__ __forceinline__ uint32_t uniform_u32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// LDS of a row while its sum is composed: the slot records, then one (even, odd) pair per record --
// the increment of the run of plain records that ends with the record, for either parity of the
// sum that enters the run (split_chain_prepare) --, then the prepared slots.
__host__ __device__ __forceinline__ size_t chain_pairs_offset(int ns) { return (static_cast<size_t>(ns) * sizeof(SlotRec) + 15) / 16 * 16; }
__host__ __device__ __forceinline__ size_t chain_rec_bytes(int ns) {
  return chain_pairs_offset(ns) + (static_cast<size_t>(ns) * sizeof(uint2) + 15) / 16 * 16;
}

// What the chain needs of a chunk of 64 records that does not depend on the running sum, worked
// out by any wave before the chain starts (sixteen waves do the chunks of a row side by side, where
// the chain's one wave would take them one after the other).  Every record is read under the
// binade pass 2 predicted for its slot.  A run is a stretch of plain records read under one
// binade: zero slots, stable slots (with or without a half-ulp tie inside), dual slots; it ends in
// front of a serial record, where the predicted binade changes, and with the chunk.  pairs[i] is
// the composition of the records of i's run up to and including i (a serial record adds nothing:
// it holds the total of the run in front of it).
__device__ __forceinline__ void split_chain_prepare(const SlotRec* recs, int ns, uint2* pairs, int first_chunk, int chunk_step) {
  const int lane = threadIdx.x & 63;
  for (int base = first_chunk * 64; base < ns; base += chunk_step * 64) {
    const int n = ns - base < 64 ? ns - base : 64;
    SlotRec r = {kSlotZero << 8, 0u, 0u, 0xffffffffu};
    if (lane < n) r = recs[base + lane];
    const uint32_t kind = (r.meta >> 8) & 7u, kb = r.meta & 255u, kb_in = (r.meta >> 16) & 255u;
    const bool runs = lane < n && (kind == kSlotZero || (kind == kSlotStable && kb == kb_in) ||
                                   (kind == kSlotDual && (kb == kb_in || kb + 1u == kb_in)));
    ParityInc v = {0u, 0u};
    if (runs && kind == kSlotStable) v = {r.even, r.odd};
    if (runs && kind == kSlotDual) v.even = v.odd = (kb == kb_in ? r.even : r.odd);
    v.even = v.even < (1u << 25) ? v.even : (1u << 25);  // (64 of them cannot wrap; 2^24 and up fails the chain's check)
    v.odd = v.odd < (1u << 25) ? v.odd : (1u << 25);
    // a lane starts a run when it is the chunk's first, when the lane in front of it is no part of a
    // run, or when it is read under another binade than the lane in front of it
    const uint64_t run_mask = __ballot(runs);
    const uint32_t kb_front = __builtin_amdgcn_update_dpp(0u, kb_in, 0x138, 0xf, 0xf, false);  // wave_shr:1
    const bool front_runs = lane > 0 && ((run_mask >> (lane - 1)) & 1ull) != 0ull;
    const bool head = lane == 0 || !front_runs || (runs && kb_in != kb_front);
    const uint64_t heads = __ballot(head);
    const int head_at = 63 - __clzll(static_cast<long long>(heads & ((2ull << lane) - 1ull)));  // (lane 0 is one)
    if (__ballot(v.even != v.odd) == 0ull) {
      // no tie in the chunk: one prefix sum, less what lies in front of the lane's run
      const uint32_t incl = wave_scan_inclusive_u32(v.even);
      const uint32_t front = static_cast<uint32_t>(__shfl(static_cast<int>(incl), head_at > 0 ? head_at - 1 : 0));
      v.even = v.odd = incl - (head_at > 0 ? front : 0u);
    } else {
      const ParityInc id = {0u, 0u};
#define ETS_SEG_STEP(CTRL, MASK, SRC)                              \
  {                                                                \
    const ParityInc o = dpp_parity_or_identity<CTRL, MASK>(v);     \
    v = compose((SRC) >= head_at ? o : id, v);                     \
  }
      ETS_SEG_STEP(0x111, 0xf, lane - 1)
      ETS_SEG_STEP(0x112, 0xf, lane - 2)
      ETS_SEG_STEP(0x114, 0xf, lane - 4)
      ETS_SEG_STEP(0x118, 0xf, lane - 8)
      ETS_SEG_STEP(0x142, 0xa, (lane & ~15) - 1)
      ETS_SEG_STEP(0x143, 0xc, 31)
#undef ETS_SEG_STEP
    }
    if (lane < n) pairs[base + lane] = make_uint2(v.even, v.odd);
  }
}

// The sequential softmax sum of one row (sampler.cpp:199-203) from the slot records, by ONE wave.
// `recs` (ns records) and `prep` (the first `n_prep` prepared slots) are in LDS.  Sixty-four
// records at a time, one per lane.  Under the binade K of the exact running sum a record is
// "plain" when its increment is known whatever the sum's parity: a zero slot, a stable slot folded
// for K without a tie, a dual slot folded for K or K - 1.  One prefix sum over the plain increments
// (redone only when K changes) gives, for every run of plain records, the exact sum behind each of
// them; a run is committed up to the first record that is not plain or behind which the sum
// would leave binade K.  That record is then worked out exactly -- a stable slot with a tie takes
// the increment for the sum's parity; a slot pass 2 prepared goes through resolve_lanes(); anything
// else is redone entry by entry from the logits -- and the walk goes on behind it.  Every step
// advances by at least one record.
template <int DT>
__device__ __forceinline__ float split_chain_walk(const SlotRec* recs, int ns, const PrepSlot* prep, uint32_t n_prep,
                                                  const char* logits, int V, float inv, float m, const uint64_t* tab,
                                                  const FusedOps& fused, uint64_t* stats, const RowDivisor* div,
                                                  float threshold, int* stop, int base0, int cur0, float s0);

// Slot `slot` of a multinomial row's probabilities p = fl(e / S) entry by entry from the logits, from
// running sum `from`, up to the first entry behind which the sum exceeds `threshold` (`hit`: its index).
template <int DT>
__device__ __forceinline__ float walk_redo(const char* logits, int slot, int V, float inv, float m, const uint64_t* tab,
                                           const FusedOps& fused, const RowDivisor& div, float threshold, float from, int& hit) {
  const int lane = threadIdx.x & 63;
  const float kInf = __uint_as_float(0x7f800000u);
  float l[8];
  uint32_t b[8];
  load_slot_lane<DT>(logits, slot, lane, V, inv < 0.0f ? kInf : -kInf, l, fused);
#pragma unroll
  for (int k = 0; k < 8; ++k) b[k] = __float_as_uint(div_row(expf_core(__builtin_fmaxf(l[k] * inv - m, -104.0f), tab), div));
  float t = from;
  wave_resolve<8>(t, hit, b, slot * kSlot + lane * 8, V, threshold);
  return t;
}

// WALKING: the records are those of a multinomial row's probabilities p = fl(e / S) (`div`), and the
// walk ends at the first entry behind which the running sum exceeds `threshold` (sampler.cpp:58-70):
// `*stop` is its index (-1: none), the value returned the sum there.  Increments are not negative, so
// the sum is compared with the threshold at the stops only; the record at which it is first exceeded
// is then looked up among the run's prefixes and redone entry by entry from the sum in front of it.
template <int DT, bool WALKING = false>
__device__ __forceinline__ float split_chain(const SlotRec* recs, const uint2* pairs, int ns, const PrepSlot* prep, uint32_t n_prep,
                                             const char* logits, int V, float inv, float m, const uint64_t* tab,
                                             const FusedOps& fused, uint64_t* stats = nullptr, const RowDivisor* div = nullptr,
                                             float threshold = 0.0f, int* stop = nullptr) {
  const int lane = threadIdx.x & 63;
  const float kInf = __uint_as_float(0x7f800000u);
  const float fill = inv < 0.0f ? kInf : -kInf;
  n_prep = uniform_u32(n_prep);
  float s = 0.0f;
  if (WALKING) *stop = -1;
  uint64_t c_start = 0;
  uint32_t n_iter = 0, n_generic = 0, n_prep_used = 0, n_tie = 0, n_inner = 0;
  uint64_t c_prep = 0;
  if (stats) c_start = wall_clock64();
  uint64_t ph_load = 0, ph_scan = 0, ph_walk = 0, ph_t = 0;
  for (int base = 0; base < ns; base += 64) {
    if (stats) ph_t = wall_clock64();
    SlotRec r = {kSlotZero << 8, 0u, 0u, 0xffffffffu};
    if (base + lane < ns) r = recs[base + lane];
    const uint32_t kind = (r.meta >> 8) & 7u, kb = r.meta & 255u;
    int cur = 0;
    if (base == 0 && readlane_u32(kind, 0) == kSlotExact) {  // pass 2 worked the first slot out
      s = __uint_as_float(readlane_u32(r.even, 0));
      cur = 1;
      if (WALKING && s > threshold) return walk_redo<DT>(logits, 0, V, inv, m, tab, fused, *div, threshold, 0.0f, *stop);
    }
    if (stats) {
      const uint64_t now = wall_clock64();
      ph_load += now - ph_t;
      ph_t = now;
    }
    // ---- the usual chunk, with as few instructions on this one wave's path as it takes (a wave on its
    //      own issues an instruction every few nanoseconds, whatever the instruction is).  The runs of
    //      plain records were added up beforehand (split_chain_prepare), each under the binade predicted
    //      for it and for either parity of the sum that enters it, so the walk goes from stop to stop
    //      on the scalar unit, the sum kept as (binade, integer).  A stop is a record that is no part
    //      of a run (a serial one), the last record in front of a change of the predicted binade, or
    //      the chunk's last.  At a stop the run that ends there is committed after checking that the
    //      sum entered it in the binade it was read under and stays inside it (increments are not
    //      negative, so the total decides for every prefix); a prepared slot without ties then takes
    //      the short form of resolve_lanes() below, any other serial record the general code.  A run
    //      that fails a check goes to the record-by-record loop further down, with the rest of the chunk.
    bool fast_ok = true;
    {
      const int n = ns - base < 64 ? ns - base : 64;
      const uint2 pr = lane < n ? pairs[base + lane] : make_uint2(0u, 0u);
      const uint32_t kb_in = (r.meta >> 16) & 255u;  // (a serial record: the binade predicted behind it)
      const bool runs = lane < n && (kind == kSlotZero || (kind == kSlotStable && kb == kb_in) ||
                                     (kind == kSlotDual && (kb == kb_in || kb + 1u == kb_in)));
      const uint64_t run_mask = __ballot(runs);
      const uint32_t kb_front = __builtin_amdgcn_update_dpp(0u, kb_in, 0x138, 0xf, 0xf, false);  // wave_shr:1
      const bool turn = lane > 0 && runs && ((run_mask >> (lane - 1)) & 1ull) != 0ull && kb_in != kb_front;  // a run starts here, behind another
      const uint64_t in_chunk = n < 64 ? (1ull << n) - 1ull : ~0ull;
      const uint64_t stop_mask = ((~run_mask) | (__ballot(turn) >> 1) | (1ull << (n - 1))) & in_chunk;
      // what kind of stop a lane is: kind | "prepared, in the float shortcut's range" << 3 (0 for a record that is part of a run)
      const uint32_t stop_info = runs ? 0u : (kind | (((r.meta >> 24) & 1u) << 3));
      uint32_t sb = uniform_u32(__float_as_uint(s));
      uint32_t K = sb >> 23 ? sb >> 23 : 1u;                          // sum_state()
      uint32_t S = sb >> 23 ? ((sb & 0x7fffffu) | 0x800000u) : sb;
      if (stats) {
        const uint64_t now = wall_clock64();
        ph_scan += now - ph_t;
        ph_t = now;
      }
      // WALKING: the sum exceeds the threshold behind one of the records first .. last of a run entered with (K, S)
      auto in_run = [&](int first, int last, uint32_t K_in, uint32_t S_in) {
        const uint32_t S_upto = S_in + ((S_in & 1u) ? pr.y : pr.x);
        const uint64_t cross = __ballot(lane >= first && lane <= last && sum_value(S_upto, static_cast<int>(K_in)) > threshold);
        const int q = static_cast<int>(uniform_u32(static_cast<uint32_t>(__builtin_ctzll(cross))));
        const float front = sum_value(q > first ? readlane_u32(S_upto, q - 1) : S_in, static_cast<int>(K_in));
        return walk_redo<DT>(logits, base + q, V, inv, m, tab, fused, *div, threshold, front, *stop);
      };
      while (cur < n) {
        cur = static_cast<int>(uniform_u32(static_cast<uint32_t>(cur)));
        const int t = static_cast<int>(uniform_u32(static_cast<uint32_t>(__builtin_ctzll(stop_mask & (~0ull << cur)))));  // (lane n - 1 is a stop)
        const uint32_t info_t = readlane_u32(stop_info, t);
        if (info_t == 0u) {
          // ---- a run ends with record t and nothing else happens there
          const uint32_t S_run = S + readlane_u32((S & 1u) ? pr.y : pr.x, t);
          if (K != readlane_u32(kb_in, cur) || S_run >= (1u << 24)) {
            fast_ok = false;
            break;
          }
          if (WALKING && sum_value(S_run, static_cast<int>(K)) > threshold) return in_run(cur, t, K, S);
          S = S_run;
          cur = t + 1;
          continue;
        }
        const uint32_t pi = readlane_u32(r.prep, t);
        // what a prepared slot needs is asked for before the run in front of it is committed
        const bool short_form = info_t == (kSlotSerial | 8u) && pi < n_prep;
        const PrepSlot& ps = prep[short_form ? pi : 0u];
        const float4 e0 = *reinterpret_cast<const float4*>(ps.e + lane * 8);
        const float4 e1 = *reinterpret_cast<const float4*>(ps.e + lane * 8 + 4);
        const uint32_t raw_a = ps.pre_a[lane], raw_b = ps.pre_b[lane];
        const uint32_t pre_a = raw_a & kPrepSum, pre_b = raw_b & kPrepSum;
        // ---- the run that ends in front of t (empty when lane cur is no part of a run: then t == cur)
        if ((run_mask >> cur) & 1ull) {
          const uint32_t S_run = S + readlane_u32((S & 1u) ? pr.y : pr.x, t);
          if (K != readlane_u32(kb_in, cur) || S_run >= (1u << 24)) {
            fast_ok = false;
            break;
          }
          if (WALKING && sum_value(S_run, static_cast<int>(K)) > threshold) return in_run(cur, t - 1, K, S);
          S = S_run;
        }
        cur = t;
        {
          // ---- record base + t, no part of a run
          const uint32_t K_front = K, S_front = S;
          bool done = false;
          if (short_form && K == (readlane_u32(r.meta, t) & 255u)) {
            // resolve_lanes() for a slot entered in the binade it was prepared for: the lanes in front
            // of the one in which the sum leaves the binade by their prefix sum (none of them may hold
            // a tie under that binade's ulp), that lane's eight entries natively (every lane adds; one
            // result is read), the lanes behind it by the prefix sums under the next binade (no tie
            // under its ulp among them)
            const uint32_t room = (1u << 24) - S;
            const uint64_t over = __ballot(pre_a >= room);
            const uint64_t tie_a = __ballot((raw_a & kPrepTie) != 0u), tie_b = __ballot((raw_b & kPrepTie) != 0u);
            if (over == 0ull) {
              if (tie_a == 0ull) {
                S += readlane_u32(pre_a, 63);
                done = true;
              }
            } else if ((tie_a & ((over & (0ull - over)) - 1ull)) == 0ull && (tie_b & ((~0ull << __builtin_ctzll(over)) << 1)) == 0ull) {
              const int jl = __builtin_ctzll(over);
              const uint32_t excl_a = __builtin_amdgcn_update_dpp(0u, pre_a, 0x138, 0xf, 0xf, false);  // wave_shr:1
              const uint32_t rest_b = readlane_u32(pre_b, 63) - pre_b;
              const uint32_t S_j = S + readlane_u32(excl_a, jl);
              float v = __uint_as_float(((K - 1u) << 23) + S_j);
              v = v + e0.x; v = v + e0.y; v = v + e0.z; v = v + e0.w;
              v = v + e1.x; v = v + e1.y; v = v + e1.z; v = v + e1.w;
              const uint32_t vb = readlane_u32(__float_as_uint(v), jl);
              const uint32_t S_b = ((vb & 0x7fffffu) | 0x800000u) + readlane_u32(rest_b, jl);
              if ((vb >> 23) == readlane_u32(kb_in, t) && S_b < (1u << 24)) {
                K = vb >> 23;
                S = S_b;
                done = true;
              }
            }
            if (done) ++n_prep_used;
          }
          if (!done) {
            // ---- the general code, from the exact sum in front of the record
            s = sum_value(S, static_cast<int>(K));
            const int slot = base + t;
            uint32_t bits[8];
            if (readlane_u32(kind, t) == kSlotSerial && pi < n_prep) {
              const PrepSlot& pg = prep[pi];
              const float4 g0 = *reinterpret_cast<const float4*>(pg.e + lane * 8);
              const float4 g1 = *reinterpret_cast<const float4*>(pg.e + lane * 8 + 4);
              bits[0] = __float_as_uint(g0.x); bits[1] = __float_as_uint(g0.y); bits[2] = __float_as_uint(g0.z); bits[3] = __float_as_uint(g0.w);
              bits[4] = __float_as_uint(g1.x); bits[5] = __float_as_uint(g1.y); bits[6] = __float_as_uint(g1.z); bits[7] = __float_as_uint(g1.w);
              if (uniform_u32(pg.usable)) {
                const uint64_t tie_a = (static_cast<uint64_t>(uniform_u32(pg.tie_a_hi)) << 32) | uniform_u32(pg.tie_a_lo);
                const uint64_t tie_b = (static_cast<uint64_t>(uniform_u32(pg.tie_b_hi)) << 32) | uniform_u32(pg.tie_b_lo);
                resolve_lanes(s, bits, pg.pre_a[lane] & kPrepSum, pg.pre_b[lane] & kPrepSum, tie_a, tie_b, uniform_u32(pg.kb_a), uniform_u32(pg.kb_b),
                              slot * kSlot + lane * 8, V, stats ? &n_inner : nullptr);
                ++n_prep_used;
              } else {
                int found = -1;
                wave_resolve<8>(s, found, bits, slot * kSlot + lane * 8, V, kInf);
                ++n_generic;
              }
            } else {
              float l[8];
              load_slot_lane<DT>(logits, slot, lane, V, fill, l, fused);
#pragma unroll
              for (int k = 0; k < 8; ++k) {
                float e = expf_core(__builtin_fmaxf(l[k] * inv - m, -104.0f), tab);
                if (WALKING) e = div_row(e, *div);
                bits[k] = __float_as_uint(e);
              }
              int found = -1;
              wave_resolve<8>(s, found, bits, slot * kSlot + lane * 8, V, kInf);
              ++n_generic;
            }
            sb = uniform_u32(__float_as_uint(s));
            K = sb >> 23 ? sb >> 23 : 1u;
            S = sb >> 23 ? ((sb & 0x7fffffu) | 0x800000u) : sb;
          }
          ++n_iter;
          if (WALKING && sum_value(S, static_cast<int>(K)) > threshold) {
            return walk_redo<DT>(logits, base + t, V, inv, m, tab, fused, *div, threshold, sum_value(S_front, static_cast<int>(K_front)), *stop);
          }
        }
        cur = t + 1;
      }
      s = sum_value(S, static_cast<int>(K));
      if (fast_ok) cur = 64;
    }
    if (stats) {
      const uint64_t now = wall_clock64();
      ph_walk += now - ph_t;
      ph_t = now;
    }
    // ---- record by record (a run in which the sum leaves its binade)
    if (WALKING && cur < 64) {
      return split_chain_walk<DT>(recs, ns, prep, n_prep, logits, V, inv, m, tab, fused, nullptr, div, threshold, stop, base, cur, s);
    }
    int K_scan = -1;
    uint32_t incl = 0u;
    uint64_t plain_mask = 0ull;
    while (cur < 64) {
      s = uniform_f32(s);
      const SumState ss = sum_state(s);
      const uint32_t K = static_cast<uint32_t>(ss.kb);
      if (ss.kb != K_scan) {
        const bool plain = kind == kSlotZero || (kind == kSlotStable && kb == K && r.even == r.odd) ||
                           (kind == kSlotDual && (kb == K || kb + 1u == K));
        const uint32_t inc = kind == kSlotZero ? 0u : ((kind == kSlotDual && kb != K) ? r.odd : r.even);
        incl = wave_scan_inclusive_u32(plain ? inc : 0u);  // 64 values of at most 2^26 each
        plain_mask = __ballot(plain);
        K_scan = ss.kb;
      }
      const uint64_t from_cur = ~0ull << cur;
      const uint64_t not_plain = ~plain_mask & from_cur;
      const int jn = not_plain ? __ffsll(static_cast<long long>(not_plain)) - 1 : 64;
      const uint32_t before = cur > 0 ? readlane_u32(incl, cur - 1) : 0u;
      const uint32_t S_upto = ss.S + (incl - before);
      const uint64_t over = __ballot(lane >= cur && lane < jn && S_upto >= (1u << 24));
      const int jo = over ? __ffsll(static_cast<long long>(over)) - 1 : 64;
      const int j = jn < jo ? jn : jo;
      if (j > cur) s = sum_value(readlane_u32(S_upto, j - 1), ss.kb);
      if (j == 64) break;
      // ---- record base + j, exactly
      const int slot = base + j;
      const uint32_t kind_j = readlane_u32(kind, j), kb_j = readlane_u32(kb, j);
      bool resolved = false;
      if (j == jn && kind_j == kSlotStable && kb_j == K) {  // a tie inside: the increment follows the parity
        const SumState sj = sum_state(s);
        const uint32_t inc = (sj.S & 1u) ? readlane_u32(r.odd, j) : readlane_u32(r.even, j);
        if (sj.S + inc < (1u << 24)) {
          s = sum_value(sj.S + inc, sj.kb);
          resolved = true;
          ++n_tie;
        }
      }
      if (!resolved) {
        const uint32_t pi = readlane_u32(r.prep, j);
        uint32_t bits[8];
        if (j == jn && kind_j == kSlotSerial && pi < n_prep) {
          const PrepSlot& ps = prep[pi];
          const float4 e0 = *reinterpret_cast<const float4*>(ps.e + lane * 8);
          const float4 e1 = *reinterpret_cast<const float4*>(ps.e + lane * 8 + 4);
          bits[0] = __float_as_uint(e0.x); bits[1] = __float_as_uint(e0.y); bits[2] = __float_as_uint(e0.z); bits[3] = __float_as_uint(e0.w);
          bits[4] = __float_as_uint(e1.x); bits[5] = __float_as_uint(e1.y); bits[6] = __float_as_uint(e1.z); bits[7] = __float_as_uint(e1.w);
          if (uniform_u32(ps.usable)) {
            const uint64_t tie_a = (static_cast<uint64_t>(uniform_u32(ps.tie_a_hi)) << 32) | uniform_u32(ps.tie_a_lo);
            const uint64_t tie_b = (static_cast<uint64_t>(uniform_u32(ps.tie_b_hi)) << 32) | uniform_u32(ps.tie_b_lo);
            const uint64_t cb = stats ? wall_clock64() : 0;
            resolve_lanes(s, bits, ps.pre_a[lane] & kPrepSum, ps.pre_b[lane] & kPrepSum, tie_a, tie_b, uniform_u32(ps.kb_a), uniform_u32(ps.kb_b), slot * kSlot + lane * 8, V,
                          stats ? &n_inner : nullptr);
            if (stats) c_prep += wall_clock64() - cb;
            ++n_prep_used;
          } else {
            int found = -1;
            wave_resolve<8>(s, found, bits, slot * kSlot + lane * 8, V, kInf);
            ++n_generic;
          }
        } else {
          float l[8];
          load_slot_lane<DT>(logits, slot, lane, V, fill, l, fused);
#pragma unroll
          for (int k = 0; k < 8; ++k) bits[k] = __float_as_uint(expf_core(__builtin_fmaxf(l[k] * inv - m, -104.0f), tab));
          int found = -1;
          wave_resolve<8>(s, found, bits, slot * kSlot + lane * 8, V, kInf);
          ++n_generic;
        }
      }
      cur = j + 1;
      ++n_iter;
    }
    if (stats && base == 0 && lane == 0) stats[5] = wall_clock64() - c_start;
  }
  if (stats && lane == 0) {
    stats[4] = 0;
    stats[6] = static_cast<uint64_t>(n_iter & 255u) | (static_cast<uint64_t>(n_generic & 255u) << 8) | ((ph_load & 0xffff) << 16) |
               ((ph_scan & 0xffff) << 32) | ((ph_walk & 0xffff) << 48);
    stats[7] = static_cast<uint64_t>(n_prep_used) | (static_cast<uint64_t>(n_tie) << 16) | (static_cast<uint64_t>(n_inner) << 32) |
               (c_prep << 48);
  }
  return uniform_f32(s);
}

// The chain of a multinomial row's probabilities record by record, from record `cur0` of the chunk
// at `base0` and the exact sum `s0` in front of it: where split_chain<DT, true>() goes on when a run
// does not stay in the binade predicted for it.  The walk stops at the first entry behind which the
// running sum exceeds `threshold` (sampler.cpp:58-70): `*stop` is its index (-1: none), the
// value returned the sum there.  Sums behind records are exact, so the first record behind which
// the sum exceeds the threshold holds that entry; it is redone entry by entry from the sum in front of it.
template <int DT>
__device__ __forceinline__ float split_chain_walk(const SlotRec* recs, int ns, const PrepSlot* prep, uint32_t n_prep,
                                                  const char* logits, int V, float inv, float m, const uint64_t* tab,
                                                  const FusedOps& fused, uint64_t* stats, const RowDivisor* div,
                                                  float threshold, int* stop, int base0, int cur0, float s0) {
  constexpr bool WALK = true;
  n_prep = uniform_u32(n_prep);
  const int lane = threadIdx.x & 63;
  const float kInf = __uint_as_float(0x7f800000u);
  float s = s0;
  auto redo = [&](int slot, float from, int& hit) {
    return walk_redo<DT>(logits, slot, V, inv, m, tab, fused, *div, threshold, from, hit);
  };
  *stop = -1;
  uint64_t c_start = 0;
  uint32_t n_iter = 0, n_generic = 0, n_prep_used = 0, n_tie = 0, n_inner = 0;
  uint64_t c_prep = 0;
  if (stats) c_start = wall_clock64();
  auto note = [&]() {
    if (stats && lane == 0) {
      stats[4] = wall_clock64() - c_start;
      stats[6] = static_cast<uint64_t>(n_iter) | (static_cast<uint64_t>(n_generic) << 32);
      stats[7] = static_cast<uint64_t>(n_prep_used) | (static_cast<uint64_t>(n_tie) << 16) | (static_cast<uint64_t>(n_inner) << 32) |
                 (c_prep << 48);
    }
  };
  for (int base = base0; base < ns; base += 64) {
    SlotRec r = {kSlotZero << 8, 0u, 0u, 0xffffffffu};
    if (base + lane < ns) r = recs[base + lane];
    const uint32_t kind = (r.meta >> 8) & 7u, kb = r.meta & 255u;
    int cur = base == base0 ? cur0 : 0;  // (a first slot that pass 2 worked out lies in front of cur0)
    // A stable slot with a half-ulp tie inside (one increment for an even sum in front of it, one for
    // an odd sum) counts as plain here, and the prefix is a composition of such pairs (compose()),
    // which follows the parity through the run; it is redone behind every record worked out
    // exactly while ties lie ahead.  (The composition costs several times the plain prefix sum of
    // split_chain(): it pays where ties are many, as among the probabilities of a 16-bit row, few
    // distinct values of which some sit on a tie every time they occur.)
    int K_scan = -1, cur_scan = -1;
    ParityInc incl = {0u, 0u};
    uint64_t plain_mask = 0ull, tie_mask = 0ull;
    while (cur < 64) {
      s = uniform_f32(s);
      const SumState ss = sum_state(s);
      const uint32_t K = static_cast<uint32_t>(ss.kb);
      {
        if (ss.kb != K_scan || (cur != cur_scan && (tie_mask >> cur) != 0ull)) {
          const bool plain = kind == kSlotZero || (kind == kSlotStable && kb == K) || (kind == kSlotDual && (kb == K || kb + 1u == K));
          ParityInc inc = {r.even, r.odd};
          if (kind == kSlotDual) inc.even = inc.odd = kb != K ? r.odd : r.even;
          if (kind == kSlotZero || !plain || lane < cur) inc = {0u, 0u};
          incl = wave_scan_inclusive(inc, lane);  // (saturating at 2^26)
          plain_mask = __ballot(plain);
          tie_mask = __ballot(plain && lane >= cur && inc.even != inc.odd);
          K_scan = ss.kb;
          cur_scan = cur;
          if (stats) n_tie += static_cast<uint32_t>(__popcll(tie_mask));
        }
      }
      const uint64_t from_cur = ~0ull << cur;
      const uint64_t not_plain = ~plain_mask & from_cur;
      const int jn = not_plain ? __ffsll(static_cast<long long>(not_plain)) - 1 : 64;
      const uint32_t incl_p = (ss.S & 1u) ? incl.odd : incl.even;
      const uint32_t before = cur > 0 ? readlane_u32(incl_p, cur - 1) : 0u;
      const uint32_t S_upto = ss.S + (incl_p - before);
      const uint64_t over = __ballot(lane >= cur && lane < jn && S_upto >= (1u << 24));
      const int jo = over ? __ffsll(static_cast<long long>(over)) - 1 : 64;
      const int j = jn < jo ? jn : jo;
      if (WALK) {
        // the first plain record of the run behind which the sum exceeds the threshold
        const uint64_t cross = __ballot(lane >= cur && lane < j && sum_value(S_upto, ss.kb) > threshold);
        if (cross != 0ull) {
          const int q = __ffsll(static_cast<long long>(cross)) - 1;
          if (q > cur) s = sum_value(readlane_u32(S_upto, q - 1), ss.kb);
          note();
          return redo(base + q, s, *stop);
        }
      }
      if (j > cur) s = sum_value(readlane_u32(S_upto, j - 1), ss.kb);
      if (j == 64) break;
      // ---- record base + j, exactly
      const int slot = base + j;
      const uint32_t kind_j = readlane_u32(kind, j);
      const float s_front = s;
      {
        const uint32_t pi = readlane_u32(r.prep, j);
        uint32_t bits[8];
        if (j == jn && kind_j == kSlotSerial && pi < n_prep) {
          const PrepSlot& ps = prep[pi];
          const float4 e0 = *reinterpret_cast<const float4*>(ps.e + lane * 8);
          const float4 e1 = *reinterpret_cast<const float4*>(ps.e + lane * 8 + 4);
          bits[0] = __float_as_uint(e0.x); bits[1] = __float_as_uint(e0.y); bits[2] = __float_as_uint(e0.z); bits[3] = __float_as_uint(e0.w);
          bits[4] = __float_as_uint(e1.x); bits[5] = __float_as_uint(e1.y); bits[6] = __float_as_uint(e1.z); bits[7] = __float_as_uint(e1.w);
          if (uniform_u32(ps.usable)) {
            const uint64_t tie_a = (static_cast<uint64_t>(uniform_u32(ps.tie_a_hi)) << 32) | uniform_u32(ps.tie_a_lo);
            const uint64_t tie_b = (static_cast<uint64_t>(uniform_u32(ps.tie_b_hi)) << 32) | uniform_u32(ps.tie_b_lo);
            const uint64_t cb = stats ? wall_clock64() : 0;
            resolve_lanes(s, bits, ps.pre_a[lane] & kPrepSum, ps.pre_b[lane] & kPrepSum, tie_a, tie_b, uniform_u32(ps.kb_a), uniform_u32(ps.kb_b), slot * kSlot + lane * 8, V,
                          stats ? &n_inner : nullptr);
            if (stats) c_prep += wall_clock64() - cb;
            ++n_prep_used;
          } else {
            int found = -1;
            wave_resolve<8>(s, found, bits, slot * kSlot + lane * 8, V, kInf);
            ++n_generic;
          }
        } else {
          int hit = -1;
          s = redo(slot, s, hit);
          if (WALK && hit >= 0) {
            *stop = hit;
            note();
            return s;
          }
          ++n_generic;
        }
      }
      if (WALK && s > threshold) {
        note();
        return redo(slot, s_front, *stop);
      }
      cur = j + 1;
      ++n_iter;
    }
    if (stats && base == 0 && lane == 0) stats[5] = wall_clock64() - c_start;
  }
  note();
  return uniform_f32(s);
}

// What the histogram says before the normaliser is known:
//   b_sel      the candidates in buckets 0 .. b_sel safely carry more than topp of the mass
//              whatever the exact normaliser turns out to be (-1: no such bucket);
//   n_sel      how many they are;
//   b_band     candidates in buckets below b_band reach the cutoff for certain;
//   n_certain  how many they are.
struct HistPlan {
  int b_sel, n_sel, b_band, n_certain;
};

// Shared by the phases of the finish kernel.
constexpr int kBandCap = 4096;
struct FinishShared {
  uint32_t count[kMaxRowWorkgroups];  // candidates per workgroup of pass 2
  uint32_t offset[kMaxRowWorkgroups + 1];
  uint32_t hist[kHistBuckets];        // the row's candidates by size
  uint64_t sel[64];                   // the candidates of the largest buckets (exp bits << 32 | index)
  uint32_t band[kBandCap];            // exp bits of the candidates that may or may not reach the cutoff
  uint32_t sel_count, band_count;
  uint32_t overflow;
  HistPlan plan;
  FusedOps fused;  // (the draw functions are calls: they read the launch's processors from here)
  float pre_sum[4];  // softmax sums of the rows of a unit (kChainRows), composed before their draws
};
constexpr int kChainRows = 4;

// By the whole workgroup, two buckets per lane; `plan_out` is LDS.  Ends with a barrier.
__device__ __forceinline__ HistPlan split_plan(const uint32_t* hist, float a_total, float topp, float cutoff, int V,
                                               HistPlan* plan_out, BlockScratch& sm) {
  static_assert(kHistBuckets == 2 * kBlock, "two buckets per lane");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const float target = (topp * 1.004f + 1e-6f) * a_total * (1.0f + split_eps(V));
  const float cut_hi = cutoff * a_total * (1.0f + split_eps(V)) * 1.001f;
  const int b_band = (cut_hi <= 1.0f && cut_hi > 0.0f) ? static_cast<int>(hist_bucket(__float_as_uint(cut_hi))) : 0;
  const int b0 = 2 * tid;
  const uint32_t c0 = hist[b0], c1 = hist[b0 + 1];
  const float m0 = static_cast<float>(c0) * hist_edge(b0 + 1), m1 = static_cast<float>(c1) * hist_edge(b0 + 2);
  const uint32_t certain = (b0 < b_band ? c0 : 0u) + (b0 + 1 < b_band ? c1 : 0u);
  const uint32_t inclC = wave_scan_inclusive_u32(c0 + c1);
  const float inclM = wave_scan_inclusive_f32(m0 + m1, lane);
  const uint32_t certain_w = wave_sum_u32(certain);
  if (lane == 63) {
    sm.red_u[wave] = inclC;
    sm.red_f[wave] = inclM;
  }
  if (lane == 0) sm.first_flag[wave] = static_cast<int>(certain_w);
  if (tid == 0) *plan_out = {-1, 0, b_band, 0};
  __syncthreads();
  uint32_t cnt_before = 0u;
  float mass_before = 0.0f;
  int n_certain = 0;
  for (int w = 0; w < kWaves; ++w) {
    if (w < wave) {
      cnt_before += sm.red_u[w];
      mass_before += sm.red_f[w];
    }
    n_certain += sm.first_flag[w];
  }
  // the lane in which the mass reaches the target (at most one: `below` is what lies in front of it)
  const float upto = mass_before + inclM;
  const float below = upto - (m0 + m1);
  if (upto >= target && !(below >= target)) {
    const bool first = below + m0 >= target;
    plan_out->b_sel = first ? b0 : b0 + 1;
    plan_out->n_sel = static_cast<int>(cnt_before + inclC - (first ? c1 : 0u));
  }
  if (tid == 0) plan_out->n_certain = n_certain;
  __syncthreads();
  return *plan_out;
}

// ---- top-p draw of 16-bit rows by runs of equal probability ----------------------------------------
// A row of 16-bit logits has at most 65536 distinct probabilities, and the reference's sorted
// candidate array (sampler.cpp:145-148) is the row's bit patterns in falling order, each repeated
// as often as it occurs (among equal probabilities the tie rule orders by token index).  Its two
// CDF walks (sampler.cpp:150-170) therefore add runs of equal values, and c sequential additions
// of the same p have a closed form inside one binade of the running sum.  Pass 2 counted the
// entries per pattern; here the runs are walked with the scheme of the softmax sum: approximate
// cumulative masses place every group of 64 patterns inside a binade, each group is folded once
// under that binade's ulp, one wave composes the groups from the exact running sum and works out
// the few groups in which the sum changes binade, meets a half-ulp tie or crosses the threshold.
// No sort, no gather; the token is the k-th occurrence, in index order, of the probability the
// walk stops at.

struct RunSlotRec {
  uint32_t meta;  // kind << 8 | kb
  uint32_t inc_a, inc_b;
  uint32_t pad;
};

// Where counter word w lies in LDS: a pad word behind every 32, so that lanes that each walk a
// stretch of bins of their own (32 bins are 16 words) do not all read from the same two banks.
__device__ __forceinline__ int run_word(int w) { return w + (w >> 5); }

// Probability and count of the bin at sorted position q (bins in falling key order).
template <int DT>
struct RunBins {
  const uint32_t* cnt;  // LDS: two 16-bit counters per word, at run_word()
  int key_cut, n_bins, mag_min;
  float inv, m, cutoff;
  RowDivisor div;
  const uint64_t* tab;
  __device__ __forceinline__ void at(int q, float& prob, uint32_t& count) const {
    prob = 0.0f;
    count = 0u;
    if (q < n_bins) {
      const int bin = n_bins - 1 - q;
      const float l = pattern_value<DT>(key_pattern(key_cut + bin, mag_min));
      const float e = expf_core(__builtin_fmaxf(l * inv - m, -104.0f), tab);
      prob = div_row(e, div);
      const uint32_t c = (cnt[run_word(bin >> 1)] >> ((bin & 1) << 4)) & 0xffffu;
      count = (prob >= cutoff) ? c : 0u;  // sampler.cpp:137-143
    }
  }
  // The same with the probability from the hardware's exp2 (relative error below 1e-5): enough to
  // place the cumulative masses; the count is exact (a bin whose probability is within 1e-3 of
  // the cutoff is evaluated exactly).
  __device__ __forceinline__ void at_approx(int q, float& prob, uint32_t& count) const {
    prob = 0.0f;
    count = 0u;
    if (q < n_bins) {
      const int bin = n_bins - 1 - q;
      const uint32_t c = (cnt[run_word(bin >> 1)] >> ((bin & 1) << 4)) & 0xffffu;
      if (c != 0u) {
        const float l = pattern_value<DT>(key_pattern(key_cut + bin, mag_min));
        const float x = __builtin_fmaxf(l * inv - m, -104.0f);
        prob = fast_exp2(x * kLog2e) * static_cast<float>(div.recip);
        bool in = prob >= cutoff;
        if (__builtin_fabsf(prob - cutoff) <= cutoff * 1e-3f) in = div_row(expf_core(x, tab), div) >= cutoff;
        count = in ? c : 0u;
      }
    }
  }
};

// One wave works the 64 bins of group t out exactly from running sum s; `before` is the number of
// candidates in front of the group.  Returns the sorted position (0-based) behind which s first
// exceeds T, or -1 (then s is the sum behind the group).
template <int DT>
__device__ __forceinline__ int resolve_run_group(float& s, int t, uint32_t before, float T, const RunBins<DT>& bins) {
  const int lane = threadIdx.x & 63;
  float prob;
  uint32_t count;
  bins.at(64 * t + lane, prob, count);
  const uint32_t cnt_incl = wave_scan_inclusive_u32(count);
  int cur = 0;
  while (cur < 64) {
    s = uniform_f32(s);
    const SumState ss = sum_state(s);
    const bool shortcut = ss.kb >= 64 && ss.kb <= 250;
    const float scale = shortcut ? __uint_as_float(static_cast<uint32_t>(277 - ss.kb) << 23) : 0.0f;
    const float tq = prob * scale;
    const float rq = __builtin_rintf(tq);
    const bool live = lane >= cur && count != 0u;
    // a lane is an event when its adds depend on their order or cannot be counted in ulps
    const bool odd_one = live && (!shortcut || !(tq < 16777216.0f) || __builtin_fabsf(tq - rq) == 0.5f);
    const float incf = live && !odd_one ? __builtin_fminf(rq * static_cast<float>(count), 33554432.0f) : 0.0f;
    const uint32_t incl = wave_scan_inclusive_u32(static_cast<uint32_t>(incf));
    uint32_t limit = 1u << 24;
    const float tt = T * scale;
    if (shortcut && tt < 16777216.0f) {
      const uint32_t Tn = tt >= 0.0f ? static_cast<uint32_t>(__builtin_floorf(tt)) + 1u : 0u;
      limit = Tn < limit ? Tn : limit;
    }
    const uint32_t room = limit > ss.S ? limit - ss.S : 0u;
    const int j = next_event(__ballot(odd_one || (live && incl >= room)), cur, 64);
    uint32_t S_j = ss.S;
    if (j > 0) S_j += readlane_u32(incl, j > 63 ? 63 : j - 1);  // lanes below cur hold 0
    if (j == 64) {
      s = sum_value(S_j, ss.kb);
      return -1;
    }
    float sj = 0.0f;
    uint32_t hit = 0u;
    if (lane == j) {
      sj = sum_value(S_j, ss.kb);
      hit = run_walk(sj, prob, count, T);
    }
    s = readlane_f32(sj, j);
    hit = readlane_u32(hit, j);
    if (hit != 0u) {
      const uint32_t in_front = readlane_u32(cnt_incl - count, j);
      return static_cast<int>(before + in_front + hit - 1u);
    }
    cur = j + 1;
  }
  return -1;
}

struct RunWalk {
  int position;  // sorted position behind which the sum first exceeded the threshold, or -1
  float sum;     // the sum there (or behind the last group walked)
};

// Needs p.row.lds_keys * 8 bytes of LDS at `lds` (the key buffer); every lane of the workgroup
// calls it.  Returns false when the runs cannot be used (no pattern histogram, a counter that
// overflowed, probabilities that do not fall along the patterns): the caller sorts instead.
// What draw_topp_runs() needs of the launch and the row, by value (a reference to the kernel's
// argument block would move that block to private memory for the whole kernel).
struct RunArgs {
  const uint32_t* phist;  // this row's first region
  int32_t phist_words, row_wgs, lds_keys, ns;
  int32_t key_cut, n_bins, mag_min;
  uint32_t expected;      // candidates pass 2 listed: what the counters must add up to
  float m;
  const FusedOps* fused;  // (LDS)
};

template <int DT>
__device__ __noinline__ bool draw_topp_runs(RunArgs a, const char* logits, int V, float inv, float S, float cutoff, float topp,
                                            float coin, uint64_t* lds, RowDebug& dbg, int32_t& token, BlockScratch& sm) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n_bins = a.n_bins;
  if (n_bins <= 0) return false;
  const int n_groups = (n_bins + 63) / 64;
  const int words = (n_bins + 1) / 2;
  // ---- LDS: counters | group records | exact sums at group boundaries | candidates in front of
  //      each group | approximate masses in front of each group
  uint32_t* cnt = reinterpret_cast<uint32_t*>(lds);
  RunSlotRec* recs = reinterpret_cast<RunSlotRec*>(cnt + (run_word(words) + 4) / 4 * 4);
  float* sbound = reinterpret_cast<float*>(recs + n_groups);
  uint32_t* cbound = reinterpret_cast<uint32_t*>(sbound + n_groups + 1);
  float* mbound = reinterpret_cast<float*>(cbound + n_groups + 1);
  float* gfirst = mbound + n_groups + 1;  // probability of a group's first and last candidate bin (-1: none)
  float* glast = gfirst + n_groups;
  char* const lds_end = reinterpret_cast<char*>(lds) + static_cast<size_t>(a.lds_keys) * 8;
  if (reinterpret_cast<char*>(glast + n_groups) > lds_end) return false;
  // ... | groups in which the sum is expected to change binade, prepared for the walk (kSideGroups
  //      of them, if that much is left: the number taken, the groups, per bin the prefix sums of the
  //      increments under the two ulps and the probability)
  constexpr int kSideGroups = 24;
  uint32_t* side_n = reinterpret_cast<uint32_t*>(glast + n_groups);
  uint32_t* side_group = side_n + 1;
  uint32_t* side_a = side_group + kSideGroups;
  uint32_t* side_b = side_a + kSideGroups * 64;
  float* side_p = reinterpret_cast<float*>(side_b + kSideGroups * 64);
  const int side_cap = reinterpret_cast<char*>(side_p + kSideGroups * 64) <= lds_end ? kSideGroups : 0;
  if (side_cap > 0 && tid == 0) *side_n = 0u;  // (barriers follow before pass B counts)
  // ---- the workgroups' counters, added up (16-bit halves add without carries unless one overflows,
  //      which the totals give away)
  {
    const uint32_t* in = a.phist;
    uint32_t sum16 = 0u;
    if (a.row_wgs == 1) {
      // one workgroup's counters: a copy, eight words of a lane requested at a time
      for (int w0 = tid; w0 < words; w0 += 8 * kBlock) {
        uint32_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = w0 + k * kBlock < words ? in[w0 + k * kBlock] : 0u;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if (w0 + k * kBlock < words) cnt[run_word(w0 + k * kBlock)] = v[k];
          sum16 += (v[k] & 0xffffu) + (v[k] >> 16);
        }
      }
    } else
    for (int w = tid; w < words; w += kBlock) {
      uint32_t lo = 0u, hi = 0u;
      for (int g = 0; g < a.row_wgs; g += 4) {
        uint32_t v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = in[static_cast<int64_t>(g + k < a.row_wgs ? g + k : g) * a.phist_words + w];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (g + k < a.row_wgs) {
            lo += v[k] & 0xffffu;
            hi += v[k] >> 16;
          }
        }
      }
      const bool fits = lo <= 0xffffu && hi <= 0xffffu;
      cnt[run_word(w)] = fits ? (lo | (hi << 16)) : 0u;
      sum16 += fits ? lo + hi : 0x40000000u;  // (spoils the total)
    }
    sum16 = wave_sum_u32(sum16);
    if (lane == 0) sm.red_u[wave] = sum16;
    __syncthreads();
    uint32_t total = 0u;
    for (int w = 0; w < kWaves; ++w) total += sm.red_u[w];
    __syncthreads();
    if (total != a.expected) return false;
  }
  const RunBins<DT> bins = {cnt, a.key_cut, n_bins, a.mag_min, inv, a.m, cutoff, row_divisor(S), sm.exp2tab};
  // ---- pass A: per group the candidates (exactly) and their approximate mass
  //      Eight lanes take a group, eight bins each, one bin after the other: no sums over a whole wave
  //      (a wave to a group would spend most of its instructions on them), and the groups go round
  //      the workgroup's lanes evenly.
  constexpr int kPer = 8;  // bins of a lane; 64 / kPer lanes to a group
  const int n_units = n_groups * (64 / kPer);
  for (int u0 = 0; u0 < n_units; u0 += kBlock) {
    const int u = u0 + tid;
    const int t = u / (64 / kPer);
    float mass = 0.0f;
    uint32_t c = 0u;
    if (u < n_units) {
#pragma unroll 2
      for (int i = 0; i < kPer; ++i) {
        float prob;
        uint32_t count;
        bins.at_approx(kPer * u + i, prob, count);
        mass += static_cast<float>(count) * prob;
        c += count;
      }
    }
#pragma unroll
    for (int d = 1; d < 64 / kPer; d <<= 1) {
      mass += __shfl_xor(mass, d);
      c += static_cast<uint32_t>(__shfl_xor(static_cast<int>(c), d));
    }
    if (u < n_units && (lane & (64 / kPer - 1)) == 0) {
      mbound[t + 1] = mass;
      cbound[t + 1] = c;
    }
  }
  __syncthreads();
  // prefix sums over the groups (at most kBlock of them)
  {
    const float mine = tid < n_groups ? mbound[tid + 1] : 0.0f;
    const uint32_t mine_c = tid < n_groups ? cbound[tid + 1] : 0u;
    const float incl = wave_scan_inclusive_f32(mine, lane);
    const uint32_t incl_c = wave_scan_inclusive_u32(mine_c);
    __syncthreads();
    if (lane == 63) {
      sm.red_f[wave] = incl;
      sm.red_u[wave] = incl_c;
    }
    __syncthreads();
    float before = 0.0f;
    uint32_t before_c = 0u;
    for (int w = 0; w < wave; ++w) {
      before += sm.red_f[w];
      before_c += sm.red_u[w];
    }
    if (tid < n_groups) {
      mbound[tid + 1] = before + incl;
      cbound[tid + 1] = before_c + incl_c;
    }
    if (tid == 0) {
      mbound[0] = 0.0f;
      cbound[0] = 0u;
    }
    __syncthreads();
  }
  if (n_groups > kBlock) return false;
  const uint32_t n0 = cbound[n_groups];
  dbg.n_candidates = static_cast<int>(n0);
  if (n0 == 0u) {
    token = -1;  // the reference reads probindex[-1] here
    return true;
  }
  // ---- pass B: the exact probabilities, group by group, as far as the walk can get (cumulative mass
  //      up to topp).  They must not rise along the sorted positions (a larger logit with a smaller
  //      probability would not be where the reference's sort puts it).  Every group is folded once,
  //      under the ulp(s) of the binade(s) the cumulative sum can be in while it passes the group;
  //      one that may hold the place where the sum exceeds topp, that spans more than two binades
  //      or in which an entry ties is left to the ordered walk.
  //      As in pass A eight lanes take a group, eight bins each in order, and put their parts together.
  bool rising = false;
  for (int u0 = 0; u0 < n_units; u0 += kBlock) {
    const int u = u0 + tid;
    const int t = u / (64 / kPer);
    const bool valid = u < n_units;
    const uint32_t c_in = valid ? cbound[t] : 0u, c_out = valid ? cbound[t + 1] : 0u;
    RunSlotRec rec = {kSlotZero << 8, 0u, 0u, 0u};
    bool walked = false, folded = false;
    uint32_t kb_lo = 0u, kb_hi = 0u;
    if (c_out != c_in) {
      const float eps_in = static_cast<float>(c_in) * (1.02f / 16777216.0f) + 6e-5f;
      const float eps_out = static_cast<float>(c_out) * (1.02f / 16777216.0f) + 6e-5f;
      const float lo = mbound[t] * (1.0f - eps_in), hi = mbound[t + 1] * (1.0f + eps_out);
      kb_lo = __float_as_uint(lo > 0.0f ? lo : 0.0f) >> 23;
      kb_hi = __float_as_uint(hi) >> 23;
      const bool near_topp = !(hi < topp * 0.9999f);  // (the walk ends there: nothing behind it is needed)
      rec.meta = (kSlotSerial << 8) | (kb_lo & 255u);
      walked = !(lo > topp * 1.001f);  // (a group the walk cannot reach stays "serial": worked out exactly if reached after all)
      folded = walked && !near_topp && lo > 0.0f && kb_lo >= 70u && kb_hi <= 250u && kb_hi <= kb_lo + 1u;
    }
    // this lane's part of the group: its first and last candidate bin, whether the probabilities
    // rise from one candidate bin to the next, the increments under the two ulps
    float first_p = -1.0f, last_p = -1.0f;
    bool up = false, tie = false;
    uint32_t ia = 0u, ib = 0u;
    if (walked) {
      const float scale_a = __uint_as_float((277u - kb_lo) << 23), scale_b = __uint_as_float((276u - kb_lo) << 23);
      for (int i = 0; i < kPer; ++i) {
        float prob;
        uint32_t count;
        bins.at(kPer * u + i, prob, count);
        if (count != 0u) {
          if (first_p < 0.0f) first_p = prob;
          if (last_p >= 0.0f && prob > last_p) up = true;
          last_p = prob;
          if (folded) {
            const float ta = prob * scale_a, tb = prob * scale_b;
            const float ra = __builtin_rintf(ta), rb = __builtin_rintf(tb);
            tie = tie || __builtin_fabsf(ta - ra) == 0.5f || (kb_hi != kb_lo && __builtin_fabsf(tb - rb) == 0.5f);
            const float fc = static_cast<float>(count);
            ia += static_cast<uint32_t>(__builtin_fminf(ra * fc, 33554432.0f));  // (64 of them to a group: below 2^31)
            ib += static_cast<uint32_t>(__builtin_fminf(rb * fc, 33554432.0f));
          }
        }
      }
    }
    // the parts of a group, put together pair by pair (of two partners the one with the lower lane
    // holds the earlier bins); every lane of the group ends up with the whole
#pragma unroll
    for (int d = 1; d < 64 / kPer; d <<= 1) {
      const float o_first = __shfl_xor(first_p, d), o_last = __shfl_xor(last_p, d);
      const bool o_up = __shfl_xor(up ? 1 : 0, d) != 0, o_tie = __shfl_xor(tie ? 1 : 0, d) != 0;
      ia += static_cast<uint32_t>(__shfl_xor(static_cast<int>(ia), d));
      ib += static_cast<uint32_t>(__shfl_xor(static_cast<int>(ib), d));
      const bool left = (lane & d) == 0;
      const float l_first = left ? first_p : o_first, l_last = left ? last_p : o_last;
      const float r_first = left ? o_first : first_p, r_last = left ? o_last : last_p;
      up = up || o_up || (l_last >= 0.0f && r_first >= 0.0f && r_first > l_last);
      tie = tie || o_tie;
      first_p = l_first >= 0.0f ? l_first : r_first;
      last_p = r_last >= 0.0f ? r_last : l_last;
    }
    if (valid && (lane & (64 / kPer - 1)) == 0) {
      if (folded && !tie) {
        rec.meta = ((kb_hi == kb_lo ? kSlotStable : kSlotDual) << 8) | kb_lo;
        rec.inc_a = ia < kSat ? ia : kSat;
        rec.inc_b = ib < kSat ? ib : kSat;
        if (kb_hi != kb_lo && side_cap > 0) {  // the sum is expected to change binade inside: prepared below
          const uint32_t d = atomicAdd(side_n, 1u);
          if (d < static_cast<uint32_t>(side_cap)) {
            side_group[d] = static_cast<uint32_t>(t);
            rec.pad = d + 1u;
          }
        }
      }
      recs[t] = rec;
      gfirst[t] = first_p;
      glast[t] = last_p;
    }
    if (up) rising = true;
  }
  {
    const uint64_t any = __ballot(rising);
    if (lane == 0) sm.red_u[wave] = any ? 1u : 0u;
  }
  __syncthreads();
  {
    uint32_t bad = 0u;
    for (int w = 0; w < kWaves; ++w) bad |= sm.red_u[w];
    // ... and from group to group: a group's first candidate against the last one in front of it
    if (wave == 0) {
      float prev_last = __uint_as_float(0x7f800000u);
      bool up = false;
      for (int base = 0; base < n_groups; base += 64) {
        const int g = base + lane;
        const float f = g < n_groups ? gfirst[g] : -1.0f;
        const float l = g < n_groups ? glast[g] : -1.0f;
        const uint64_t occ = __ballot(f >= 0.0f);
        const uint64_t below = occ & ((1ull << lane) - 1ull);
        const int prev = below ? 63 - __clzll(static_cast<long long>(below)) : lane;
        float before = __shfl(l, prev);
        if (!below) before = prev_last;
        if (f >= 0.0f && f > before) up = true;
        if (occ) prev_last = readlane_f32(l, 63 - __clzll(static_cast<long long>(occ)));
      }
      const uint64_t any = __ballot(up);
      if (lane == 0) sm.flag = any ? 1 : 0;
    }
    __syncthreads();
    bad |= static_cast<uint32_t>(sm.flag);
    __syncthreads();
    if (bad != 0u) return false;
  }
  // ---- the groups in which the sum is expected to change binade (kb -> kb + 1), a wave each: per bin
  //      the exact probability and the prefix sums of the increments under either ulp.  The walk
  //      then finds the bin in which the sum leaves binade kb from the first prefix sums, adds that
  //      bin's copies in closed form and the bins behind it from the second.  (No bin of a folded
  //      group ties under either ulp.)  A group with a bin whose increment is not below 2^25 is not
  //      prepared.
  if (side_cap > 0) {
    const int n_side = static_cast<int>(*side_n < static_cast<uint32_t>(side_cap) ? *side_n : static_cast<uint32_t>(side_cap));
    for (int d = wave; d < n_side; d += kWaves) {
      const int t = static_cast<int>(side_group[d]);
      const uint32_t kb = recs[t].meta & 255u;
      float prob;
      uint32_t count;
      bins.at(64 * t + lane, prob, count);
      const float fc = static_cast<float>(count);
      const float va = __builtin_rintf(prob * __uint_as_float((277u - kb) << 23)) * fc;
      const float vb = __builtin_rintf(prob * __uint_as_float((276u - kb) << 23)) * fc;
      const bool big = !(va < 33554432.0f) || !(vb < 33554432.0f);
      const uint32_t pre_a = wave_scan_inclusive_u32(big ? 0u : static_cast<uint32_t>(va));
      const uint32_t pre_b = wave_scan_inclusive_u32(big ? 0u : static_cast<uint32_t>(vb));
      side_a[d * 64 + lane] = pre_a;
      side_b[d * 64 + lane] = pre_b;
      side_p[d * 64 + lane] = count != 0u ? prob : 0.0f;
      if (__ballot(big) != 0ull && lane == 0) recs[t].pad = 0u;
    }
    __syncthreads();
  }
  // ---- walk 1 (sampler.cpp:150-158): the groups in order until the sum exceeds topp.  One wave.
  if (wave == 0) {
    float s = 0.0f;
    int found = -1;
    int last_group = n_groups - 1;
    if (lane == 0) sbound[0] = 0.0f;
    for (int base = 0; base < n_groups && found < 0; base += 64) {
      RunSlotRec r = {kSlotZero << 8, 0u, 0u, 0u};
      if (base + lane < n_groups) r = recs[base + lane];
      const uint32_t kind = (r.meta >> 8) & 7u, kb = r.meta & 255u;
      int cur = 0;
      int K_scan = -1;
      uint32_t incl = 0u;
      uint64_t plain_mask = 0ull;
      while (cur < 64 && found < 0) {
        s = uniform_f32(s);
        const SumState ss = sum_state(s);
        const uint32_t K = static_cast<uint32_t>(ss.kb);
        if (ss.kb != K_scan) {
          const bool plain = kind == kSlotZero || (kind == kSlotStable && kb == K) || (kind == kSlotDual && (kb == K || kb + 1u == K));
          const uint32_t inc = kind == kSlotZero ? 0u : ((kind == kSlotDual && kb != K) ? r.inc_b : r.inc_a);
          incl = wave_scan_inclusive_u32(plain ? inc : 0u);
          plain_mask = __ballot(plain);
          K_scan = ss.kb;
        }
        const uint64_t not_plain = ~plain_mask & (~0ull << cur);
        const int jn = not_plain ? __ffsll(static_cast<long long>(not_plain)) - 1 : 64;
        const uint32_t before = cur > 0 ? readlane_u32(incl, cur - 1) : 0u;
        const uint32_t S_upto = ss.S + (incl - before);
        // the sum must stay inside the binade and must not exceed topp inside a folded group
        uint32_t limit = 1u << 24;
        if (ss.kb >= 64 && ss.kb <= 250) {
          const float tt = topp * __uint_as_float(static_cast<uint32_t>(277 - ss.kb) << 23);
          if (tt < 16777216.0f) {
            const uint32_t Tn = static_cast<uint32_t>(__builtin_floorf(tt)) + 1u;
            limit = Tn < limit ? Tn : limit;
          }
        }
        const uint64_t over = __ballot(lane >= cur && lane < jn && S_upto >= limit);
        const int jo = over ? __ffsll(static_cast<long long>(over)) - 1 : 64;
        const int j = jn < jo ? jn : jo;
        if (lane >= cur && lane < j && base + lane < n_groups) sbound[base + lane + 1] = sum_value(S_upto, ss.kb);
        if (j > cur) s = sum_value(readlane_u32(S_upto, j - 1), ss.kb);
        if (j == 64) break;
        const int t = base + j;
        if (t >= n_groups) break;
        // ---- a prepared group folded for this binade that the sum leaves inside it, topp far away
        const uint32_t side = readlane_u32(r.pad, j);
        if (j == jo && side != 0u && readlane_u32(kb, j) == K && limit == (1u << 24) && K < 250u) {
          const int d = static_cast<int>(side) - 1;
          const uint32_t pre_a = side_a[d * 64 + lane], pre_b = side_b[d * 64 + lane];
          const SumState sj = sum_state(uniform_f32(s));
          const uint32_t room = (1u << 24) - sj.S;
          const uint64_t out = __ballot(pre_a >= room);
          if (out != 0ull && sj.kb == ss.kb) {
            const int jl = static_cast<int>(uniform_u32(static_cast<uint32_t>(__builtin_ctzll(out))));
            const uint32_t front_a = jl > 0 ? readlane_u32(pre_a, jl - 1) : 0u;
            const uint32_t S_j = sj.S + front_a;  // below 2^24
            const float pl = side_p[d * 64 + jl];
            // bin jl: c copies of pl, each n_a under this ulp (their product is the bin's increment)
            const float scale_a = __uint_as_float((277u - K) << 23), scale_b = __uint_as_float((276u - K) << 23);
            const float n_af = __builtin_rintf(pl * scale_a);
            const uint32_t n_a = static_cast<uint32_t>(n_af), n_b = static_cast<uint32_t>(__builtin_rintf(pl * scale_b));
            const uint32_t inc_l = readlane_u32(pre_a, jl) - front_a;  // c * n_a, at least the room left: n_a is not 0
            // copies after which the sum is still below 2^24 ulps: floor((2^24 - S_j - 1) / n_a), fewer than c
            const uint32_t x = (1u << 24) - S_j - 1u;
            uint32_t stay = static_cast<uint32_t>(static_cast<float>(x) / n_af);
            if (stay * n_a > x) --stay;
            if ((stay + 1u) * n_a <= x) ++stay;
            // the next copy goes natively and takes the sum into binade K + 1; the rest and the
            // bins behind jl add under its ulp
            const float crossed = sum_value(S_j + stay * n_a, static_cast<int>(K)) + pl;
            const uint32_t cb = __float_as_uint(crossed);
            const int bin_l = n_bins - 1 - (64 * t + jl);  // (a candidate bin: its increment is not 0)
            const uint32_t c_l = uniform_u32((cnt[run_word(bin_l >> 1)] >> ((bin_l & 1) << 4)) & 0xffffu);
            const uint32_t rest = readlane_u32(pre_b, 63) - readlane_u32(pre_b, jl);
            uint32_t limit_b = 1u << 24;
            {
              const float tt = topp * scale_b;
              if (tt < 16777216.0f) {
                const uint32_t Tn = static_cast<uint32_t>(__builtin_floorf(tt)) + 1u;
                limit_b = Tn < limit_b ? Tn : limit_b;
              }
            }
            const uint64_t S_b = static_cast<uint64_t>((cb & 0x7fffffu) | 0x800000u) +
                                 static_cast<uint64_t>(c_l - stay - 1u) * n_b + rest;
            if (n_a != 0u && c_l * n_a == inc_l && stay < c_l && (cb >> 23) == K + 1u && S_b < limit_b) {
              s = sum_value(static_cast<uint32_t>(S_b), static_cast<int>(K + 1u));
              if (lane == 0) sbound[t + 1] = s;
              cur = j + 1;
              continue;
            }
          }
        }
        found = resolve_run_group<DT>(s, t, cbound[t], topp, bins);
        if (lane == 0) sbound[t + 1] = s;
        if (found >= 0) last_group = t;
        cur = j + 1;
      }
    }
    if (lane == 0) {
      sm.bc_sum = s;
      sm.bc_found = found;
      sm.flag = last_group;
    }
  }
  __syncthreads();
  const float mass = sm.bc_sum;
  const int last_idx = sm.bc_found >= 0 ? sm.bc_found : static_cast<int>(n0) - 1;
  const int last_group = sm.flag;
  const float r = coin * mass;  // sampler.cpp:162
  __syncthreads();
  // ---- walk 2 (sampler.cpp:163-168): the same partial sums against r; the group in which they
  //      first exceed it is worked out once more
  if (wave == 0) {
    int t2 = -1;
    for (int base = 0; base <= last_group && t2 < 0; base += 64) {
      const int t = base + lane;
      const uint64_t ballot = __ballot(t <= last_group && sbound[t + 1] > r);
      if (ballot) t2 = base + __ffsll(static_cast<long long>(ballot)) - 1;
    }
    int pos = last_idx;
    if (t2 >= 0) {
      float s2 = sbound[t2];
      const int hit = resolve_run_group<DT>(s2, t2, cbound[t2], r, bins);
      if (hit >= 0 && hit < last_idx) pos = hit;
    }
    if (lane == 0) sm.bc_found = pos;
  }
  __syncthreads();
  const int pos = sm.bc_found;
  __syncthreads();
  dbg.last_idx = last_idx;
  dbg.cumulative = mass;
  dbg.r = r;
  dbg.position = pos;
  // ---- the token: the bins that share the probability at `pos`, and the occurrence wanted of them
  //      in index order
  if (wave == 0) {
    int t = 0;
    for (int base = 0; base < n_groups; base += 64) {
      const int g = base + lane;
      const uint64_t ballot = __ballot(g < n_groups && cbound[g + 1] > static_cast<uint32_t>(pos));
      if (ballot) {
        t = base + __ffsll(static_cast<long long>(ballot)) - 1;
        break;
      }
    }
    float prob;
    uint32_t count;
    bins.at(64 * t + lane, prob, count);
    const uint32_t incl = wave_scan_inclusive_u32(count);
    const uint64_t holds = __ballot(cbound[t] + incl > static_cast<uint32_t>(pos));
    const int jl = __ffsll(static_cast<long long>(holds)) - 1;  // not empty: the group's total exceeds pos
    const float p_star = readlane_f32(prob, jl);
    // equal probabilities lie next to each other: look 64 positions to either side
    const int q_star = 64 * t + jl;
    float p_up, p_down;
    uint32_t c_up, c_down;
    bins.at(q_star - 64 + lane >= 0 ? q_star - 64 + lane : n_bins, p_up, c_up);  // positions q_star-64 .. q_star-1
    bins.at(q_star + 1 + lane, p_down, c_down);                                   // positions q_star+1 .. q_star+64
    const uint64_t same_up = __ballot(c_up != 0u && p_up == p_star);
    const uint64_t same_down = __ballot(c_down != 0u && p_down == p_star);
    const uint32_t group_up = wave_sum_u32((c_up != 0u && p_up == p_star) ? c_up : 0u);
    // sorted position of the first entry with this probability, and the key range that holds them
    const uint32_t first_pos = cbound[t] + readlane_u32(incl - count, jl) - group_up;
    const int q_lo = same_up ? q_star - 64 + (__ffsll(static_cast<long long>(same_up)) - 1) : q_star;
    const int q_hi = same_down ? q_star + 1 + (63 - __clzll(static_cast<long long>(same_down))) : q_star;
    if (lane == 0) {
      // (an equal probability at the window's edge could go on beyond it: then sort instead)
      sm.flag = ((same_up & 1ull) && q_star - 64 > 0) || (same_down >> 63) ? -1 : static_cast<int>(static_cast<uint32_t>(pos) - first_pos);
      sm.first_flag[0] = a.key_cut + (n_bins - 1 - q_hi);  // smallest key of the range
      sm.first_flag[1] = a.key_cut + (n_bins - 1 - q_lo);  // largest
    }
  }
  __syncthreads();
  const int want = sm.flag;
  const int key_lo = sm.first_flag[0], key_hi = sm.first_flag[1];
  __syncthreads();
  if (want < 0) return false;
  // occurrences per slot of the row, in index order
  const int ns = a.ns;
  uint32_t* occ = reinterpret_cast<uint32_t*>(lds);  // (the counters are dead) ns + 1 words
  const float kInf = __uint_as_float(0x7f800000u);
  // Keys rise with the values, and a key above 0x8001 or below 0x7ffe belongs to one pattern that is
  // not a zero: a range of such keys of one sign is a range of values, and an entry is compared as a
  // number (two comparisons instead of its key; the zeros of the two signs compare equal and have
  // different keys, which is why they stay with the keys).
  const bool by_value = key_lo > 0x8001 || key_hi < 0x7ffe;
  const float v_lo = pattern_value<DT>(key_pattern(key_lo, a.mag_min)), v_hi = pattern_value<DT>(key_pattern(key_hi, a.mag_min));
  auto matching = [&](const float (&l)[8], int s_, int lane_) -> uint32_t {
    uint32_t mask = 0u;
    if (by_value) {
#pragma unroll
      for (int k = 0; k < 8; ++k) mask |= (l[k] >= v_lo && l[k] <= v_hi) ? (1u << k) : 0u;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int key = pattern_key(value_pattern<DT>(l[k]), a.mag_min);
        mask |= (key >= key_lo && key <= key_hi) ? (1u << k) : 0u;
      }
    }
    const int left = V - (s_ * kSlot + lane_ * 8);  // (entries past the row's end)
    return mask & (left >= 8 ? 0xffu : (left > 0 ? (1u << left) - 1u : 0u));
  };
  auto matches = [&](int s_, int lane_) -> uint32_t {
    float l[8];
    load_slot_lane<DT>(logits, s_, lane_, V, -kInf, l, *a.fused);
    return matching(l, s_, lane_);
  };
  {
    // (five slots of a wave requested at a time: a slot is 16 bytes per lane of a 16-bit row)
    constexpr int kAhead = 5;
    static_assert(VecElems<DT>::value == 8, "a lane's eight entries are one 16-byte load");
    const bool plain = by_value && a.fused->n == 0;
    for (int s0 = wave; s0 < ns; s0 += kAhead * kWaves) {
      uint4 raw[kAhead];
#pragma unroll
      for (int j = 0; j < kAhead; ++j) {
        const int s_ = s0 + j * kWaves;
        raw[j] = {0u, 0u, 0u, 0u};
        if (s_ < ns && (s_ + 1) * kSlot <= V)
          raw[j] = *reinterpret_cast<const uint4*>(logits + static_cast<int64_t>(s_ * kSlot + lane * 8) * ElemSize<DT>::value);
      }
#pragma unroll
      for (int j = 0; j < kAhead; ++j) {
        const int s_ = s0 + j * kWaves;
        if (s_ < ns) {
          float l[8];
          uint32_t c;
          if (plain && (s_ + 1) * kSlot <= V) {
            // the usual slot: two comparisons per entry, their outcomes over the wave counted on
            // the scalar unit (no mask per lane, no sum over the lanes)
            decode_vec<DT>(raw[j], l);
            c = 0u;
#pragma unroll
            for (int k = 0; k < 8; ++k) c += static_cast<uint32_t>(__popcll(__ballot(l[k] >= v_lo && l[k] <= v_hi)));
          } else {
            if ((s_ + 1) * kSlot <= V) {
              decode_vec<DT>(raw[j], l);
              if (a.fused->n > 0) apply_fused<DT, 8>(l, *a.fused);
            } else {
              load_slot_lane<DT>(logits, s_, lane, V, -kInf, l, *a.fused);
            }
            c = wave_sum_u32(static_cast<uint32_t>(__popc(matching(l, s_, lane))));
          }
          if (lane == 0) occ[s_] = c;
        }
      }
    }
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t seen = 0u;
    int32_t tok = -1;
    for (int base = 0; base < ns && tok < 0; base += 64) {
      const uint32_t c = base + lane < ns ? occ[base + lane] : 0u;
      const uint32_t incl = wave_scan_inclusive_u32(c);
      const uint64_t ballot = __ballot(seen + incl > static_cast<uint32_t>(want));
      if (ballot) {
        const int js = __ffsll(static_cast<long long>(ballot)) - 1;
        const uint32_t before = seen + readlane_u32(incl - c, js);
        const int s_ = base + js;
        const uint32_t mask = matches(s_, lane);
        const uint32_t mine = static_cast<uint32_t>(__popc(mask));
        const uint32_t lincl = wave_scan_inclusive_u32(mine);
        const uint64_t b2 = __ballot(before + lincl > static_cast<uint32_t>(want));
        const int jl = __ffsll(static_cast<long long>(b2)) - 1;
        uint32_t skip = static_cast<uint32_t>(want) - (before + readlane_u32(lincl - mine, jl));
        uint32_t mk = readlane_u32(mask, jl);
        while (skip > 0u) {
          mk &= mk - 1u;
          --skip;
        }
        tok = s_ * kSlot + jl * 8 + (__ffs(static_cast<int>(mk)) - 1);
      }
      seen += readlane_u32(incl, 63);
    }
    if (lane == 0) sm.bc_found = tok;
  }
  __syncthreads();
  token = sm.bc_found;
  __syncthreads();
  return token >= 0;
}

// split_chain() as a call, for the looping finish kernel: the chain's registers are then the
// callee's own and do not add to what the loop over the rows keeps alive.  (`fused` points into LDS: a
// reference into the kernel's argument block would move that block to private memory.)
template <int DT>
__device__ __noinline__ float split_chain_call(const SlotRec* recs, const uint2* pairs, int ns, const PrepSlot* prep, uint32_t n_prep,
                                               const char* logits, int V, float inv, float m, const uint64_t* tab,
                                               const FusedOps* fused) {
  return split_chain<DT>(recs, pairs, ns, prep, n_prep, logits, V, inv, m, tab, *fused, nullptr);
}

// grid = rows; dynamic LDS: the key buffer of the draw (p.row.lds_keys keys), which holds the
// slot records and the prepared slots while the sum is composed.
// LOOP: fewer workgroups than rows, a workgroup takes one row after the other (the loop costs
// registers, so a launch with a workgroup per row uses the instantiation without it).
// TOPK: some row of the launch may be a top-k row.  EXTRAS: the launch may write the probabilities
// or fill the phase clocks (a launch that does neither runs the code without them: the branches
// cost a launch of plain top-p rows more than a microsecond in registers and instructions).
template <int DT, bool LOOP, bool TOPK = false, bool EXTRAS = true>
__global__ void __launch_bounds__(kBlock) split_finish_kernel(SplitParams p) {
  uint64_t* const timers = (ETS_PHASE_CLOCKS && EXTRAS) ? p.timers : nullptr;
  float* const probs_out = EXTRAS ? p.row.probs : nullptr;
  extern __shared__ __align__(16) uint64_t lds_keys[];
  __shared__ BlockScratch sm;
  __shared__ FinishShared fs;
  __shared__ int next_lrow;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int V = p.row.vocab;
  const int ns = p.ns;
  // A unit of work is one row, or, in the looping instantiation, p.chain_rows consecutive rows of
  // the launch: the softmax sum of a row is composed by ONE wave while the others have little to
  // do, so the sums of a unit's rows are composed side by side, a wave each, before the rows are
  // drawn one after the other.
  const int R = LOOP ? p.chain_rows : 1;
  const int n_units = (p.row.rows + R - 1) / R;
  const size_t lds_bytes = static_cast<size_t>(p.row.lds_keys) * sizeof(uint64_t);
  const size_t rec_bytes = chain_rec_bytes(ns);  // the records and, behind them, the pairs of split_chain_prepare()
  const size_t pairs_at = chain_pairs_offset(ns);
  for (int unit = blockIdx.x; unit < n_units; unit = LOOP ? take_row(p.row, &next_lrow, n_units) : n_units) {
  if (LOOP) request_row(p.row, &next_lrow, n_units);
  const int r_first = unit * R;
  const int r_count = !LOOP ? 1 : (p.row.rows - r_first < R ? p.row.rows - r_first : R);
  const bool chained = LOOP && R > 1;
  if (chained) {
    if (tid < 32) sm.exp2tab[tid] = kExp2Table[tid];
    if (tid == 0) fs.fused = p.row.fused;  // (the barrier behind the staging comes before the chains)
    // every row gets an equal share of the key buffer for its records and prepared slots
    const size_t share = lds_bytes / static_cast<size_t>(R) / 16 * 16;
    const uint32_t fit = share > rec_bytes ? static_cast<uint32_t>((share - rec_bytes) / sizeof(PrepSlot)) : 0u;
    auto prepared = [&](const RowState& st) -> uint32_t {
      uint32_t n = st.prep_count < static_cast<uint32_t>(p.prep_cap) ? st.prep_count : static_cast<uint32_t>(p.prep_cap);
      return n < fit ? n : fit;
    };
    for (int k = 0; k < r_count; ++k) {
      const int row_k = p.row.row_map ? p.row.row_map[r_first + k] : r_first + k;
      const RowState st = p.row_state[row_k];
      if (st.nan != 0u) continue;
      uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<char*>(lds_keys) + static_cast<size_t>(k) * share);
      const uint4* rec_src = reinterpret_cast<const uint4*>(p.slot_rec + static_cast<int64_t>(row_k) * p.ns_stride);
      for (int i = tid; i < ns; i += kBlock) dst[i] = rec_src[i];
      const uint4* prep_src = reinterpret_cast<const uint4*>(p.prep + static_cast<int64_t>(row_k) * p.prep_cap);
      const int prep_vecs = static_cast<int>(prepared(st) * (sizeof(PrepSlot) / 16));
      for (int i = tid; i < prep_vecs; i += kBlock) dst[rec_bytes / 16 + i] = prep_src[i];
    }
    __syncthreads();
    {
      // the runs of every row's records, the rows' chunks spread over the waves (a NaN row's share
      // holds stale records: nothing reads what comes of them)
      const int k = wave % r_count, per_row = kWaves / r_count;
      if (wave / r_count < per_row) {
        char* mine = reinterpret_cast<char*>(lds_keys) + static_cast<size_t>(k) * share;
        split_chain_prepare(reinterpret_cast<const SlotRec*>(mine), ns, reinterpret_cast<uint2*>(mine + pairs_at), wave / r_count, per_row);
      }
    }
    __syncthreads();
    if (wave < r_count) {
      const int row_k = p.row.row_map ? p.row.row_map[r_first + wave] : r_first + wave;
      const RowState st = p.row_state[row_k];
      float sum = __uint_as_float(0x7fc00000u);
      if (st.nan == 0u) {
        const float inv_k = p.row.row_cfg ? p.row.row_cfg[row_k].inv_temperature : p.row.inv_temperature;
        const char* logits_k = static_cast<const char*>(p.row.logits) + static_cast<int64_t>(row_k) * p.row.row_stride * ElemSize<DT>::value;
        const char* mine = reinterpret_cast<const char*>(lds_keys) + static_cast<size_t>(wave) * share;
        sum = split_chain_call<DT>(reinterpret_cast<const SlotRec*>(mine), reinterpret_cast<const uint2*>(mine + pairs_at), ns,
                                   reinterpret_cast<const PrepSlot*>(mine + rec_bytes),
                                   prepared(st), logits_k, V, inv_k, st.m, sm.exp2tab, &fs.fused);
      }
      if (lane == 0) fs.pre_sum[wave] = sum;
    }
    __syncthreads();
  }
  // lrow, the row of this launch, indexes the buffers whose layout depends on the launch
  for (int lrow = r_first; lrow < r_first + r_count; ++lrow) {
  const int row = p.row.row_map ? p.row.row_map[lrow] : lrow;
  const float inv = p.row.row_cfg ? p.row.row_cfg[row].inv_temperature : p.row.inv_temperature;
  const float topp = p.row.row_cfg ? p.row.row_cfg[row].topp : p.row.topp;
  const char* logits = static_cast<const char*>(p.row.logits) + static_cast<int64_t>(row) * p.row.row_stride * ElemSize<DT>::value;
  const float kNaN = __uint_as_float(0x7fc00000u);
  // What the row's state does not decide is requested before the state is looked at (one trip to
  // memory instead of two in a row): the lane's first slot record, its bucket of the first
  // workgroups' histograms, the workgroups' list counts.
  const uint4* rec_src = reinterpret_cast<const uint4*>(p.slot_rec + static_cast<int64_t>(row) * p.ns_stride);
  const uint4* prep_src = reinterpret_cast<const uint4*>(p.prep + static_cast<int64_t>(row) * p.prep_cap);
  uint4 early_rec = {0u, 0u, 0u, 0u};
  uint32_t early_count = 0u;
  const bool early = !chained;
  if (early) {
    if (tid < ns) early_rec = rec_src[tid];
    if (tid < p.row_wgs) early_count = p.list_count[static_cast<int64_t>(lrow) * kMaxRowWorkgroups + tid];
  }
  uint32_t early_hist[4] = {0u, 0u, 0u, 0u};  // bucket `tid` of the first four workgroups' histograms
  if (early) {
    const uint32_t* hist_in = p.hist + static_cast<int64_t>(lrow) * p.row_wgs * kHistBuckets;
#pragma unroll
    for (int k = 0; k < 4; ++k) early_hist[k] = hist_in[(k < p.row_wgs ? k : 0) * kHistBuckets + tid];
  }
  const RowState rs = p.row_state[row];
  // (the number by which the fused launch tags what its workgroups hand over: the next launch gets another)
  if (lrow == 0 && tid == 0 && p.arrive) next_launch_number(p.arrive);
  const float m = rs.m;
  const bool row_nan = rs.nan != 0u;
  const float cutoff = (1.0f - topp) / static_cast<float>(V - 1);  // sampler.cpp:136
  uint64_t t0 = 0, t1 = 0, t2 = 0;
  if (timers) t0 = wall_clock64();
  if (tid < 32) sm.exp2tab[tid] = kExp2Table[tid];
  if (tid == 0) fs.fused = p.row.fused;  // (barriers follow before any draw function reads it)
  uint64_t coin_state = 0ull;  // asked for now, needed once the sum is known
  if (tid == 0) coin_state = p.row.rng[row];

  float S = kNaN;
  int n_listed = 0;
  HistPlan plan = {-1, 0, 0, 0};
  bool lists_ok = false;
  bool topk_few = false;
  if (!row_nan) {
    // ---- how many candidates the workgroups of pass 2 listed; their histograms, added up
    if (tid < 64) {
      const uint32_t c = tid < p.row_wgs ? (early ? early_count : p.list_count[static_cast<int64_t>(lrow) * kMaxRowWorkgroups + tid]) : 0u;
      const uint32_t incl = wave_scan_inclusive_u32(c);
      fs.count[tid] = c;
      fs.offset[tid + 1] = incl;
      if (tid == 0) fs.offset[0] = 0u;
      const uint64_t over = __ballot(c > static_cast<uint32_t>(p.list_region));
      if (tid == 0) {
        fs.overflow = over ? 1u : 0u;
        fs.sel_count = 0u;
        fs.band_count = 0u;
      }
    }
    {
      // (four workgroups' counts are requested at a time: a loop of one load each would wait for each)
      const uint32_t* hist_in = p.hist + static_cast<int64_t>(lrow) * p.row_wgs * kHistBuckets;
      const int n_hist = rs.listed_buckets == kNoLists ? 0 : (rs.listed_buckets != 0u ? static_cast<int>(rs.listed_buckets) : kHistBuckets);  // (the rest was not written)
      uint32_t c[kHistBuckets / kBlock];
#pragma unroll
      for (int q = 0; q < kHistBuckets / kBlock; ++q) c[q] = 0u;
      for (int g = 0; g < p.row_wgs; g += 4) {
        uint32_t v[4][kHistBuckets / kBlock];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int gk = g + k < p.row_wgs ? g + k : g;
#pragma unroll
          for (int q = 0; q < kHistBuckets / kBlock; ++q) {
            if (q == 0 && early && g == 0) {
              v[k][q] = tid < n_hist ? early_hist[k] : 0u;  // (what lies behind the listed buckets is stale)
            } else {
              v[k][q] = q * kBlock + tid < n_hist ? hist_in[gk * kHistBuckets + q * kBlock + tid] : 0u;
            }
          }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
          for (int q = 0; q < kHistBuckets / kBlock; ++q) c[q] += g + k < p.row_wgs ? v[k][q] : 0u;
        }
      }
#pragma unroll
      for (int q = 0; q < kHistBuckets / kBlock; ++q) fs.hist[q * kBlock + tid] = c[q];
    }
    // ---- LDS: the records, then as many prepared slots as fit (one that does not is redone from
    //      the logits when its turn comes); not when the unit's sums have been composed already
    uint32_t n_prep = rs.prep_count < static_cast<uint32_t>(p.prep_cap) ? rs.prep_count : static_cast<uint32_t>(p.prep_cap);
    const uint32_t fit = static_cast<uint32_t>((lds_bytes - rec_bytes) / sizeof(PrepSlot));
    n_prep = n_prep < fit ? n_prep : fit;
    uint4* lds_vec = reinterpret_cast<uint4*>(lds_keys);
    uint4* prep_dst = lds_vec + rec_bytes / 16;
    if (!chained) {
      const int prep_vecs = static_cast<int>(n_prep * (sizeof(PrepSlot) / 16));
      if (early) {
        if (tid < ns) lds_vec[tid] = early_rec;
        for (int i = tid + kBlock; i < ns; i += kBlock) lds_vec[i] = rec_src[i];
        for (int i = tid; i < prep_vecs; i += kBlock) prep_dst[i] = prep_src[i];
      } else {
        for (int i = tid; i < ns; i += kBlock) lds_vec[i] = rec_src[i];
        for (int i = tid; i < prep_vecs; i += kBlock) prep_dst[i] = prep_src[i];
      }
    }
    __syncthreads();
    // the runs of the row's records, a chunk of 64 per wave (the barriers of split_plan() lie between this and the chain)
    if (!chained)
      split_chain_prepare(reinterpret_cast<const SlotRec*>(lds_keys), ns,
                          reinterpret_cast<uint2*>(reinterpret_cast<char*>(lds_keys) + pairs_at), wave, kWaves);
    n_listed = static_cast<int>(fs.offset[p.row_wgs]);
    lists_ok = fs.overflow == 0u;
    plan = split_plan(fs.hist, rs.a_total, topp, cutoff, V, &fs.plan, sm);
    if (timers) t1 = wall_clock64();
    // (a top-k row whose lists hold at most 64 entries, at least topk of them: one wave can draw it)
    const int32_t row_topk_early = !TOPK ? 0 : (p.row.row_cfg ? p.row.row_cfg[row].topk : p.row.topk);
    topk_few = TOPK && row_topk_early > 0 && row_topk_early < V && lists_ok && rs.listed_buckets != 0u && rs.listed_buckets != kNoLists &&
               n_listed >= row_topk_early && n_listed <= 64;
    if (wave == 0) {
      if (!chained) {
        float sum;
        if constexpr (LOOP) {  // (fs.fused was stored before the barrier behind the staging)
          sum = split_chain_call<DT>(reinterpret_cast<const SlotRec*>(lds_keys),
                                     reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(lds_keys) + pairs_at), ns,
                                     reinterpret_cast<const PrepSlot*>(prep_dst), n_prep, logits, V, inv, m, sm.exp2tab, &fs.fused);
        } else {
          sum = split_chain<DT>(reinterpret_cast<const SlotRec*>(lds_keys),
                                reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(lds_keys) + pairs_at), ns,
                                reinterpret_cast<const PrepSlot*>(prep_dst), n_prep, logits, V, inv, m, sm.exp2tab,
                                p.row.fused, timers ? timers + static_cast<int64_t>(row) * 8 : nullptr);
        }
        if (lane == 0) sm.bc_sum = sum;
#if ETS_PHASE_CLOCKS
        if (timers) {  // the same chain once more, its code now in the instruction cache and no clocks inside
          const uint64_t ta = wall_clock64();
          const float again = split_chain<DT>(reinterpret_cast<const SlotRec*>(lds_keys),
                                              reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(lds_keys) + pairs_at), ns,
                                              reinterpret_cast<const PrepSlot*>(prep_dst), n_prep, logits, V, inv, m, sm.exp2tab,
                                              p.row.fused, nullptr);
          const uint64_t tb = wall_clock64();
          if (lane == 0) timers[static_cast<int64_t>(row) * 8 + 5] = (tb - ta) | (again == sum ? 0ull : 1ull << 40);
        }
#endif
      } else if (lane == 0) {
        sm.bc_sum = fs.pre_sum[lrow - r_first];
      }
    } else if (TOPK && topk_few) {
      // ---- the second wave, meanwhile: the listed entries of a top-k row, all of them
      if (wave == 1) {
        for (int g = 0; g < p.row_wgs; ++g) {
          const uint64_t* src = p.list + (static_cast<int64_t>(lrow) * p.row_wgs + g) * p.list_region;
          const int c = static_cast<int>(fs.count[g]);
          if (lane < c) fs.sel[fs.offset[g] + lane] = src[lane];
        }
      }
    } else if (lists_ok && plan.b_sel >= 0 && plan.n_sel <= 64) {
      // ---- the other waves, meanwhile: one pass over the listed candidates picks out those of the
      //      largest buckets and those that may or may not reach the cutoff
      for (int g = 0; g < p.row_wgs; ++g) {
        const uint64_t* src = p.list + (static_cast<int64_t>(lrow) * p.row_wgs + g) * p.list_region;
        const int c = static_cast<int>(fs.count[g]);
        for (int j = (wave - 1) * 64 + lane; j < c; j += (kWaves - 1) * 64) {
          const uint64_t ent = src[j];
          const int b = static_cast<int>(hist_bucket(static_cast<uint32_t>(ent >> 32)));
          if (b <= plan.b_sel) {
            const uint32_t at = atomicAdd(&fs.sel_count, 1u);
            if (at < 64u) fs.sel[at] = ent;
          }
          if (b >= plan.b_band) {
            const uint32_t at = atomicAdd(&fs.band_count, 1u);
            if (at < static_cast<uint32_t>(kBandCap)) fs.band[at] = static_cast<uint32_t>(ent >> 32);
          }
        }
      }
    }
    __syncthreads();
    S = sm.bc_sum;
    if (timers) t2 = wall_clock64();
  }

  // ---- The usual row of a launch that asks for nothing but tokens -- short lists, a selection of at
  //      most 64 entries, all of them picked out while the chain ran -- is finished by the first wave
  //      alone: coin, keys, rank, the two walks and the token in registers, no barrier between them
  //      (the steps below, for any row, hand every intermediate result round the workgroup through
  //      LDS: eight barriers).  If the selection turns out not to decide the draw the wave leaves
  //      everything as it was, coin state included, and the row takes the steps below.
  if constexpr (!EXTRAS) {
    const int32_t row_topk = !TOPK ? 0 : (p.row.row_cfg ? p.row.row_cfg[row].topk : p.row.topk);
    const bool is_topk = TOPK && row_topk > 0 && row_topk < V;
    const bool small_tail = !row_nan && p.row.debug == nullptr && lists_ok &&
                            (is_topk ? topk_few
                                     : (rs.listed_buckets != 0u && plan.b_sel >= 0 && plan.n_sel >= 1 && plan.n_sel <= 64 &&
                                        fs.sel_count == static_cast<uint32_t>(plan.n_sel) && plan.b_sel < static_cast<int>(rs.listed_buckets)));
    if (small_tail) {
      if (wave == 0) {
        uint64_t st = (static_cast<uint64_t>(readlane_u32(static_cast<uint32_t>(coin_state >> 32), 0)) << 32) |
                      readlane_u32(static_cast<uint32_t>(coin_state), 0);
        st ^= st >> 12;
        st ^= st << 25;
        st ^= st >> 27;
        const uint32_t u = static_cast<uint32_t>((st * 0x2545F4914F6CDD1Dull) >> 32);
        const float coin1 = static_cast<float>(u >> 8) / 16777216.0f;
        const RowDivisor div = row_divisor(S);
        const int n_sel = is_topk ? n_listed : plan.n_sel;
        bool is_in = true;
        uint64_t key = ~0ull;
        if (lane < n_sel) {
          const uint64_t ent = fs.sel[lane];
          const float pj = div_row(__uint_as_float(static_cast<uint32_t>(ent >> 32)), div);
          is_in = is_topk || pj >= cutoff;  // sampler.cpp:137-143 (every entry is a candidate of a top-k draw)
          key = cand_key(pj, static_cast<int>(static_cast<uint32_t>(ent)));
        }
        int pos = -2, last_idx = 0;
        float mass = 0.0f, r = 0.0f;
        uint32_t tok = 0u;
        if (TOPK && is_topk) {
          // (sampler.cpp:72-120: the first topk of the sorted entries; what is not listed lies below the lists' floor)
          const float list_floor = __uint_as_float(0x3F800000u - (rs.listed_buckets << 17) + 1u);
          pos = small_wave_core(key, n_sel, n_sel, topp, coin1, row_topk, div_row(list_floor, div), last_idx, mass, r, tok);
        } else if (__ballot(!is_in) == 0ull) {
          // (more candidates exist than the lists hold; entries outside the selection have exps up to the edge of the next bucket)
          pos = small_wave_core(key, n_sel, 0x7fffffff, topp, coin1, 0, div_row(hist_edge(plan.b_sel + 1), div), last_idx, mass, r, tok);
        }
        if (lane == 0) {
          if (pos != -2) {
            p.row.rng[row] = st;
            p.row.tokens[row] = static_cast<int32_t>(tok);
          }
          sm.flag = pos != -2 ? 1 : 0;
        }
      }
      __syncthreads();
      const bool tail_done = sm.flag != 0;
      __syncthreads();
      if (tail_done) continue;  // (the next row of the unit, if any)
    }
  }
  // ---- one coin per call (sampler.cpp:237, 210-220)
  if (tid == 0) {
    uint64_t st = coin_state;
    st ^= st >> 12;
    st ^= st << 25;
    st ^= st >> 27;
    p.row.rng[row] = st;
    const uint32_t u = static_cast<uint32_t>((st * 0x2545F4914F6CDD1Dull) >> 32);
    sm.red_f[0] = static_cast<float>(u >> 8) / 16777216.0f;
  }
  __syncthreads();  // (the records and prepared slots are dead from here on: the buffer becomes the key buffer)
  const float coin = sm.red_f[0];
  __syncthreads();

  if (probs_out) {
    float* probs = probs_out + static_cast<int64_t>(row) * V;
    if (row_nan) {
      for (int i = tid; i < V; i += kBlock) {
        const float x = load_logit<DT>(logits, i, p.row.fused) * inv;
        probs[i] = expf_nonpositive(x - m, sm.exp2tab) / S;
      }
    } else {
      const RowDivisor div = row_divisor(S);
      for (int i = tid; i < V; i += kBlock) {
        const float x = load_logit<DT>(logits, i, p.row.fused) * inv;
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
    token = -1;  // a NaN row keeps no candidate, where the reference reads probindex[-1]
  }
  __syncthreads();
  int path = 0;
  const int32_t topk = !TOPK ? 0 : (p.row.row_cfg ? p.row.row_cfg[row].topk : p.row.topk);
  if (TOPK && topk > 0 && topk < V) {
    // ---- a top-k row (sampler.cpp:72-120, before top-p: :239): pass 2 listed the entries of the
    //      histogram's first buckets, at least topk of them; they are sorted and the first topk walked.
    //      Every probability NaN: every entry ties, the first topk in index order, the last of them drawn.
    path = 6;
    if (row_nan) {
      token = topk - 1;
    } else {
      bool done = false;
      const uint32_t lb = rs.listed_buckets;
      if (lb != 0u && lb != kNoLists && lists_ok && n_listed >= topk && n_listed <= p.row.lds_keys - kBlock) {
        for (int g = wave; g < p.row_wgs; g += kWaves) {
          const uint64_t* src = p.list + (static_cast<int64_t>(lrow) * p.row_wgs + g) * p.list_region;
          uint64_t* dst = lds_keys + kBlock + fs.offset[g];
          const int c = static_cast<int>(fs.count[g]);
          for (int j = lane; j < c; j += 64) dst[j] = src[j];
        }
        __syncthreads();
        const float list_floor = __uint_as_float(0x3F800000u - (lb << 17) + 1u);  // what is not listed is below this
        done = draw_topk_listed(lds_keys, p.row.lds_keys, kBlock, n_listed, S, list_floor, topk, topp, coin, V, dbg, token, sm);
      }
      if (!done) {
        uint64_t* scratch = p.row.scratch + static_cast<int64_t>(blockIdx.x) * p.row.scratch_stride;
        token = draw_general<DT>(logits, V, inv, m, S, true, topk, topp, 0.0f, coin, scratch, p.row.scratch_stride, lds_keys,
                                 p.row.lds_keys, dbg, sm, p.row.fused.n > 0 ? &fs.fused : nullptr);
      }
    }
  } else if (!row_nan) {
    bool done = false;
    const RowDivisor div = row_divisor(S);
    // Short lists (RowState::listed_buckets): the lists hold every entry of the histogram's first
    // buckets and nothing else, so the number of candidates is unknown ("more exist") and a walk
    // that does not end inside the listed entries is redone from the row.
    const bool short_lists = rs.listed_buckets != 0u;
    const int kMore = 0x7fffffff;
    if (lists_ok && n_listed == 0 && !short_lists) {
      done = true;  // no candidate (the reference reads probindex[-1] here)
    } else if (lists_ok && plan.b_sel >= 0 && plan.n_sel >= 1 && plan.n_sel <= 64 &&
               fs.sel_count == static_cast<uint32_t>(plan.n_sel) &&
               (short_lists ? plan.b_sel < static_cast<int>(rs.listed_buckets)
                            : (fs.band_count <= static_cast<uint32_t>(kBandCap) &&
                               fs.band_count + static_cast<uint32_t>(plan.n_certain) == static_cast<uint32_t>(n_listed)))) {
      // ---- exact candidate count (sampler.cpp:137-143): the certain ones, plus those of the band
      //      whose probability reaches the cutoff
      const int n_band = short_lists ? 0 : static_cast<int>(fs.band_count);
      uint32_t cnt = 0u;
      for (int j = tid; j < n_band; j += kBlock) cnt += div_row(__uint_as_float(fs.band[j]), div) >= cutoff ? 1u : 0u;
      cnt = wave_sum_u32(cnt);
      if (lane == 0) sm.red_u[wave] = cnt;
      // ---- the short selection: every selected entry must be a candidate
      const int n_sel = plan.n_sel;
      if (tid < 64) {
        bool is_in = true;
        uint64_t key = ~0ull;
        if (tid < n_sel) {
          const uint64_t ent = fs.sel[tid];
          const float pj = div_row(__uint_as_float(static_cast<uint32_t>(ent >> 32)), div);
          is_in = pj >= cutoff;
          key = cand_key(pj, static_cast<int>(static_cast<uint32_t>(ent)));
        }
        lds_keys[tid] = key;
        const uint64_t out = __ballot(!is_in);
        if (tid == 0) sm.flag = out ? 0 : 1;
      }
      __syncthreads();
      uint32_t n0 = static_cast<uint32_t>(plan.n_certain);
      for (int w = 0; w < kWaves; ++w) n0 += sm.red_u[w];
      if (short_lists) n0 = static_cast<uint32_t>(kMore);
      const bool ok = sm.flag != 0;
      __syncthreads();
      if (n0 == 0u) {
        dbg.n_candidates = 0;
        done = true;
      } else if (ok) {
        // entries outside the selection have exp up to the edge of the next bucket
        const float p_floor = (n_sel == static_cast<int>(n0)) ? -1.0f : div_row(hist_edge(plan.b_sel + 1), div);
        dbg.n_candidates = static_cast<int>(n0);
        done = draw_small_wave((LdsKeys)lds_keys, n_sel, static_cast<int>(n0), topp, coin, dbg, token, sm, 0, p_floor) != -2;
        path = 1;
      }
    }
    if constexpr (DT == kDtypeBFloat16 || DT == kDtypeHalf) {
      // ---- a longer nucleus of a 16-bit row: runs of equal probabilities
      if (!done && !short_lists && rs.n_bins > 0 && (!lists_ok || n_listed > 4096)) {
        const RunArgs ra = {p.phist + static_cast<int64_t>(lrow) * p.row_wgs * p.phist_words, p.phist_words, p.row_wgs,
                            p.row.lds_keys, ns, rs.key_cut, rs.n_bins, rs.mag_min, static_cast<uint32_t>(n_listed), m, &fs.fused};
        done = draw_topp_runs<DT>(ra, logits, V, inv, S, cutoff, topp, coin, lds_keys, dbg, token, sm);
        path = 4;
      }
    }
    // (a list too long for LDS is worth the passes over it only when the histogram says that the
    // entries to sort will fit)
    if (!done && lists_ok && n_listed > 0 && static_cast<int64_t>(n_listed) <= p.row.scratch_stride &&
        (n_listed <= p.row.lds_keys - kBlock || (plan.b_sel >= 0 && plan.n_sel <= p.row.lds_keys))) {
      // ---- a longer nucleus: the list goes to LDS as far as it fits and to the workgroup's scratch
      //      row beyond that (entry j at position j of either), then selection by probability,
      //      sort of the selected entries, walks
      const int lds_cap = p.row.lds_keys - kBlock;
      uint64_t* lds_list = lds_keys + kBlock;
      uint64_t* far_list = p.row.scratch + static_cast<int64_t>(blockIdx.x) * p.row.scratch_stride;
      for (int g = wave; g < p.row_wgs; g += kWaves) {
        const uint64_t* src = p.list + (static_cast<int64_t>(lrow) * p.row_wgs + g) * p.list_region;
        const int first = static_cast<int>(fs.offset[g]);
        const int c = static_cast<int>(fs.count[g]);
        for (int j = lane; j < c; j += 64) {
          const uint64_t ent = src[j];
          if (first + j < lds_cap) {
            lds_list[first + j] = ent;
          } else {
            far_list[first + j] = ent;
          }
        }
      }
      __threadfence_block();  // (the scratch row's entries are read by other lanes of the workgroup)
      __syncthreads();
      // (the buckets the plan selected carry more than topp: the probability of their lower edge is the threshold to try)
      const float tau_hint = plan.b_sel >= 0 ? div_row(hist_edge(plan.b_sel + 1), div) : 0.0f;
      done = draw_topp_listed(far_list, lds_list, lds_cap, kBlock, n_listed, S, cutoff, topp, coin, lds_keys, p.row.lds_keys, dbg,
                              token, sm, short_lists, tau_hint);
      path = 2;
    }
    if (!done) {
      uint64_t* scratch = p.row.scratch + static_cast<int64_t>(blockIdx.x) * p.row.scratch_stride;
      token = draw_general<DT>(logits, V, inv, m, S, false, 0, topp, cutoff, coin, scratch, p.row.scratch_stride, lds_keys,
                               p.row.lds_keys, dbg, sm, p.row.fused.n > 0 ? &fs.fused : nullptr);
      path = 3;
    }
  }
  if (tid == 0) {
    p.row.tokens[row] = token;
    if (p.row.debug) p.row.debug[row] = dbg;
    if (timers) {
      uint64_t* t = timers + static_cast<int64_t>(row) * 8;
      t[0] = t1 - t0;
      t[1] = t2 - t1;
      t[2] = wall_clock64() - t2;
      t[3] = static_cast<uint64_t>(n_listed) | (static_cast<uint64_t>(rs.prep_count) << 32);
      t[4] = static_cast<uint64_t>(path) | (static_cast<uint64_t>(plan.n_sel) << 8) | (static_cast<uint64_t>(fs.band_count) << 32);
    }
  }
  }  // rows of the unit
  }  // units of this workgroup
}

// ---- multinomial rows (sampler.cpp:58-70, 236-247) -------------------------------------------------
// Their draw is a second sequential sum over the row, of p = fl(e / S), up to the first entry behind
// which it exceeds the coin.  Five launches: pass 1; pass 2 (records of the sum of e); this kernel,
// PHASE 0: the exact S by the chain, the coin; pass 2 again in its WALK instantiation (records of the
// sum of p); this kernel, PHASE 1: the chain over those, stopped by the coin.
// grid = rows, kWalkBlock lanes: all of them stage the row's records and prepared slots in LDS
// (dynamic: `lds_bytes`), the first wave walks.
constexpr int kWalkBlock = 256;
template <int DT, int PHASE>
__global__ void __launch_bounds__(kWalkBlock) split_walk_kernel(SplitParams p, uint32_t lds_bytes) {
  extern __shared__ __align__(16) uint64_t walk_lds[];
  __shared__ uint64_t exp2tab[32];
  uint64_t* const walk_timers = ETS_PHASE_CLOCKS ? p.timers : nullptr;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int V = p.row.vocab;
  const int ns = p.ns;
  const int row = p.row.row_map ? p.row.row_map[blockIdx.x] : blockIdx.x;
  const RowState rs = p.row_state[row];
  if (tid < 32) exp2tab[tid] = kExp2Table[tid];
  // (the number by which a launch with pass 1 inside pass 2 tags what its workgroups hand over: the next one gets another)
  if (PHASE == 0 && blockIdx.x == 0 && tid == 0 && p.arrive) next_launch_number(p.arrive);
  auto toss = [&]() {  // one coin per call (sampler.cpp:237, 210-220)
    uint64_t st = p.row.rng[row];
    st ^= st >> 12;
    st ^= st << 25;
    st ^= st >> 27;
    p.row.rng[row] = st;
    const uint32_t u = static_cast<uint32_t>((st * 0x2545F4914F6CDD1Dull) >> 32);
    return static_cast<float>(u >> 8) / 16777216.0f;
  };
  if (rs.nan != 0u) {
    // every probability is NaN: the walk never stops and returns the last index
    if (PHASE == 0 && tid == 0) {
      const float coin = toss();
      p.row.tokens[row] = V - 1;
      if (p.row.debug) p.row.debug[row] = RowDebug{rs.m, __uint_as_float(0x7fc00000u), coin, 0.0f, 0.0f, 0, 0, 0};
    }
    return;
  }
  const float inv = p.row.row_cfg ? p.row.row_cfg[row].inv_temperature : p.row.inv_temperature;
  const char* logits = static_cast<const char*>(p.row.logits) + static_cast<int64_t>(row) * p.row.row_stride * ElemSize<DT>::value;
  const size_t rec_bytes = chain_rec_bytes(ns);
  uint32_t n_prep = rs.prep_count < static_cast<uint32_t>(p.prep_cap) ? rs.prep_count : static_cast<uint32_t>(p.prep_cap);
  const uint32_t fit = lds_bytes > rec_bytes ? static_cast<uint32_t>((lds_bytes - rec_bytes) / sizeof(PrepSlot)) : 0u;
  n_prep = n_prep < fit ? n_prep : fit;  // (a prepared slot that does not fit is redone from the logits)
  uint4* lds_vec = reinterpret_cast<uint4*>(walk_lds);
  const uint4* rec_src = reinterpret_cast<const uint4*>(p.slot_rec + static_cast<int64_t>(row) * p.ns_stride);
  const uint4* prep_src = reinterpret_cast<const uint4*>(p.prep + static_cast<int64_t>(row) * p.prep_cap);
  for (int i = tid; i < ns; i += kWalkBlock) lds_vec[i] = rec_src[i];
  const int prep_vecs = static_cast<int>(n_prep * (sizeof(PrepSlot) / 16));
  for (int i = tid; i < prep_vecs; i += kWalkBlock) lds_vec[rec_bytes / 16 + i] = prep_src[i];
  __syncthreads();
  uint2* pairs = reinterpret_cast<uint2*>(reinterpret_cast<char*>(walk_lds) + chain_pairs_offset(ns));
  // the runs of the row's records, a chunk of 64 per wave
  split_chain_prepare(reinterpret_cast<const SlotRec*>(walk_lds), ns, pairs, tid >> 6, kWalkBlock / 64);
  __syncthreads();
  if (tid >= 64) return;
  const SlotRec* recs = reinterpret_cast<const SlotRec*>(walk_lds);
  const PrepSlot* prep = reinterpret_cast<const PrepSlot*>(reinterpret_cast<const char*>(walk_lds) + rec_bytes);
  if (PHASE == 0) {
    const float S = split_chain<DT>(recs, pairs, ns, prep, n_prep, logits, V, inv, rs.m, exp2tab, p.row.fused,
                                    walk_timers ? walk_timers + static_cast<int64_t>(row) * 8 : nullptr);
    if (lane == 0) p.walk[row] = make_float2(S, toss());
  } else {
    const float2 w = p.walk[row];
    const RowDivisor div = row_divisor(w.x);
    int stop = -1;
    const float cdf = split_chain<DT, true>(recs, pairs, ns, prep, n_prep, logits, V, inv, rs.m, exp2tab, p.row.fused, nullptr, &div, w.y, &stop);
    if (lane == 0) {
      const int32_t token = stop >= 0 ? stop : V - 1;
      p.row.tokens[row] = token;
      if (p.row.debug) p.row.debug[row] = RowDebug{rs.m, w.x, w.y, cdf, 0.0f, 0, 0, token};
    }
  }
}

}  // namespace ets
