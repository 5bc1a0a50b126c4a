// Host side of the C ABI declared in include/et_sampler.h: handle bookkeeping, argument
// checks and kernel launches.  Compiled with hipcc for gfx950 only.
#include "../../include/et_sampler.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cmath>
#include <cstring>
#include <ctime>
#include <mutex>
#include <new>
#include <string>

#include <cstdlib>

#include "ets_host.h"


namespace {

thread_local std::string g_thread_error;

struct ErrorSink {
  std::string* where;
};

}  // namespace

namespace ets_host {

ets_status fail(ets_sampler* s, ets_status code, const std::string& msg) {
  if (s) {
    s->last_error = msg;
  } else {
    g_thread_error = msg;
  }
  return code;
}

ets_status hip_fail(ets_sampler* s, hipError_t e, const char* what) {
  return fail(s, e == hipErrorOutOfMemory ? ETS_MEMORY_ALLOCATION_FAILED : ETS_INTERNAL,
              std::string(what) + ": " + hipGetErrorString(e));
}

// Raises a kernel's dynamic-LDS limit to `bytes` on the handle's device.  The limit is kept per
// kernel and device, so it is set again only when a handle asks for more than was set before.
ets_status allow_dynamic_lds(ets_sampler* s, const void* kernel, size_t bytes, std::atomic<size_t>* set_bytes) {
  const int dev = s->device >= 0 && s->device < kMaxDevices ? s->device : 0;
  if (set_bytes[dev].load(std::memory_order_acquire) >= bytes) return ETS_OK;
  ETS_HIP(s, hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
  set_bytes[dev].store(bytes, std::memory_order_release);
  return ETS_OK;
}

// ---- rows spread over several workgroups (ets_split.h) -------------------------------------------

// Workgroups per row of pass 2: as many as keep the launch within one workgroup per CU (a second,
// partly filled round would cost more than the longer sweeps), sixteen slots each at least.
// (ETS_SPLIT_WORKGROUPS forces a number; not for a call that brings its own work buffers, whose
// layout was made for the automatic choice.)
int pass2_workgroups(const ets_sampler* s, int32_t rows, int32_t ns, int32_t beside) {
  static const int forced = [] {
    const char* e = std::getenv("ETS_SPLIT_WORKGROUPS");
    return e ? std::atoi(e) : 0;
  }();
  // (launches that run side by side share the compute units: each takes its share of them, so that
  // the workgroups of both are resident at once)
  int g = (forced > 0 && !s->wb) ? forced : (s->num_cus > 0 ? s->num_cus : 256) / (rows + beside);
  const int by_len = (ns + 15) / 16;
  if (g > by_len) g = by_len;
  if (g > ets::kMaxRowWorkgroups) g = ets::kMaxRowWorkgroups;
  if (s->wb && g > s->wb->max_row_wgs) g = s->wb->max_row_wgs;
  return g < 1 ? 1 : g;
}

// Candidates one workgroup of pass 2 can list when `g` of them share a row: all of its entries,
// up to kListRegion.
int32_t list_region(int32_t ns, int g) {
  const int per_wg = ((ns + g - 1) / g + 15) / 16 * 16;
  const int64_t entries = static_cast<int64_t>(per_wg) * ets::kSlot;
  return static_cast<int32_t>(entries < ets::kListRegion ? entries : ets::kListRegion);
}

ets_status ensure_split(ets_sampler* s) {
  if (s->d_split) return ETS_OK;
  ets::SplitParams& sp = s->split;
  const size_t rows = static_cast<size_t>(s->max_batch);
  sp.ns = (s->vocab + ets::kSlot - 1) / ets::kSlot;
  sp.ns_stride = static_cast<int32_t>(round_up(static_cast<size_t>(sp.ns), 4));
  sp.prep_cap = ets::kPrepCap;
  // the candidate lists of the largest launch: rows x workgroups per row x region
  size_t list_entries = 0, row_wgs = 0;
  // (with nothing beside the launch: a launch of r rows beside b others gets the workgroups per row
  // of a launch of r + b rows, which this loop covers)
  for (int32_t r = 1; r <= s->max_batch; ++r) {
    const int g = pass2_workgroups(s, r, sp.ns, 0);
    const size_t need = static_cast<size_t>(r) * g * list_region(sp.ns, g);
    if (need > list_entries) list_entries = need;
    if (static_cast<size_t>(r) * g > row_wgs) row_wgs = static_cast<size_t>(r) * g;
  }
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t here = at;
    at = round_up(at + bytes, 256);
    return here;
  };
  const size_t o_max = take(rows * sp.ns_stride * sizeof(float));
  const size_t o_max2 = take(rows * sp.ns_stride * sizeof(float));
  const size_t o_sum = take(rows * sp.ns_stride * sizeof(float));
  const size_t o_rec = take(rows * sp.ns_stride * sizeof(ets::SlotRec));
  const size_t o_prep = take(rows * sp.prep_cap * sizeof(ets::PrepSlot));
  const size_t o_state = take(rows * sizeof(ets::RowState));
  const size_t o_walk = take(rows * sizeof(float2));
  const size_t o_count = take(rows * ets::kMaxRowWorkgroups * sizeof(uint32_t));
  const size_t o_arrive = take(rows * 2 * sizeof(uint32_t));
  const size_t o_pack = take(rows * sp.ns_stride * sizeof(float4));
  const size_t o_timers = take(rows * 12 * sizeof(uint64_t));
  const size_t o_hist = take(row_wgs * ets::kHistBuckets * sizeof(uint32_t));
  const size_t o_list = take(list_entries * sizeof(uint64_t));
  ETS_HIP(s, hipMalloc(&s->d_split, at));
  char* base = static_cast<char*>(s->d_split);
  ETS_HIP(s, hipMemset(base + o_arrive, 0, rows * 2 * sizeof(uint32_t)));  // (launches are numbered from 1)
  ETS_HIP(s, hipMemset(base + o_pack, 0, rows * sp.ns_stride * sizeof(float4)));  // (no record carries a launch's tag yet)
  sp.arrive = reinterpret_cast<uint32_t*>(base + o_arrive);
  sp.slot_pack = reinterpret_cast<float4*>(base + o_pack);
  sp.slot_max = reinterpret_cast<float*>(base + o_max);
  sp.slot_max2 = reinterpret_cast<float*>(base + o_max2);
  sp.slot_sum = reinterpret_cast<float*>(base + o_sum);
  sp.slot_rec = reinterpret_cast<ets::SlotRec*>(base + o_rec);
  sp.prep = reinterpret_cast<ets::PrepSlot*>(base + o_prep);
  sp.row_state = reinterpret_cast<ets::RowState*>(base + o_state);
  sp.walk = reinterpret_cast<float2*>(base + o_walk);
  sp.list_count = reinterpret_cast<uint32_t*>(base + o_count);
  sp.hist = reinterpret_cast<uint32_t*>(base + o_hist);
  sp.list = reinterpret_cast<uint64_t*>(base + o_list);
  sp.timers = (ETS_PHASE_CLOCKS && std::getenv("ETS_SPLIT_TIMERS")) ? reinterpret_cast<uint64_t*>(base + o_timers) : nullptr;  // (profiling builds only)
  s->split_row_wgs = row_wgs;
  return ETS_OK;
}


ets_status ensure_phist(ets_sampler* s) {
  if (s->d_phist) return ETS_OK;
  const size_t bytes = round_up(s->split_row_wgs * kPhistWordsHalf * sizeof(uint32_t), 256);
  ETS_HIP(s, hipMalloc(&s->d_phist, bytes));
  s->split.phist = static_cast<uint32_t*>(s->d_phist);
  return ETS_OK;
}

namespace {
bool g_static_arrive_dirty[kMaxDevices] = {};
}

bool* arrive_dirty_flag(ets_sampler* s) {
  if (!s->wb) return &s->arrive_dirty;
  return &g_static_arrive_dirty[s->device >= 0 && s->device < kMaxDevices ? s->device : 0];
}

}  // namespace ets_host

using namespace ets_host;

namespace {

bool dtype_ok(int32_t dtype) {
  return dtype == ETS_DTYPE_FLOAT || dtype == ETS_DTYPE_HALF || dtype == ETS_DTYPE_BFLOAT16 ||
         dtype == ETS_DTYPE_UINT16;
}

size_t dtype_size(int32_t dtype) { return dtype == ETS_DTYPE_FLOAT ? 4 : 2; }

// Device guard: the handle's buffers live on the device that was current at creation.
struct DeviceGuard {
  int prev = -1;
  bool switched = false;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) == hipSuccess && prev != dev) switched = (hipSetDevice(dev) == hipSuccess);
  }
  ~DeviceGuard() {
    if (switched) (void)hipSetDevice(prev);
  }
};

// ---- device timing ------------------------------------------------------------------------------
ets_status harvest_timing_slot(ets_sampler* s, int slot) {
  if (!s->t_busy[slot]) return ETS_OK;
  ETS_HIP(s, hipEventSynchronize(s->t_end[slot]));
  float ms = 0.0f;
  ETS_HIP(s, hipEventElapsedTime(&ms, s->t_begin[slot], s->t_end[slot]));
  s->t_busy[slot] = false;
  s->stats.calls += 1;
  s->stats.rows += static_cast<uint64_t>(s->t_rows[slot]);
  s->stats.last_call_us = static_cast<double>(ms) * 1e3;
  s->stats.aggregate_sampling_time_us += s->stats.last_call_us;
  return ETS_OK;
}

// Brackets one call's launches on `stream`; `slot` < 0 when timing is off.
ets_status timing_begin(ets_sampler* s, hipStream_t stream, int32_t rows, int* slot) {
  *slot = -1;
  if (!s->timing) return ETS_OK;
  const int k = static_cast<int>(s->t_next % ets_sampler::kTimingSlots);
  ets_status st = harvest_timing_slot(s, k);
  if (st != ETS_OK) return st;
  if (!s->t_begin[k]) {
    ETS_HIP(s, hipEventCreate(&s->t_begin[k]));
    ETS_HIP(s, hipEventCreate(&s->t_end[k]));
  }
  ETS_HIP(s, hipEventRecord(s->t_begin[k], stream));
  s->t_rows[k] = rows;
  *slot = k;
  return ETS_OK;
}

ets_status timing_end(ets_sampler* s, hipStream_t stream, int slot) {
  if (slot < 0) return ETS_OK;
  ETS_HIP(s, hipEventRecord(s->t_end[slot], stream));
  s->t_busy[slot] = true;
  s->t_next += 1;
  return ETS_OK;
}

// Workgroups per row of the partial kernels: enough to fill 256 CUs a few times over, but no
// segment under 4096 entries.
int row_splits(int32_t vocab, int32_t rows) {
  int splits = (1024 + rows - 1) / rows;
  const int max_by_len = (vocab + 4095) / 4096;
  if (splits > max_by_len) splits = max_by_len;
  if (splits > kMaxSplits) splits = kMaxSplits;
  return splits < 1 ? 1 : splits;
}

template <int DT>
ets_status launch_argmax(ets_sampler* s, const void* d_logits, int32_t batch, int64_t stride, int32_t* d_tokens,
                         hipStream_t stream, const int32_t* d_row_map = nullptr) {
  const int splits = row_splits(s->vocab, batch);
  const size_t esz = ets::ElemSize<DT>::value;
  const bool aligned = (reinterpret_cast<uintptr_t>(d_logits) % 16 == 0) && ((static_cast<size_t>(stride) * esz) % 16 == 0);
  uint64_t* partials = s->wb ? s->wb->partials : s->d_partials;
  const dim3 grid(splits, batch);
  if (aligned) {
    hipLaunchKernelGGL((ets::argmax_partial_kernel<DT, true>), grid, dim3(ets::kArgmaxBlock), 0, stream, d_logits, stride,
                       s->vocab, partials, d_row_map);
  } else {
    hipLaunchKernelGGL((ets::argmax_partial_kernel<DT, false>), grid, dim3(ets::kArgmaxBlock), 0, stream, d_logits, stride,
                       s->vocab, partials, d_row_map);
  }
  ETS_HIP(s, hipGetLastError());
  hipLaunchKernelGGL((ets::argmax_finish_kernel<DT>), dim3(batch), dim3(64), 0, stream, d_logits, stride, partials,
                     splits, d_tokens, d_row_map);
  ETS_HIP(s, hipGetLastError());
  return ETS_OK;
}

// Which draw follows the softmax (sampler.cpp:238-249).
int draw_mode(int32_t vocab, float topp, int32_t topk) {
  if (topk > 0 && topk < vocab) return ets::kDrawTopK;
  if (topp <= 0.0f || topp >= 1.0f) return ets::kDrawMultinomial;
  return ets::kDrawTopP;
}

float inverse_temperature_ctor(float temperature) {
  // sampler.cpp:178: static_cast<bool>(temperature) ? 1.0f / temperature : 0
  return (temperature != 0.0f) ? 1.0f / temperature : 0.0f;
}

ets_status ensure_scratch(ets_sampler* s) {
  if (s->d_scratch || s->wb) return ETS_OK;
  const size_t bytes = static_cast<size_t>(s->scratch_rows) * static_cast<size_t>(s->scratch_stride) * sizeof(uint64_t);
  ETS_HIP(s, hipMalloc(reinterpret_cast<void**>(&s->d_scratch), bytes));
  return ETS_OK;
}

ets_status argmax_device(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t rows, int64_t stride,
                         int32_t* d_tokens, hipStream_t stream, const int32_t* d_row_map) {
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      return launch_argmax<ets::kDtypeFloat>(s, d_logits, rows, stride, d_tokens, stream, d_row_map);
    case ETS_DTYPE_HALF:
      return launch_argmax<ets::kDtypeHalf>(s, d_logits, rows, stride, d_tokens, stream, d_row_map);
    case ETS_DTYPE_BFLOAT16:
      return launch_argmax<ets::kDtypeBFloat16>(s, d_logits, rows, stride, d_tokens, stream, d_row_map);
    default:
      return launch_argmax<ets::kDtypeUInt16>(s, d_logits, rows, stride, d_tokens, stream, d_row_map);
  }
}

const char* const kUint16Message =
    "stochastic sampling of UInt16 logits is not supported (integer softmax of the reference degenerates to "
    "0/1 weights); use temperature 0 or dequantise first";


// Whether rows with draw `draw` take the path that spreads a row over several workgroups.
// (Top-p rows; top-k rows whose k the slots' largest entries can vouch for, two per slot; multinomial
// rows, by five launches instead of three, unless the caller wants the probabilities written.)
bool use_split(const ets_sampler* s, const void* d_logits, int64_t stride, int32_t dtype, int draw, int32_t topk,
               bool probs = false) {
  if (s->split_mode == ETS_ROW_SPLIT_OFF) return false;
  if (draw == ets::kDrawMultinomial && probs) return false;
  if (draw == ets::kDrawTopK && topk > (s->vocab + ets::kSlot - 1) / ets::kSlot) return false;
  const size_t esz = dtype_size(dtype);
  const bool aligned = (reinterpret_cast<uintptr_t>(d_logits) % 16 == 0) && ((static_cast<size_t>(stride) * esz) % 16 == 0);
  if (!aligned || (s->vocab + ets::kSlot - 1) / ets::kSlot > ets::kMaxSlots) return false;
  return s->split_mode == ETS_ROW_SPLIT_ON || s->vocab >= 8192;
}

ets_status launch_split_walk_any(ets_sampler* s, const ets::RowParams& p, int32_t dtype, int32_t rows, hipStream_t stream) {
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      return launch_split_walk_f32(s, p, rows, stream);
    case ETS_DTYPE_HALF:
      return launch_split_walk_f16(s, p, rows, stream);
    default:
      return launch_split_walk_bf16(s, p, rows, stream);
  }
}

// The three launches for rows that use_split() accepted (each row's draw follows from its parameters).
// topk_rows: some row of the launch has a top-k of its own or the launch-wide one applies.
ets_status launch_split_any(ets_sampler* s, const ets::RowParams& p, int32_t dtype, int32_t rows, hipStream_t stream,
                            bool topk_rows) {
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      return launch_split_f32(s, p, rows, stream, topk_rows);
    case ETS_DTYPE_HALF:
      return launch_split_f16(s, p, rows, stream, topk_rows);
    default:
      return launch_split_bf16(s, p, rows, stream, topk_rows);
  }
}

ets_status rows_device(ets_sampler* s, const ets::RowParams& p, int32_t dtype, int32_t rows, hipStream_t stream,
                       int draw) {
  if (draw != ets::kDrawAny && use_split(s, p.logits, p.row_stride, dtype, draw, p.topk, p.probs != nullptr)) {
    if (draw == ets::kDrawMultinomial) return launch_split_walk_any(s, p, dtype, rows, stream);
    return launch_split_any(s, p, dtype, rows, stream, draw == ets::kDrawTopK);
  }
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      return launch_rows_f32(s, p, rows, stream, draw);
    case ETS_DTYPE_HALF:
      return launch_rows_f16(s, p, rows, stream, draw);
    default:
      return launch_rows_bf16(s, p, rows, stream, draw);
  }
}

ets_status sample_device(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch, int64_t stride,
                         int32_t* d_tokens, float* d_probs, ets_row_debug* d_debug, hipStream_t stream,
                         const ets::FusedOps* fused = nullptr) {
  if (s->inv_temperature == 0.0f) {
    // greedy: no coin is consumed (sampler.cpp:226-228)
    return argmax_device(s, d_logits, dtype, batch, stride, d_tokens, stream, nullptr);
  }
  if (dtype == ETS_DTYPE_UINT16) return fail(s, ETS_NOT_SUPPORTED, kUint16Message);
  ets_status st = ensure_scratch(s);
  if (st != ETS_OK) return st;
  ets::RowParams p = {};
  if (fused) p.fused = *fused;  // (the caller has checked that these rows take the path that applies them)
  p.logits = d_logits;
  p.row_stride = stride;
  p.vocab = s->vocab;
  p.inv_temperature = s->inv_temperature;
  p.topp = s->topp;
  p.topk = s->topk;
  p.rng = s->d_rng;
  p.tokens = d_tokens;
  p.probs = d_probs;
  p.debug = reinterpret_cast<ets::RowDebug*>(d_debug);
  p.scratch = s->wb ? s->wb->scratch : s->d_scratch;
  p.scratch_stride = s->wb ? s->wb->scratch_stride : s->scratch_stride;
  p.grid_cap = s->wb ? s->wb->scratch_rows : s->scratch_rows;
  p.lds_keys = s->lds_keys;
  p.row_map = nullptr;
  p.row_cfg = nullptr;
  return rows_device(s, p, dtype, batch, stream, draw_mode(s->vocab, s->topp, s->topk));
}

// ---- the entry point that allocates nothing ------------------------------------------------------
// Its work buffers live in this array: one copy per GPU the library runs on, held until the
// process ends.  Host code never uses the array's name as an address: the device address is looked
// up once per device (at the first handle created there) and kept.
constexpr size_t kStaticScratchBytes = size_t{32} << 20;
constexpr int kStaticArriveRows = 1024;
constexpr size_t kStaticPackBytes = 320 << 10;  // (256 workgroups x 64 slots x 16 bytes, and the rows' padding)
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

std::mutex g_static_mutex;
void* g_static_ptr[kMaxDevices] = {};

// With the handle's device current.
ets_status static_scratch_address(ets_sampler* s, int device, void** out) {
  if (device < 0 || device >= kMaxDevices) return fail(s, ETS_NOT_SUPPORTED, "device index beyond the static scratch table");
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[device]) {
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(s, e, "hipGetSymbolAddress(scratch)");
    g_static_ptr[device] = ptr;
  }
  *out = g_static_ptr[device];
  return ETS_OK;
}

// Lays the work buffers of a call of `rows` rows out from `base`; returns the bytes needed.
size_t layout_static(const ets_sampler* s, int32_t dtype, int32_t rows, char* base, WorkBuffers* wb) {
  ets::SplitParams& sp = wb->split;
  sp = ets::SplitParams{};
  sp.ns = (s->vocab + ets::kSlot - 1) / ets::kSlot;
  sp.ns_stride = static_cast<int32_t>(round_up(static_cast<size_t>(sp.ns), 4));
  sp.prep_cap = ets::kPrepCap;
  wb->max_row_wgs = 4;
  int g = (s->num_cus > 0 ? s->num_cus : 256) / rows;
  const int by_len = (sp.ns + 15) / 16;
  g = g > by_len ? by_len : g;
  g = g > wb->max_row_wgs ? wb->max_row_wgs : (g < 1 ? 1 : g);
  const size_t r = static_cast<size_t>(rows);
  const size_t phist_words = dtype == ETS_DTYPE_HALF ? kPhistWordsHalf : (dtype == ETS_DTYPE_BFLOAT16 ? kPhistWordsBFloat16 : 0);
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t here = at;
    at = round_up(at + bytes, 256);
    return base + here;
  };
  wb->tickets = reinterpret_cast<uint32_t*>(take(16 * sizeof(uint32_t)));  // always the array's first bytes: 0 between launches
  // (the same bytes whatever the call's sizes: the launches' number, and the slot values that the
  // workgroups of a fused launch hand to each other -- bytes that never hold anything else, so that what
  // a reader finds there is a whole record of some launch or the zeros the array starts with.  A fused
  // launch has at most one workgroup per compute unit and 64 slots per workgroup; a call whose rows
  // need more does not use it.)
  sp.arrive = reinterpret_cast<uint32_t*>(take(kStaticArriveRows * 2 * sizeof(uint32_t)));
  wb->arrive_rows = kStaticArriveRows;
  sp.slot_pack = reinterpret_cast<float4*>(take(kStaticPackBytes));
  wb->pack_bytes = kStaticPackBytes;
  sp.slot_max = reinterpret_cast<float*>(take(r * sp.ns_stride * sizeof(float)));
  sp.slot_max2 = reinterpret_cast<float*>(take(r * sp.ns_stride * sizeof(float)));
  sp.slot_sum = reinterpret_cast<float*>(take(r * sp.ns_stride * sizeof(float)));
  sp.slot_rec = reinterpret_cast<ets::SlotRec*>(take(r * sp.ns_stride * sizeof(ets::SlotRec)));
  sp.prep = reinterpret_cast<ets::PrepSlot*>(take(r * sp.prep_cap * sizeof(ets::PrepSlot)));
  sp.row_state = reinterpret_cast<ets::RowState*>(take(r * sizeof(ets::RowState)));
  sp.walk = reinterpret_cast<float2*>(take(r * sizeof(float2)));
  sp.list_count = reinterpret_cast<uint32_t*>(take(r * ets::kMaxRowWorkgroups * sizeof(uint32_t)));
  sp.hist = reinterpret_cast<uint32_t*>(take(r * g * ets::kHistBuckets * sizeof(uint32_t)));
  sp.phist = reinterpret_cast<uint32_t*>(take(r * g * phist_words * sizeof(uint32_t)));
  sp.list = reinterpret_cast<uint64_t*>(take(r * g * list_region(sp.ns, g) * sizeof(uint64_t)));
  sp.timers = nullptr;
  wb->scratch_stride = s->scratch_stride;
  wb->scratch_rows = rows < s->scratch_rows ? rows : s->scratch_rows;
  wb->scratch = reinterpret_cast<uint64_t*>(take(static_cast<size_t>(wb->scratch_rows) * static_cast<size_t>(s->scratch_stride) * sizeof(uint64_t)));
  wb->partials = reinterpret_cast<uint64_t*>(take(r * kMaxSplits * sizeof(uint64_t)));
  return at;
}

// ---- per-row parameters ------------------------------------------------------------------------
// Staging layout for a batch of B rows: reseed u64[B] | RowConfig[B] | row maps int32[4][B]
// (greedy, top-p, multinomial, top-k).
struct StageLayout {
  size_t reseed, cfg, maps, bytes;
  explicit StageLayout(int32_t rows) {
    reseed = 0;
    cfg = reseed + sizeof(uint64_t) * rows;
    maps = cfg + sizeof(ets::RowConfig) * rows;
    maps = (maps + 15) / 16 * 16;
    bytes = maps + sizeof(int32_t) * 4 * rows;
  }
};

// The upload of a staging buffer: a kernel that reads the pinned host buffer and writes the device
// copy.  (An asynchronous copy of a few kilobytes enqueued behind a kernel held the calling thread
// until that kernel had run -- tens of microseconds per call, serialising host and GPU; a launch
// does not.)
__global__ void stage_upload_kernel(const uint4* host, uint4* device, int32_t n) {
  const int32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) device[i] = host[i];
}
ets_status stage_upload(ets_sampler* s, const void* h, void* d, size_t bytes, hipStream_t stream) {
  const int32_t n = static_cast<int32_t>((bytes + 15) / 16);  // (both buffers are allocated in multiples of 256 bytes)
  hipLaunchKernelGGL(stage_upload_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, static_cast<const uint4*>(h),
                     static_cast<uint4*>(d), n);
  ETS_HIP(s, hipGetLastError());
  return ETS_OK;
}

__global__ void reseed_kernel(uint64_t* rng, const uint64_t* reseed, int32_t rows) {
  const int32_t b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < rows && reseed[b] != 0ull) rng[b] = reseed[b];
}

ets_status ensure_stage(ets_sampler* s) {
  if (s->h_stage) return ETS_OK;
  const StageLayout full(s->max_batch);
  s->stage_bytes = round_up(full.bytes, 256);
  ETS_HIP(s, hipHostMalloc(&s->h_stage, s->stage_bytes * ets_sampler::kStageSlots, hipHostMallocDefault));
  ETS_HIP(s, hipMalloc(&s->d_stage, s->stage_bytes));
  for (int i = 0; i < ets_sampler::kStageSlots; ++i) ETS_HIP(s, hipEventCreateWithFlags(&s->stage_event[i], hipEventDisableTiming));
  ETS_HIP(s, hipEventCreateWithFlags(&s->stage_done, hipEventDisableTiming));
  return ETS_OK;
}

// The pinned buffer this call fills: the next of the ring, once the upload last made from it has left it.
ets_status stage_host_buffer(ets_sampler* s, char** out) {
  const int slot = s->stage_next;
  if (s->stage_pending[slot]) {
    ETS_HIP(s, hipEventSynchronize(s->stage_event[slot]));
    s->stage_pending[slot] = false;
  }
  *out = static_cast<char*>(s->h_stage) + static_cast<size_t>(slot) * s->stage_bytes;
  return ETS_OK;
}
// Behind the upload from that buffer.
ets_status stage_uploaded(ets_sampler* s, hipStream_t stream) {
  const int slot = s->stage_next;
  ETS_HIP(s, hipEventRecord(s->stage_event[slot], stream));
  s->stage_pending[slot] = true;
  s->stage_next = (slot + 1) % ets_sampler::kStageSlots;
  return ETS_OK;
}

// The device copy of the staging data is read by the launches of the call that uploaded it.  A
// later call on the same stream is ordered behind them; one on another stream waits for the event
// recorded behind the earlier call's last launch.
ets_status stage_acquire(ets_sampler* s, hipStream_t stream) {
  if (s->stage_used && s->stage_stream != stream) ETS_HIP(s, hipStreamWaitEvent(stream, s->stage_done, 0));
  return ETS_OK;
}
ets_status stage_release(ets_sampler* s, hipStream_t stream) {
  ETS_HIP(s, hipEventRecord(s->stage_done, stream));
  s->stage_stream = stream;
  s->stage_used = true;
  return ETS_OK;
}

ets_status ensure_aux_streams(ets_sampler* s) {
  if (s->fork_event) return ETS_OK;
  ETS_HIP(s, hipStreamCreateWithFlags(&s->aux_stream, hipStreamNonBlocking));
  ETS_HIP(s, hipEventCreateWithFlags(&s->join_event, hipEventDisableTiming));
  ETS_HIP(s, hipEventCreateWithFlags(&s->fork_event, hipEventDisableTiming));
  return ETS_OK;
}

ets_status sample_device_configs(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch, int64_t stride,
                                 const ets_sampling_config* configs, int32_t* d_tokens, ets_row_debug* d_debug,
                                 hipStream_t stream) {
  ets_status st = ensure_stage(s);
  if (st != ETS_OK) return st;
  const StageLayout lay(batch);
  char* h = nullptr;
  st = stage_host_buffer(s, &h);
  if (st != ETS_OK) return st;
  char* d = static_cast<char*>(s->d_stage);
  uint64_t* h_reseed = reinterpret_cast<uint64_t*>(h + lay.reseed);
  ets::RowConfig* h_cfg = reinterpret_cast<ets::RowConfig*>(h + lay.cfg);
  int32_t* h_maps = reinterpret_cast<int32_t*>(h + lay.maps);
  std::memset(h, 0, lay.bytes);  // (what this call does not fill must not differ from call to call: see the comparison below)
  // Four groups of rows: arg-max rows, top-p and top-k rows that take the three-launch path,
  // multinomial rows that take the five-launch path, and every other row that draws (one launch of
  // the one-workgroup-per-row kernel, which picks each row's draw from its parameters).
  // maps[g * batch + i]: the i-th row of group g.
  enum { kGreedy = 0, kSplit = 1, kRows = 2, kWalk = 3 };
  int32_t count[4] = {0, 0, 0, 0};
  bool split_topk = false;  // some row of the three-launch group is a top-k row
  bool any_reseed = false;
  bool inv_ordinary = true;
  for (int32_t b = 0; b < batch; ++b) {
    const ets_sampling_config& c = configs[b];
    // temperature < 0: the handle's own (SamplingConfig: "-1 temperature means implementation default")
    const float inv = c.temperature < 0.0f ? s->inv_temperature : inverse_temperature_ctor(c.temperature);
    inv_ordinary = inv_ordinary && std::fabs(inv) < 3.0e38f;
    h_cfg[b].inv_temperature = inv;
    h_cfg[b].topp = c.top_p;
    h_cfg[b].topk = c.top_k;
    h_reseed[b] = c.seed;
    any_reseed = any_reseed || c.seed != 0;
    int group = kGreedy;
    if (inv != 0.0f) {
      const int draw = draw_mode(s->vocab, c.top_p, c.top_k);
      group = !use_split(s, d_logits, stride, dtype, draw, c.top_k) ? kRows : (draw == ets::kDrawMultinomial ? kWalk : kSplit);
      split_topk = split_topk || (group == kSplit && draw == ets::kDrawTopK);
    }
    if (group != kGreedy && dtype == ETS_DTYPE_UINT16) return fail(s, ETS_NOT_SUPPORTED, kUint16Message);
    h_maps[group * batch + count[group]++] = b;
  }
  if (count[kSplit] + count[kRows] + count[kWalk] > 0) {
    st = ensure_scratch(s);
    if (st != ETS_OK) return st;
  }
  st = stage_acquire(s, stream);
  if (st != ETS_OK) return st;
  if (!(s->stage_shadow_valid && s->stage_shadow.size() == lay.bytes && std::memcmp(s->stage_shadow.data(), h, lay.bytes) == 0)) {
    s->stage_shadow_valid = false;
    st = stage_upload(s, h, d, lay.bytes, stream);
    if (st != ETS_OK) return st;
    st = stage_uploaded(s, stream);
    if (st != ETS_OK) return st;
    s->stage_shadow.assign(h, lay.bytes);
    s->stage_shadow_valid = true;
  }
  if (any_reseed) {
    hipLaunchKernelGGL(reseed_kernel, dim3((batch + 255) / 256), dim3(256), 0, stream, s->d_rng,
                       reinterpret_cast<const uint64_t*>(d + lay.reseed), batch);
    ETS_HIP(s, hipGetLastError());
  }
  const int32_t* d_maps = reinterpret_cast<const int32_t*>(d + lay.maps);
  ets::RowParams p = {};
  p.logits = d_logits;
  p.row_stride = stride;
  p.vocab = s->vocab;
  p.inv_temperature = s->inv_temperature;
  p.topp = s->topp;
  p.topk = s->topk;
  p.rng = s->d_rng;
  p.tokens = d_tokens;
  p.probs = nullptr;
  p.debug = reinterpret_cast<ets::RowDebug*>(d_debug);
  p.scratch_stride = s->scratch_stride;
  p.lds_keys = s->lds_keys;
  p.row_cfg = reinterpret_cast<const ets::RowConfig*>(d + lay.cfg);
  // The groups touch different rows and different work buffers.  The one-workgroup-per-row launch
  // and the multinomial rows' five launches are the longest and run on the caller's stream; when
  // there are any, the other groups run beside them on a second stream, between a fork and a join (one of each: they cost more on the
  // host than the kernels they order).  The two launches that draw share the scratch rows (a
  // workgroup owns the scratch row of its index in its launch).
  const bool fork = count[kRows] + count[kWalk] > 0 && count[kSplit] + count[kGreedy] > 0;
  hipStream_t side = stream;
  if (fork) {
    st = ensure_aux_streams(s);
    if (st != ETS_OK) return st;
    side = s->aux_stream;
    ETS_HIP(s, hipEventRecord(s->fork_event, stream));
    ETS_HIP(s, hipStreamWaitEvent(side, s->fork_event, 0));
  }
  const bool both_draw = count[kRows] > 0 && count[kSplit] > 0;
  const int32_t share = both_draw ? s->scratch_rows / 2 : s->scratch_rows;
  // Every exit from here on goes through the join and the release below: a launch that fails must
  // not leave the side stream running unjoined, nor the staging copy unguarded, while kernels that
  // were launched before it still read the row maps and parameters.
  ets_status first = ETS_OK;
  if (count[kSplit] + count[kRows] > 0 && share < 1)
    first = fail(s, ETS_INTERNAL, "ets_sampler_sample_batch_configs: no scratch rows");
  if (first == ETS_OK && count[kRows] > 0) {
    p.scratch = s->d_scratch;
    p.grid_cap = share;
    p.row_map = d_maps + kRows * batch;
    first = rows_device(s, p, dtype, count[kRows], stream, ets::kDrawAny);
  }
  // (the multinomial rows' launches and the three launches of the top-p and top-k rows run side by side)
  s->cfg_inv_ordinary = inv_ordinary;
  if (first == ETS_OK && count[kWalk] > 0) {  // (no scratch rows, no tickets)
    p.row_map = d_maps + kWalk * batch;
    s->beside_rows = fork ? count[kSplit] : 0;
    first = launch_split_walk_any(s, p, dtype, count[kWalk], stream);
  }
  if (first == ETS_OK && count[kSplit] > 0) {
    p.scratch = s->d_scratch + (both_draw ? static_cast<int64_t>(share) * s->scratch_stride : 0);
    p.grid_cap = share;
    p.row_map = d_maps + kSplit * batch;
    s->beside_rows = fork ? count[kWalk] + count[kRows] : 0;  // (what the caller's stream runs meanwhile)
    first = launch_split_any(s, p, dtype, count[kSplit], side, split_topk);
  }
  s->beside_rows = 0;
  if (first == ETS_OK && count[kGreedy] > 0)
    first = argmax_device(s, d_logits, dtype, count[kGreedy], stride, d_tokens, side, d_maps + kGreedy * batch);
  const std::string first_message = s->last_error;
  ets_status closing = ETS_OK;
  if (fork) {
    hipError_t e = hipEventRecord(s->join_event, side);
    if (e == hipSuccess) e = hipStreamWaitEvent(stream, s->join_event, 0);
    if (e != hipSuccess) closing = hip_fail(s, e, "joining the side stream");
  }
  const ets_status released = stage_release(s, stream);
  if (first != ETS_OK) {
    s->last_error = first_message;
    return first;
  }
  return closing != ETS_OK ? closing : released;
}

}  // namespace

static_assert(sizeof(ets_row_debug) == sizeof(ets::RowDebug), "debug record layouts must agree");

extern "C" {

ets_status ets_sampler_create(int32_t vocab_size, float temperature, float topp, uint64_t rng_seed,
                              int32_t max_batch, ets_sampler** out) {
  if (!out) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_create: out is null");
  *out = nullptr;
  if (vocab_size < 1) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_create: vocab_size must be >= 1");
  // counts of a row's entries are carried in floats in places (exact below 2^24)
  if (vocab_size >= (1 << 24)) return fail(nullptr, ETS_NOT_SUPPORTED, "ets_sampler_create: vocab_size must be below 16777216");
  if (max_batch < 1) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_create: max_batch must be >= 1");
  // rows are the second dimension of several launch grids
  if (max_batch > 65535) return fail(nullptr, ETS_NOT_SUPPORTED, "ets_sampler_create: max_batch must be at most 65535");
  ets_sampler* s = new (std::nothrow) ets_sampler();
  if (!s) return fail(nullptr, ETS_MEMORY_ALLOCATION_FAILED, "ets_sampler_create: out of host memory");
  s->vocab = vocab_size;
  s->inv_temperature = inverse_temperature_ctor(temperature);
  s->topp = topp;
  s->topk = 0;
  s->max_batch = max_batch;
  if (const char* e = std::getenv("ETS_ROW_SPLIT")) {  // default of ets_sampler_set_row_split()
    const int mode = std::atoi(e);
    if (mode == ETS_ROW_SPLIT_ON || mode == ETS_ROW_SPLIT_OFF) s->split_mode = mode;
  }
  auto bail = [&](hipError_t e, const char* what) {
    ets_status st = hip_fail(nullptr, e, what);
    ets_sampler_destroy(s);
    return st;
  };
  hipError_t e = hipGetDevice(&s->device);
  if (e != hipSuccess) return bail(e, "hipGetDevice");
  int lds_limit = 0;
  e = hipDeviceGetAttribute(&lds_limit, hipDeviceAttributeMaxSharedMemoryPerBlock, s->device);
  if (e != hipSuccess) return bail(e, "hipDeviceGetAttribute(MaxSharedMemoryPerBlock)");
  {
    void* unused = nullptr;  // (kept per device; the entry point that allocates nothing reads it)
    ets_status sst = static_scratch_address(nullptr, s->device, &unused);
    if (sst != ETS_OK) {
      ets_sampler_destroy(s);
      return sst;
    }
  }
  e = hipDeviceGetAttribute(&s->num_cus, hipDeviceAttributeMultiprocessorCount, s->device);
  if (e != hipSuccess) return bail(e, "hipDeviceGetAttribute(MultiprocessorCount)");
  // the row kernel's static LDS (reduction scratch, selection buffer, histogram) stays under 16 KiB
  int keys = 1;
  while (static_cast<size_t>(keys) * 2 * sizeof(uint64_t) + 16384 <= static_cast<size_t>(lds_limit)) keys *= 2;
  // the radix sort of large candidate sets keeps a 48 KiB table in the key buffer
  if (keys < 8192) {
    ets_sampler_destroy(s);
    return fail(nullptr, ETS_INTERNAL, "ets_sampler_create: device reports too little LDS per workgroup");
  }
  s->lds_keys = keys;
  s->lds_bytes = static_cast<size_t>(keys) * sizeof(uint64_t);
  // two buffers of a row's sort keys (the radix sort of large candidate sets moves between them)
  s->scratch_stride = 2 * ((static_cast<int64_t>(vocab_size) + 63) / 64 * 64);

  // the row kernels keep one workgroup per CU resident (their LDS): that many rows of scratch
  s->scratch_rows = max_batch < s->num_cus ? max_batch : (s->num_cus > 0 ? s->num_cus : 1);
  e = hipMalloc(reinterpret_cast<void**>(&s->d_tickets), sizeof(uint32_t) * 16);
  if (e != hipSuccess) return bail(e, "hipMalloc(tickets)");
  e = hipMemset(s->d_tickets, 0, sizeof(uint32_t) * 16);
  if (e != hipSuccess) return bail(e, "hipMemset(tickets)");
  e = hipMalloc(reinterpret_cast<void**>(&s->d_rng), sizeof(uint64_t) * max_batch);
  if (e != hipSuccess) return bail(e, "hipMalloc(rng states)");
  e = hipMalloc(reinterpret_cast<void**>(&s->d_partials), sizeof(uint64_t) * max_batch * kMaxSplits);
  if (e != hipSuccess) return bail(e, "hipMalloc(argmax partials)");
  e = hipMalloc(&s->d_row, static_cast<size_t>(vocab_size) * 4);
  if (e != hipSuccess) return bail(e, "hipMalloc(row staging)");
  e = hipMalloc(reinterpret_cast<void**>(&s->d_token), sizeof(int32_t));
  if (e != hipSuccess) return bail(e, "hipMalloc(token staging)");
  // row b's stream starts at rng_seed + b
  uint64_t* seeds = new (std::nothrow) uint64_t[max_batch];
  if (!seeds) {
    ets_sampler_destroy(s);
    return fail(nullptr, ETS_MEMORY_ALLOCATION_FAILED, "ets_sampler_create: out of host memory");
  }
  for (int32_t b = 0; b < max_batch; ++b) seeds[b] = rng_seed + static_cast<uint64_t>(b);
  e = hipMemcpy(s->d_rng, seeds, sizeof(uint64_t) * max_batch, hipMemcpyHostToDevice);
  delete[] seeds;
  if (e != hipSuccess) return bail(e, "hipMemcpy(rng states)");
  *out = s;
  return ETS_OK;
}

ets_status ets_sampler_create_default(int32_t vocab_size, float temperature, int32_t max_batch, ets_sampler** out) {
  return ets_sampler_create(vocab_size, temperature, 0.9f, static_cast<uint64_t>(std::time(nullptr)), max_batch, out);
}

ets_status ets_sampler_destroy(ets_sampler* s) {
  if (!s) return ETS_OK;
  {
    DeviceGuard g(s->device);
    (void)hipFree(s->d_rng);
    (void)hipFree(s->d_tickets);
    (void)hipFree(s->d_scratch);
    (void)hipFree(s->d_split);
    (void)hipFree(s->d_phist);
    (void)hipFree(s->d_partials);
    (void)hipFree(s->d_row);
    (void)hipFree(s->d_token);
    (void)hipFree(s->d_stage);
    if (s->h_stage) (void)hipHostFree(s->h_stage);
    if (s->aux_stream) (void)hipStreamDestroy(s->aux_stream);
    if (s->join_event) (void)hipEventDestroy(s->join_event);
    if (s->fork_event) (void)hipEventDestroy(s->fork_event);
    for (int i = 0; i < ets_sampler::kStageSlots; ++i) {
      if (s->stage_event[i]) (void)hipEventDestroy(s->stage_event[i]);
    }
    if (s->stage_done) (void)hipEventDestroy(s->stage_done);
    for (int i = 0; i < ets_sampler::kTimingSlots; ++i) {
      if (s->t_begin[i]) (void)hipEventDestroy(s->t_begin[i]);
      if (s->t_end[i]) (void)hipEventDestroy(s->t_end[i]);
    }
  }
  delete s;
  return ETS_OK;
}

ets_status ets_sampler_set_temperature(ets_sampler* s, float temperature) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_temperature: null handle");
  if (temperature < 0.0f) temperature = 0.0f;
  s->inv_temperature = (temperature != 0.0f) ? 1.0f / temperature : 0.0f;
  return ETS_OK;
}

ets_status ets_sampler_set_topk(ets_sampler* s, int32_t topk) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_topk: null handle");
  s->topk = topk;
  return ETS_OK;
}

ets_status ets_sampler_set_row_split(ets_sampler* s, int32_t mode) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_row_split: null handle");
  if (mode != ETS_ROW_SPLIT_AUTO && mode != ETS_ROW_SPLIT_ON && mode != ETS_ROW_SPLIT_OFF)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_set_row_split: unknown mode");
  s->split_mode = mode;
  return ETS_OK;
}

ets_status ets_sampler_set_topp(ets_sampler* s, float topp) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_topp: null handle");
  s->topp = topp;
  return ETS_OK;
}

ets_status ets_sampler_sample_batch_debug(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                          int64_t row_stride_elems, int32_t* d_tokens, float* d_probs,
                                          ets_row_debug* d_debug, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch: null handle");
  s->last_error.clear();
  if (!d_logits || !d_tokens) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch: null pointer");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch: unsupported dtype");
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch: batch exceeds the handle's max_batch");
  if (row_stride_elems < s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch: row stride smaller than vocab_size");
  if (batch == 0) return ETS_OK;
  DeviceGuard g(s->device);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  int slot = -1;
  ets_status st = timing_begin(s, stream, batch, &slot);
  if (st != ETS_OK) return st;
  st = sample_device(s, d_logits, dtype, batch, row_stride_elems, d_tokens, d_probs, d_debug, stream);
  if (st != ETS_OK) return st;
  return timing_end(s, stream, slot);
}

ets_status ets_sampler_sample_batch(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                    int64_t row_stride_elems, int32_t* d_tokens, void* hip_stream) {
  return ets_sampler_sample_batch_debug(s, d_logits, dtype, batch, row_stride_elems, d_tokens, nullptr, nullptr,
                                        hip_stream);
}

ets_status ets_sampler_sample_batch_static(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                           int64_t row_stride_elems, int32_t* d_tokens, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_static: null handle");
  s->last_error.clear();
  if (!d_logits || !d_tokens) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_static: null pointer");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_static: unsupported dtype");
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_static: batch exceeds the handle's max_batch");
  if (row_stride_elems < s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_static: row stride smaller than vocab_size");
  if (batch == 0) return ETS_OK;
  DeviceGuard g(s->device);
  void* base = nullptr;
  ets_status st = static_scratch_address(s, s->device, &base);
  if (st != ETS_OK) return st;
  WorkBuffers wb;
  const size_t need = layout_static(s, dtype, batch, static_cast<char*>(base), &wb);
  if (need > kStaticScratchBytes) {
    return fail(s, ETS_INVALID_ARGUMENT,
                "ets_sampler_sample_batch_static: batch x vocab_size needs " + std::to_string(need) +
                    " bytes of work buffers, the static scratch holds " + std::to_string(kStaticScratchBytes) +
                    "; use ets_sampler_sample_batch");
  }
  s->wb = &wb;
  st = sample_device(s, d_logits, dtype, batch, row_stride_elems, d_tokens, nullptr, nullptr, static_cast<hipStream_t>(hip_stream));
  s->wb = nullptr;
  return st;
}

ets_status ets_sampler_sample_batch_configs(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                            int64_t row_stride_elems, const ets_sampling_config* configs,
                                            int32_t* d_tokens, ets_row_debug* d_debug, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_configs: null handle");
  s->last_error.clear();
  if (!d_logits || !d_tokens || !configs)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_configs: null pointer");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_configs: unsupported dtype");
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_configs: batch exceeds the handle's max_batch");
  if (row_stride_elems < s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_configs: row stride smaller than vocab_size");
  if (batch == 0) return ETS_OK;
  DeviceGuard g(s->device);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  int slot = -1;
  ets_status st = timing_begin(s, stream, batch, &slot);
  if (st != ETS_OK) return st;
  st = sample_device_configs(s, d_logits, dtype, batch, row_stride_elems, configs, d_tokens, d_debug, stream);
  if (st != ETS_OK) return st;
  return timing_end(s, stream, slot);
}

ets_status ets_sampler_gumbel_max_batch(ets_sampler* s, const void* d_logits, int32_t dtype, int32_t batch,
                                        int64_t row_stride_elems, const float* temperatures, int32_t n_temperatures,
                                        const float* d_noise, int32_t* d_tokens, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: null handle");
  s->last_error.clear();
  if (!d_logits || !d_tokens || !temperatures)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: null pointer");
  if (dtype != ETS_DTYPE_FLOAT && dtype != ETS_DTYPE_HALF && dtype != ETS_DTYPE_BFLOAT16)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: element type must be Float, Half or BFloat16");
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: batch exceeds the handle's max_batch");
  if (row_stride_elems < s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: row stride smaller than vocab_size");
  if (n_temperatures != 1 && n_temperatures != batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_gumbel_max_batch: one temperature, or one per row");
  if (batch == 0) return ETS_OK;
  DeviceGuard g(s->device);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  // one temperature travels as a kernel argument; one per row goes through the pinned staging
  // buffer (waiting, if need be, until the previous upload has left it)
  ets_status st = ETS_OK;
  const float* d_row_temperatures = nullptr;
  if (n_temperatures > 1) {
    st = ensure_stage(s);
    if (st != ETS_OK) return st;
    char* h = nullptr;
    st = stage_host_buffer(s, &h);
    if (st != ETS_OK) return st;
    std::memcpy(h, temperatures, sizeof(float) * n_temperatures);
    st = stage_acquire(s, stream);
    if (st != ETS_OK) return st;
    s->stage_shadow_valid = false;  // (the device copy holds temperatures from here on)
    st = stage_upload(s, h, s->d_stage, sizeof(float) * n_temperatures, stream);
    if (st != ETS_OK) return st;
    st = stage_uploaded(s, stream);
    if (st != ETS_OK) return st;
    d_row_temperatures = static_cast<const float*>(s->d_stage);
  }
  const float temperature = temperatures[0];
  int slot = -1;
  st = timing_begin(s, stream, batch, &slot);
  if (st != ETS_OK) return st;
  // the draw is bound by instruction issue, not by bytes: more, smaller segments than the arg-max
  int splits = (2048 + batch - 1) / batch;
  const int max_by_len = (s->vocab + 1023) / 1024;
  if (splits > max_by_len) splits = max_by_len;
  if (splits > kMaxSplits) splits = kMaxSplits;
  if (splits < 1) splits = 1;
  const dim3 grid(splits, batch);
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      hipLaunchKernelGGL((ets::gumbel_partial_kernel<ets::kDtypeFloat>), grid, dim3(ets::kArgmaxBlock), 0, stream, d_logits,
                         row_stride_elems, s->vocab, temperature, d_row_temperatures, d_noise, s->d_rng, s->d_partials);
      break;
    case ETS_DTYPE_HALF:
      hipLaunchKernelGGL((ets::gumbel_partial_kernel<ets::kDtypeHalf>), grid, dim3(ets::kArgmaxBlock), 0, stream, d_logits,
                         row_stride_elems, s->vocab, temperature, d_row_temperatures, d_noise, s->d_rng, s->d_partials);
      break;
    default:
      hipLaunchKernelGGL((ets::gumbel_partial_kernel<ets::kDtypeBFloat16>), grid, dim3(ets::kArgmaxBlock), 0, stream,
                         d_logits, row_stride_elems, s->vocab, temperature, d_row_temperatures, d_noise, s->d_rng,
                         s->d_partials);
      break;
  }
  ETS_HIP(s, hipGetLastError());
  hipLaunchKernelGGL(ets::gumbel_finish_kernel, dim3(batch), dim3(64), 0, stream, s->d_partials, splits,
                     d_noise ? 0 : 1, s->d_rng, d_tokens);
  ETS_HIP(s, hipGetLastError());
  if (n_temperatures > 1) {
    st = stage_release(s, stream);
    if (st != ETS_OK) return st;
  }
  return timing_end(s, stream, slot);
}

ets_status ets_sampler_set_timing(ets_sampler* s, int32_t enabled) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_timing: null handle");
  s->last_error.clear();
  s->timing = enabled != 0;
  return ETS_OK;
}

ets_status ets_sampler_get_stats(ets_sampler* s, ets_sampler_stats* out) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_get_stats: null handle");
  s->last_error.clear();
  if (!out) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_get_stats: null pointer");
  DeviceGuard g(s->device);
  // oldest first, so that last_call_us ends up as the most recent call
  for (int i = 0; i < ets_sampler::kTimingSlots; ++i) {
    const int slot = static_cast<int>((s->t_next + static_cast<uint64_t>(i)) % ets_sampler::kTimingSlots);
    ets_status st = harvest_timing_slot(s, slot);
    if (st != ETS_OK) return st;
  }
  *out = s->stats;
  return ETS_OK;
}

ets_status ets_sampler_reset_stats(ets_sampler* s) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_reset_stats: null handle");
  s->last_error.clear();
  DeviceGuard g(s->device);
  ets_sampler_stats scratch;
  ets_status st = ets_sampler_get_stats(s, &scratch);  // drains calls still in flight
  if (st != ETS_OK) return st;
  s->stats = ets_sampler_stats{};
  return ETS_OK;
}

ets_status ets_sampler_sample(ets_sampler* s, const void* logits, int32_t dtype, int32_t* token_out) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_sample: null handle");
  s->last_error.clear();
  if (!logits || !token_out) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample: null pointer");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample: unsupported dtype");
  DeviceGuard g(s->device);
  ETS_HIP(s, hipMemcpy(s->d_row, logits, static_cast<size_t>(s->vocab) * dtype_size(dtype), hipMemcpyHostToDevice));
  ets_status st = sample_device(s, s->d_row, dtype, 1, s->vocab, s->d_token, nullptr, nullptr, nullptr);
  if (st != ETS_OK) return st;
  ETS_HIP(s, hipMemcpy(token_out, s->d_token, sizeof(int32_t), hipMemcpyDeviceToHost));
  return ETS_OK;
}

ets_status ets_sampler_set_rng_states(ets_sampler* s, int32_t first_row, int32_t count, const uint64_t* states) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_set_rng_states: null handle");
  if (!states || first_row < 0 || count < 0 || first_row + count > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_set_rng_states: bad range or null pointer");
  if (count == 0) return ETS_OK;
  DeviceGuard g(s->device);
  ETS_HIP(s, hipMemcpy(s->d_rng + first_row, states, sizeof(uint64_t) * count, hipMemcpyHostToDevice));
  return ETS_OK;
}

ets_status ets_sampler_get_rng_states(ets_sampler* s, int32_t first_row, int32_t count, uint64_t* states) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_get_rng_states: null handle");
  if (!states || first_row < 0 || count < 0 || first_row + count > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_get_rng_states: bad range or null pointer");
  if (count == 0) return ETS_OK;
  DeviceGuard g(s->device);
  ETS_HIP(s, hipMemcpy(states, s->d_rng + first_row, sizeof(uint64_t) * count, hipMemcpyDeviceToHost));
  return ETS_OK;
}

ets_status ets_sample_from_logits(ets_sampler* s, const void* data, int32_t dtype, int32_t rank, const int64_t* sizes,
                                  int32_t* token_out) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sample_from_logits: null handle");
  s->last_error.clear();
  if (!data || !sizes || !token_out || rank < 1)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits: null pointer or rank < 1");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "Unsupported dtype in sample_from_logits");
  const int64_t vocab = sizes[rank - 1];
  if (vocab != s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits: last dimension differs from the sampler's vocab_size");
  const char* p = static_cast<const char*>(data);
  if (rank == 3) {
    if (sizes[1] < 1) return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits: empty sequence dimension");
    p += static_cast<size_t>((sizes[1] - 1) * vocab) * dtype_size(dtype);  // last position of batch 0 (util.h:48-51)
  }
  return ets_sampler_sample(s, p, dtype, token_out);
}

ets_status ets_sample_from_logits_batch(ets_sampler* s, const void* d_data, int32_t dtype, int32_t rank,
                                        const int64_t* sizes, int32_t* d_tokens, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: null handle");
  s->last_error.clear();
  if (!d_data || !sizes || !d_tokens) return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: null pointer");
  if (rank != 2 && rank != 3)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: the tensor must be [batch, vocab] or [batch, seq, vocab]");
  if (!dtype_ok(dtype)) return fail(s, ETS_INVALID_ARGUMENT, "Unsupported dtype in sample_from_logits");
  const int64_t vocab = sizes[rank - 1];
  if (vocab != s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: last dimension differs from the sampler's vocab_size");
  const int64_t batch = sizes[0];
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: batch exceeds the handle's max_batch");
  const char* first = static_cast<const char*>(d_data);
  int64_t stride = vocab;
  if (rank == 3) {
    if (sizes[1] < 1) return fail(s, ETS_INVALID_ARGUMENT, "ets_sample_from_logits_batch: empty sequence dimension");
    // the last position of every batch entry (util.h:48-51 takes batch 0's)
    first += static_cast<size_t>((sizes[1] - 1) * vocab) * dtype_size(dtype);
    stride = sizes[1] * vocab;
  }
  return ets_sampler_sample_batch(s, first, dtype, static_cast<int32_t>(batch), stride, d_tokens, hip_stream);
}

ets_status ets_logits_to_token(const void* data, int32_t dtype, int32_t rank, const int64_t* sizes, float temperature,
                               int32_t* token_out) {
  if (!data || !sizes || !token_out || rank < 1)
    return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logits_to_token: null pointer or rank < 1");
  const int64_t vocab = sizes[rank - 1];
  if (vocab < 1 || vocab > INT32_MAX) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logits_to_token: bad vocab size");
  // The reference builds a temporary Sampler per call (util.h:67-69), which costs it nothing; here
  // a handle owns device buffers, so each thread keeps the one it built last and reuses it while
  // the device and the vocabulary stay the same.  What the temporary object would have had -- the
  // 2-argument constructor's parameters and a clock seed -- is set again on every call.
  struct Cached {
    ets_sampler* handle = nullptr;
    // (at thread or process exit the HIP runtime may be gone already: then nothing is freed)
    ~Cached() {
      int n = 0;
      if (handle && hipGetDeviceCount(&n) == hipSuccess && n > 0) ets_sampler_destroy(handle);
    }
  };
  thread_local Cached cache;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) device = -1;
  ets_sampler* s = cache.handle;
  if (s) {
    // a device reset since the last call leaves the handle's buffers dangling: it is dropped, not freed
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, s->d_rng) != hipSuccess) {
      (void)hipGetLastError();
      delete s;
      cache.handle = nullptr;
      s = nullptr;
    }
  }
  if (!s || s->vocab != vocab || s->device != device) {
    ets_sampler_destroy(cache.handle);
    cache.handle = nullptr;
    ets_status st = ets_sampler_create_default(static_cast<int32_t>(vocab), temperature, 1, &cache.handle);
    if (st != ETS_OK) return st;
    s = cache.handle;
  } else {
    s->inv_temperature = inverse_temperature_ctor(temperature);  // sampler.cpp:183-187
    s->topp = 0.9f;
    s->topk = 0;
    const uint64_t seed = static_cast<uint64_t>(std::time(nullptr));
    if (s->inv_temperature != 0.0f) {  // (the arg-max draws no coin)
      ets_status st = ets_sampler_set_rng_states(s, 0, 1, &seed);
      if (st != ETS_OK) return st;
    }
  }
  ets_status st = ets_sample_from_logits(s, data, dtype, rank, sizes, token_out);
  if (st != ETS_OK) g_thread_error = s->last_error;
  return st;
}

uint32_t ets_random_u32(uint64_t* state) {
  uint64_t s = *state;
  s ^= s >> 12;
  s ^= s << 25;
  s ^= s >> 27;
  *state = s;
  return static_cast<uint32_t>((s * 0x2545F4914F6CDD1Dull) >> 32);
}

float ets_random_f32(uint64_t* state) { return static_cast<float>(ets_random_u32(state) >> 8) / 16777216.0f; }

const char* ets_sampler_last_error(const ets_sampler* s) { return s ? s->last_error.c_str() : g_thread_error.c_str(); }

const char* ets_version(void) { return "et_sampler 0.1 (gfx950)"; }

}  // extern "C"

#include "ets_logit_chain.h"
