// Host-side state shared by the translation units of libet_sampler.so: the handle behind the C ABI
// of include/et_sampler.h, the work buffers of a call, error helpers, and the launchers that each
// translation unit of kernels exports to the others (every element type's kernels are compiled in
// a file of their own, so that an edit to one kernel does not rebuild all of them one after the other).
#pragma once

#include "../../include/et_sampler.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <string>

#include "ets_kernels.h"
#include "ets_split.h"

// Device memory a call works in beyond its inputs and outputs, when it is not the handle's own:
// the entry point that allocates nothing lays it out inside the library's static array.
struct WorkBuffers {
  ets::SplitParams split = {};
  uint64_t* scratch = nullptr;  // [rows, scratch_stride] keys of the general draw
  uint32_t* tickets = nullptr;
  int32_t scratch_rows = 0;
  int64_t scratch_stride = 0;
  uint64_t* partials = nullptr;  // [rows, kMaxSplits] arg-max partial results
  int max_row_wgs = 0;           // workgroups of pass 2 per row, at most
  int arrive_rows = 0;           // rows `arrive` is laid out for
  size_t pack_bytes = 0;         // bytes set aside for the slot values a fused launch's workgroups hand to each other
};

struct ets_sampler {
  const WorkBuffers* wb = nullptr;  // set for the duration of a call that brings its own buffers
  int32_t vocab = 0;
  float inv_temperature = 0.0f;
  float topp = 0.9f;
  int32_t topk = 0;
  int32_t max_batch = 0;
  int device = 0;
  int lds_keys = 0;            // keys that fit in the dynamic LDS sort buffer (power of two)
  size_t lds_bytes = 0;
  int64_t scratch_stride = 0;  // keys per row of candidate scratch (twice the vocabulary, rounded up)
  uint64_t* d_rng = nullptr;       // [max_batch]
  uint32_t* d_tickets = nullptr;   // row counters of the row kernels' launches (0 between launches), one per draw
  int32_t scratch_rows = 0;        // rows of candidate scratch: one per workgroup that can be resident, not one per row
  uint64_t* d_scratch = nullptr;   // [scratch_rows, scratch_stride], allocated on first stochastic use
  uint64_t* d_partials = nullptr;  // [max_batch, kMaxSplits] argmax partial results
  void* d_row = nullptr;           // staging for one host row (vocab * 4 bytes)
  int32_t* d_token = nullptr;      // staging for one token
  // work buffers of the path that spreads a row over several workgroups (ets_split.h): one
  // allocation, made on first use
  size_t split_row_wgs = 0;  // (row, workgroup) pairs of the largest launch
  int split_mode = 0;  // ETS_ROW_SPLIT_AUTO
  int num_cus = 0;
  void* d_split = nullptr;
  void* d_phist = nullptr;  // pattern histograms of 16-bit rows, allocated on their first use
  bool cfg_inv_ordinary = false;  // per-row parameters of the call in progress: every inverse temperature is finite
  int32_t beside_rows = 0;  // rows of other launches that run beside this one on another stream (set for the duration of a call)
  bool arrive_dirty = false;  // a fused launch was not followed by its finish kernel: the next one is given a number of its own first
  ets::SplitParams split = {};
  // per-row sampling parameters of ets_sampler_sample_batch_configs(): pinned host staging buffers
  // that take turns (a call fills the next one and waits only if the upload made from it
  // kStageSlots calls ago has not left it yet, so the host runs ahead of the GPU), the device copy,
  // and per buffer the event that says its last upload has left it
  static constexpr int kStageSlots = 4;
  void* h_stage = nullptr;  // kStageSlots buffers of stage_bytes each, one after the other
  size_t stage_bytes = 0;
  void* d_stage = nullptr;
  hipEvent_t stage_event[kStageSlots] = {};
  bool stage_pending[kStageSlots] = {};
  int stage_next = 0;
  // what the device copy holds (a call whose staging data equals it uploads nothing: the parameters
  // of a serving loop's rows rarely change from one step to the next)
  std::string stage_shadow;
  bool stage_shadow_valid = false;
  // the last stream a call that uses the staging copy ran on, and the event behind its launches: a
  // call on another stream waits for it before it overwrites the device copy
  hipEvent_t stage_done = nullptr;
  hipStream_t stage_stream = nullptr;
  bool stage_used = false;
  // ets_sampler_sample_batch_configs(): rows that take different launches run side by side, one
  // group on the call's stream and the others on a second stream (default priority) that starts
  // behind the call's stream and is joined again before the call returns
  hipStream_t aux_stream = nullptr;
  hipEvent_t fork_event = nullptr;
  hipEvent_t join_event = nullptr;
  // opt-in device timing (ets_sampler_set_timing): a ring of event pairs around the launches of a
  // call, harvested when a slot is reused or the totals are read
  bool timing = false;
  static constexpr int kTimingSlots = 32;
  hipEvent_t t_begin[kTimingSlots] = {};
  hipEvent_t t_end[kTimingSlots] = {};
  int32_t t_rows[kTimingSlots] = {};
  bool t_busy[kTimingSlots] = {};
  uint64_t t_next = 0;
  ets_sampler_stats stats = {};
  std::string last_error;
};

namespace ets_host {

constexpr int kMaxSplits = 64;    // arg-max partial results per row
constexpr int kMaxDevices = 64;

// Words of packed 16-bit counters per (row, workgroup) of the pattern histogram: what fits in
// pass 2's LDS next to the expf table.
constexpr int kPhistWordsHalf = 24576, kPhistWordsBFloat16 = 8192;

// Records `msg` in the handle (or, without one, for the calling thread) and returns `code`.
ets_status fail(ets_sampler* s, ets_status code, const std::string& msg);
ets_status hip_fail(ets_sampler* s, hipError_t e, const char* what);

#define ETS_HIP(s, call)                                             \
  do {                                                               \
    hipError_t e_ = (call);                                          \
    if (e_ != hipSuccess) return ::ets_host::hip_fail(s, e_, #call); \
  } while (0)

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Raises a kernel's dynamic-LDS limit to `bytes` on the handle's device.  The limit is kept per
// kernel and device, so it is set again only when a handle asks for more than was set before.
ets_status allow_dynamic_lds(ets_sampler* s, const void* kernel, size_t bytes, std::atomic<size_t>* set_bytes);

// Work buffers of the several-workgroups-per-row path, allocated on first use (not for a call
// that brings its own).
ets_status ensure_split(ets_sampler* s);
ets_status ensure_phist(ets_sampler* s);
// Workgroups of pass 2 per row for a launch of `rows` rows that shares the compute units with `beside`
// rows of other launches.  (The work buffers are sized for beside = 0, which covers every other case.)
int pass2_workgroups(const ets_sampler* s, int32_t rows, int32_t ns, int32_t beside);
// Whether the arrival counters of the fused launch may hold something other than 0 (a fused launch
// whose finish kernel was never launched): the handle's own flag, or, for a call that works in the
// library's static array, that device's.
bool* arrive_dirty_flag(ets_sampler* s);
int32_t list_region(int32_t ns, int g);

// ---- launchers, one translation unit per element type -------------------------------------------
// One workgroup per row (ets_kernels.h, sample_rows_kernel); `draw`: ets::kDraw*.
ets_status launch_rows_f32(ets_sampler* s, const ets::RowParams& p, int32_t batch, hipStream_t stream, int draw);
ets_status launch_rows_f16(ets_sampler* s, const ets::RowParams& p, int32_t batch, hipStream_t stream, int draw);
ets_status launch_rows_bf16(ets_sampler* s, const ets::RowParams& p, int32_t batch, hipStream_t stream, int draw);
// Several workgroups per row (ets_split.h): top-p rows and, with `topk_rows`, launches in which
// some row has a top-k.
ets_status launch_split_f32(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream, bool topk_rows);
ets_status launch_split_f16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream, bool topk_rows);
ets_status launch_split_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream, bool topk_rows);
// Multinomial rows, several workgroups per row.
ets_status launch_split_walk_f32(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);
ets_status launch_split_walk_f16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);
ets_status launch_split_walk_bf16(ets_sampler* s, const ets::RowParams& p, int32_t rows, hipStream_t stream);

}  // namespace ets_host
