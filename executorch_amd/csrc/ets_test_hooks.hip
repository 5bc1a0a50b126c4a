// TEST AND MEASUREMENT HOOKS (csrc/ets_test_hooks.h), built into a library of their own,
// libet_sampler_hooks.so: tests and the benchmark load it, the product library does not hold them.
// The kernels here instantiate the same device functions as the product (same headers, same
// compiler flags).
#include "ets_test_hooks.h"

#include <hip/hip_runtime.h>

#include <string>

#include "ets_host.h"

namespace ets {

// ---- measurement floors (hooks for the benchmark: what a launch and a plain read cost here) ------
__global__ void empty_kernel() {}

// dst = src, 16 bytes per lane and access as in the row kernels: the transfer of known size that the
// hardware's fetch and write counters are scaled by.
__global__ void __launch_bounds__(256) copy_probe_kernel(const uint4* src, uint4* dst, int64_t n_vec) {
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; j < n_vec; j += static_cast<int64_t>(gridDim.x) * 256)
    dst[j] = src[j];
}

// Every workgroup reads its share of `n_vec` 16-byte vectors (eight loads in flight per lane) and
// keeps an XOR of them: nothing but the read.
__global__ void __launch_bounds__(256) read_floor_kernel(const uint4* data, int64_t n_vec, uint32_t* out) {
  const int64_t per = (n_vec + gridDim.x - 1) / gridDim.x;
  const int64_t lo = per * blockIdx.x, hi = lo + per < n_vec ? lo + per : n_vec;
  uint32_t acc = 0u;
  for (int64_t j = lo + threadIdx.x; j < hi; j += 8 * 256) {
    uint4 r[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t jk = j + k * 256;
      r[k] = data[jk < hi ? jk : j];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) acc ^= r[k].x ^ r[k].y ^ r[k].z ^ r[k].w;
  }
  if (acc == 0x9e3779b9u) out[0] = acc;  // (keeps the loads alive; practically never taken)
}

// Evaluates expf_exact over an array (test hook for the exhaustive comparison with libm).
__global__ void __launch_bounds__(256) expf_exact_kernel(const float* x, float* y, int64_t n) {
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = kExp2Table[threadIdx.x];
  __syncthreads();
  for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += 256ll * gridDim.x) {
    const float v = x[i];
    // non-positive arguments go through the branch-free form the sampler uses
    y[i] = (v <= 0.0f) ? expf_nonpositive(v, tab) : expf_exact(v, tab);
  }
}

// Sequential float sum of an array by one workgroup (test hook).  Same loop structure as
// scan_row: groups of kGroup chunks of 4 elements per lane through seq_sum_group, the remainder
// through seq_sum_chunk.
__global__ void __launch_bounds__(kBlock)
seq_sum_kernel(const float* a, int32_t n, float s0, float threshold, float* sum_out, int32_t* stop_out) {
  __shared__ BlockScratch sm;
  constexpr int R = 4;
  const int tid = threadIdx.x;
  SeqSum st = {s0, -1, 0u};
  bool stopped = false;
  int base = 0;
  for (; !stopped && base + kGroup * kBlock * R <= n; base += kGroup * kBlock * R) {
    const float scale = fast_scale(st.s);
    FastAcc acc[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) acc[u] = {0.0f, 0.0f};
    uint32_t bits[kGroup][R];
    int first[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      first[u] = base + (u * kBlock + tid) * R;
#pragma unroll
      for (int e = 0; e < R; ++e) {
        const float v = a[first[u] + e];
        bits[u][e] = __float_as_uint(v);
        fast_fold(acc[u], v, scale);
      }
    }
    stopped = seq_sum_group<kGroup, R>(st, bits, acc, scale, first, n, threshold, sm);
  }
  for (; !stopped && base < n; base += kBlock * R) {
    uint32_t bits[R];
    const int first = base + tid * R;
#pragma unroll
    for (int e = 0; e < R; ++e) bits[e] = (first + e < n) ? __float_as_uint(a[first + e]) : 0u;
    stopped = seq_sum_chunk<R>(st, bits, first, n, threshold, sm);
  }
  if (threadIdx.x == 0) {
    *sum_out = st.s;
    *stop_out = st.stop_index;
  }
}

// What a hand-over between two workgroups costs: workgroup 0 publishes a word (release, device
// scope) and workgroup `partner` polls it (acquire), then answers through a second word; `hops`
// round trips.  Workgroups go to the dies (XCDs) in turn by their index, so partner 1 sits on
// another die and partner 8 on the same one.  Every wait is bounded by `spin_limit` polls; a wait
// that runs out ends the kernel for that workgroup (its partner's waits then run out too), and
// out[0] counts the waits that ran out.  out[1]: ticks of the 100 MHz clock workgroup 0 spent.
__global__ void __launch_bounds__(64) signal_floor_kernel(uint32_t* words, int32_t hops, int32_t spin_limit, int32_t partner,
                                                          uint32_t* out) {
  const int me = blockIdx.x == 0 ? 0 : (static_cast<int>(blockIdx.x) == partner ? 1 : -1);
  if (me < 0 || threadIdx.x != 0) return;
  uint32_t* mine = words + (me == 0 ? 0 : 32);    // (128 bytes apart: a line each)
  uint32_t* theirs = words + (me == 0 ? 32 : 0);
  const uint64_t t0 = wall_clock64();
  for (int32_t k = 1; k <= hops; ++k) {
    if (me == 0) __hip_atomic_store(mine, static_cast<uint32_t>(k), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    bool seen = false;
    for (int32_t spin = 0; spin < spin_limit; ++spin) {
      if (__hip_atomic_load(theirs, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) >= static_cast<uint32_t>(k)) {
        seen = true;
        break;
      }
    }
    if (!seen) {
      atomicAdd(out, 1u);
      break;
    }
    if (me == 1) __hip_atomic_store(mine, static_cast<uint32_t>(k), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (me == 0) out[1] = static_cast<uint32_t>(wall_clock64() - t0);
}

}  // namespace ets

namespace {

thread_local std::string g_hook_error;

ets_status hook_fail(ets_status code, const char* msg) {
  g_hook_error = msg;
  return code;
}

#define ETS_HOOK_HIP(call)                                                        \
  do {                                                                            \
    hipError_t e_ = (call);                                                       \
    if (e_ != hipSuccess) return hook_fail(ETS_INTERNAL, hipGetErrorString(e_));  \
  } while (0)

}  // namespace

extern "C" {

ets_status ets_test_expf(const float* d_x, float* d_y, int64_t n, void* hip_stream) {
  if (!d_x || !d_y || n < 0) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_expf: bad arguments");
  if (n == 0) return ETS_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(ets::expf_exact_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(hip_stream), d_x, d_y, n);
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_seq_sum(const float* d_a, int32_t n, float s0, float threshold, float* d_sum, int32_t* d_stop,
                            void* hip_stream) {
  if (!d_a || !d_sum || !d_stop || n < 0) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_seq_sum: bad arguments");
  hipLaunchKernelGGL(ets::seq_sum_kernel, dim3(1), dim3(ets::kBlock), 0, static_cast<hipStream_t>(hip_stream), d_a, n,
                     s0, threshold, d_sum, d_stop);
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_empty_launch(void* hip_stream) {
  hipLaunchKernelGGL(ets::empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(hip_stream));
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_read_floor(const void* d_data, int64_t bytes, int32_t workgroups, uint32_t* d_out, void* hip_stream) {
  if (!d_data || !d_out || bytes < 16 || workgroups < 1 || reinterpret_cast<uintptr_t>(d_data) % 16 != 0)
    return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_read_floor: bad arguments");
  hipLaunchKernelGGL(ets::read_floor_kernel, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                     static_cast<const uint4*>(d_data), bytes / 16, d_out);
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_copy_probe(const void* d_src, void* d_dst, int64_t bytes, void* hip_stream) {
  if (!d_src || !d_dst || bytes < 16 || reinterpret_cast<uintptr_t>(d_src) % 16 != 0 || reinterpret_cast<uintptr_t>(d_dst) % 16 != 0)
    return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_copy_probe: bad arguments");
  hipLaunchKernelGGL(ets::copy_probe_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(hip_stream),
                     static_cast<const uint4*>(d_src), static_cast<uint4*>(d_dst), bytes / 16);
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_signal_floor(uint32_t* d_words, int32_t hops, int32_t spin_limit, int32_t partner, uint32_t* d_out,
                                 void* hip_stream) {
  if (!d_words || !d_out || hops < 1 || spin_limit < 1 || partner < 1 || partner > 15)
    return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_signal_floor: bad arguments");
  hipLaunchKernelGGL(ets::signal_floor_kernel, dim3(16), dim3(64), 0, static_cast<hipStream_t>(hip_stream), d_words, hops,
                     spin_limit, partner, d_out);
  ETS_HOOK_HIP(hipGetLastError());
  return ETS_OK;
}

ets_status ets_test_split_timers(ets_sampler* s, uint64_t* out, int32_t rows) {
  if (!s || !out || rows < 0 || rows > s->max_batch) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_split_timers: bad arguments");
  if (!s->d_split || !s->split.timers)
    return hook_fail(ETS_INVALID_STATE,
                     "ets_test_split_timers: needs a library built with -DETS_PHASE_CLOCKS=1 and ETS_SPLIT_TIMERS set "
                     "before the handle's first stochastic call");
  int prev = -1;
  const bool switched = hipGetDevice(&prev) == hipSuccess && prev != s->device && hipSetDevice(s->device) == hipSuccess;
  const hipError_t e = hipMemcpy(out, s->split.timers, sizeof(uint64_t) * 12 * rows, hipMemcpyDeviceToHost);
  if (switched) (void)hipSetDevice(prev);
  if (e != hipSuccess) return hook_fail(ETS_INTERNAL, hipGetErrorString(e));
  return ETS_OK;
}

ets_status ets_test_handle_buffers(const ets_sampler* s, int32_t* out) {
  if (!s || !out) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_handle_buffers: null pointer");
  out[0] = s->d_scratch != nullptr;
  out[1] = s->d_split != nullptr;
  out[2] = s->d_phist != nullptr;
  out[3] = s->d_stage != nullptr;
  return ETS_OK;
}

ets_status ets_test_fused_launch_number(ets_sampler* s, int32_t mark_unfinished, uint32_t* out) {
  if (!s || !out) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_fused_launch_number: null pointer");
  if (!s->d_split) return hook_fail(ETS_INVALID_STATE, "ets_test_fused_launch_number: the handle has not sampled several workgroups a row yet");
  int prev = -1;
  const bool switched = hipGetDevice(&prev) == hipSuccess && prev != s->device && hipSetDevice(s->device) == hipSuccess;
  const hipError_t e = hipMemcpy(out, s->split.arrive, sizeof(uint32_t), hipMemcpyDeviceToHost);
  if (switched) (void)hipSetDevice(prev);
  if (e != hipSuccess) return hook_fail(ETS_INTERNAL, hipGetErrorString(e));
  if (mark_unfinished) s->arrive_dirty = true;
  return ETS_OK;
}

ets_status ets_test_set_fused_launch_number(ets_sampler* s, uint32_t value) {
  if (!s) return hook_fail(ETS_INVALID_ARGUMENT, "ets_test_set_fused_launch_number: null pointer");
  if (!s->d_split) return hook_fail(ETS_INVALID_STATE, "ets_test_set_fused_launch_number: the handle has not sampled several workgroups a row yet");
  int prev = -1;
  const bool switched = hipGetDevice(&prev) == hipSuccess && prev != s->device && hipSetDevice(s->device) == hipSuccess;
  const hipError_t e = hipMemcpy(s->split.arrive, &value, sizeof(uint32_t), hipMemcpyHostToDevice);
  if (switched) (void)hipSetDevice(prev);
  if (e != hipSuccess) return hook_fail(ETS_INTERNAL, hipGetErrorString(e));
  return ETS_OK;
}

const char* ets_test_last_error(void) { return g_hook_error.c_str(); }

}  // extern "C"
