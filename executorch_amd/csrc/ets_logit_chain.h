// Device-side logit processor chain: kernel and host side of include/et_logit_processor.h.
// Included at the end of et_sampler.hip (one translation unit, one shared library).
//
// The reference runs its processors one after the other over a host tensor
// (text_token_generator.h:59-66).  Every processor here is elementwise -- it rewrites some or all
// entries of a row, each from its own old value -- so the order only matters per entry: the row is
// cut into tiles, a workgroup owns a tile and applies the whole chain to it in registration order,
// with a workgroup barrier between processors.  One launch for any chain length.
#pragma once

#include <vector>

#include "../../include/et_logit_processor.h"

namespace ets {

constexpr int kChainBlock = 256;
constexpr int kChainTile = 8192;  // entries per workgroup when some processor touches whole rows

constexpr int32_t kOpBias = 0, kOpScale = 1, kOpMask = 2, kOpTokenBias = 3, kOpRepetition = 4;

struct ChainOp {
  int32_t kind;
  float value;            // bias / factor / penalty
  int32_t count;          // mask, token bias: list length
  int32_t serial;         // token bias: an id occurs twice, apply the list in order by one lane
  const int32_t* ids;     // mask, token bias: device list; repetition: device history [batch, stride]
  const float* values;    // token bias: device list
  int64_t stride;         // repetition: entries between rows of the history
  const int32_t* lengths; // repetition: device [batch]
};

template <int DT>
__device__ __forceinline__ void store_elem(void* row, int64_t i, float v);
template <>
__device__ __forceinline__ void store_elem<kDtypeFloat>(void* row, int64_t i, float v) {
  static_cast<float*>(row)[i] = v;
}
template <>
__device__ __forceinline__ void store_elem<kDtypeHalf>(void* row, int64_t i, float v) {
  // The fp32 result is rounded to fp32 first and to half second, as host code storing into a Half
  // tensor does; the empty asm keeps the compiler from merging the producing multiply or add with
  // the conversion into one mixed-precision instruction that rounds once.
  asm volatile("" : "+v"(v));
  static_cast<_Float16*>(row)[i] = static_cast<_Float16>(v);  // round to nearest even
}
template <>
__device__ __forceinline__ void store_elem<kDtypeBFloat16>(void* row, int64_t i, float v) {
  uint32_t b = __float_as_uint(v);
  if ((b & 0x7fffffffu) > 0x7f800000u) {
    b = 0x7fc0u;  // NaN
  } else {
    b = (b + 0x7fffu + ((b >> 16) & 1u)) >> 16;  // round to nearest even
  }
  static_cast<uint16_t*>(row)[i] = static_cast<uint16_t>(b);
}

// grid = (tiles, rows).  `base` is the tensor's first element; row r's entries start at element
// r * row_pitch + row_offset (row_offset selects the last sequence position of a rank-3 tensor).
template <int DT>
__global__ void __launch_bounds__(kChainBlock)
logit_chain_kernel(void* base, int64_t row_pitch, int64_t row_offset, int32_t vocab, int32_t tile, const ChainOp* ops,
                   int32_t n_ops) {
  extern __shared__ uint32_t seen[];  // repetition penalty: one bit per entry of the tile
  const int tid = threadIdx.x;
  const int row = blockIdx.y;
  const int t0 = blockIdx.x * tile;
  const int t1 = min(vocab, t0 + tile);
  char* data = static_cast<char*>(base) + (static_cast<int64_t>(row) * row_pitch + row_offset) * ElemSize<DT>::value;
  const float kInf = __uint_as_float(0x7f800000u);
  for (int k = 0; k < n_ops; ++k) {
    const ChainOp op = ops[k];
    if (op.kind == kOpBias) {
      for (int i = t0 + tid; i < t1; i += kChainBlock) store_elem<DT>(data, i, load_elem<DT>(data, i) + op.value);
    } else if (op.kind == kOpScale) {
      for (int i = t0 + tid; i < t1; i += kChainBlock) store_elem<DT>(data, i, load_elem<DT>(data, i) * op.value);
    } else if (op.kind == kOpMask) {
      for (int j = tid; j < op.count; j += kChainBlock) {
        const int id = op.ids[j];
        if (id >= t0 && id < t1) store_elem<DT>(data, id, -kInf);
      }
    } else if (op.kind == kOpTokenBias) {
      if (op.serial) {
        if (tid == 0) {
          for (int j = 0; j < op.count; ++j) {
            const int id = op.ids[j];
            if (id >= t0 && id < t1) store_elem<DT>(data, id, load_elem<DT>(data, id) + op.values[j]);
          }
        }
      } else {
        for (int j = tid; j < op.count; j += kChainBlock) {
          const int id = op.ids[j];
          if (id >= t0 && id < t1) store_elem<DT>(data, id, load_elem<DT>(data, id) + op.values[j]);
        }
      }
    } else if (op.kind == kOpRepetition) {
      const int words = (t1 - t0 + 31) >> 5;
      for (int w = tid; w < words; w += kChainBlock) seen[w] = 0u;
      __syncthreads();
      const int32_t* history = op.ids + static_cast<int64_t>(row) * op.stride;
      int len = op.lengths[row];
      if (len > op.stride) len = static_cast<int>(op.stride);
      for (int j = tid; j < len; j += kChainBlock) {
        const int id = history[j];
        if (id >= t0 && id < t1) {
          const uint32_t bit = 1u << ((id - t0) & 31);
          const uint32_t old = atomicOr(&seen[(id - t0) >> 5], bit);
          if (!(old & bit)) {  // first occurrence of this token: the only lane that touches its logit
            const float x = load_elem<DT>(data, id);
            store_elem<DT>(data, id, x < 0.0f ? x * op.value : x / op.value);
          }
        }
      }
    }
    __syncthreads();  // the next processor sees this one's stores (same workgroup, same tile)
  }
}

}  // namespace ets

struct ets_logit_chain {
  std::vector<ets::ChainOp> ops;
  std::vector<void*> owned;       // device copies of the lists
  ets::ChainOp* d_ops = nullptr;  // device copy of `ops`
  int32_t d_ops_capacity = 0;
  int device = 0;
  bool whole_rows = false;        // some processor touches every entry
  bool repetition = false;
  std::string last_error;
};

namespace {

ets_status chain_fail(ets_logit_chain* c, ets_status code, const std::string& msg) {
  if (c) {
    c->last_error = msg;
  } else {
    g_thread_error = msg;
  }
  return code;
}

#define ETS_CHAIN_HIP(c, call)                                                                          \
  do {                                                                                                  \
    hipError_t e_ = (call);                                                                             \
    if (e_ != hipSuccess)                                                                               \
      return chain_fail(c, e_ == hipErrorOutOfMemory ? ETS_MEMORY_ALLOCATION_FAILED : ETS_INTERNAL,     \
                        std::string(#call) + ": " + hipGetErrorString(e_));                             \
  } while (0)

// Appends `op` and refreshes the device copy of the list.
ets_status chain_push(ets_logit_chain* c, const ets::ChainOp& op) {
  c->ops.push_back(op);
  const int32_t n = static_cast<int32_t>(c->ops.size());
  if (n > c->d_ops_capacity) {
    const int32_t cap = n + 8;
    ets::ChainOp* fresh = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&fresh), sizeof(ets::ChainOp) * cap);
    if (e != hipSuccess) {
      c->ops.pop_back();
      return chain_fail(c, ETS_MEMORY_ALLOCATION_FAILED, std::string("hipMalloc(chain): ") + hipGetErrorString(e));
    }
    // the old list may still be read by a launch in flight: free it only after the device is idle
    if (c->d_ops) {
      (void)hipDeviceSynchronize();
      (void)hipFree(c->d_ops);
    }
    c->d_ops = fresh;
    c->d_ops_capacity = cap;
  } else {
    (void)hipDeviceSynchronize();  // a launch in flight reads the list that is about to change
  }
  hipError_t e = hipMemcpy(c->d_ops, c->ops.data(), sizeof(ets::ChainOp) * n, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    c->ops.pop_back();
    return chain_fail(c, ETS_INTERNAL, std::string("hipMemcpy(chain): ") + hipGetErrorString(e));
  }
  return ETS_OK;
}

template <typename T>
ets_status chain_upload(ets_logit_chain* c, const T* host, int32_t count, const T** device) {
  *device = nullptr;
  if (count == 0) return ETS_OK;
  void* d = nullptr;
  ETS_CHAIN_HIP(c, hipMalloc(&d, sizeof(T) * count));
  hipError_t e = hipMemcpy(d, host, sizeof(T) * count, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(d);
    return chain_fail(c, ETS_INTERNAL, std::string("hipMemcpy(list): ") + hipGetErrorString(e));
  }
  c->owned.push_back(d);
  *device = static_cast<const T*>(d);
  return ETS_OK;
}

template <int DT>
ets_status chain_launch(ets_logit_chain* c, void* d_logits, int64_t row_pitch, int64_t row_offset, int32_t vocab,
                        int32_t rows, hipStream_t stream, int32_t n_ops = -1) {
  // (n_ops: only the chain's first processors; the rest is left to the caller)
  if (n_ops < 0) n_ops = static_cast<int32_t>(c->ops.size());
  bool whole_rows = false;
  for (int32_t k = 0; k < n_ops; ++k) whole_rows = whole_rows || c->ops[k].kind == ets::kOpBias || c->ops[k].kind == ets::kOpScale;
  // whole-row processors want many workgroups per row; lists alone are cheapest with one
  const int32_t tile = whole_rows ? ets::kChainTile : vocab;
  const int32_t tiles = (vocab + tile - 1) / tile;
  const size_t lds = c->repetition ? static_cast<size_t>((tile + 31) / 32) * sizeof(uint32_t) : 0;
  if (lds > 64 * 1024) {
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
      attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(&ets::logit_chain_kernel<DT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
    });
    if (attr_err != hipSuccess) {
      return chain_fail(c, ETS_INTERNAL, std::string("hipFuncSetAttribute: ") + hipGetErrorString(attr_err));
    }
  }
  hipLaunchKernelGGL((ets::logit_chain_kernel<DT>), dim3(tiles, rows), dim3(ets::kChainBlock), lds, stream, d_logits,
                     row_pitch, row_offset, vocab, tile, c->d_ops, n_ops);
  ETS_CHAIN_HIP(c, hipGetLastError());
  return ETS_OK;
}

}  // namespace

extern "C" {

ets_status ets_logit_chain_create(ets_logit_chain** out) {
  if (!out) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_create: out is null");
  *out = nullptr;
  ets_logit_chain* c = new (std::nothrow) ets_logit_chain();
  if (!c) return chain_fail(nullptr, ETS_MEMORY_ALLOCATION_FAILED, "ets_logit_chain_create: out of host memory");
  hipError_t e = hipGetDevice(&c->device);
  if (e != hipSuccess) {
    delete c;
    return chain_fail(nullptr, ETS_INTERNAL, std::string("hipGetDevice: ") + hipGetErrorString(e));
  }
  *out = c;
  return ETS_OK;
}

ets_status ets_logit_chain_destroy(ets_logit_chain* c) {
  if (!c) return ETS_OK;
  {
    DeviceGuard g(c->device);
    (void)hipDeviceSynchronize();
    for (void* d : c->owned) (void)hipFree(d);
    (void)hipFree(c->d_ops);
  }
  delete c;
  return ETS_OK;
}

int32_t ets_logit_chain_size(const ets_logit_chain* c) { return c ? static_cast<int32_t>(c->ops.size()) : 0; }

ets_status ets_logit_chain_add_bias(ets_logit_chain* c, float bias) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_bias: null chain");
  c->last_error.clear();
  DeviceGuard g(c->device);
  ets::ChainOp op = {ets::kOpBias, bias, 0, 0, nullptr, nullptr, 0, nullptr};
  ets_status st = chain_push(c, op);
  if (st == ETS_OK) c->whole_rows = true;
  return st;
}

ets_status ets_logit_chain_add_scale(ets_logit_chain* c, float factor) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_scale: null chain");
  c->last_error.clear();
  DeviceGuard g(c->device);
  ets::ChainOp op = {ets::kOpScale, factor, 0, 0, nullptr, nullptr, 0, nullptr};
  ets_status st = chain_push(c, op);
  if (st == ETS_OK) c->whole_rows = true;
  return st;
}

ets_status ets_logit_chain_add_mask(ets_logit_chain* c, const int32_t* tokens, int32_t count) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_mask: null chain");
  c->last_error.clear();
  if (count < 0 || (count > 0 && !tokens))
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_mask: bad list");
  DeviceGuard g(c->device);
  ets::ChainOp op = {ets::kOpMask, 0.0f, count, 0, nullptr, nullptr, 0, nullptr};
  ets_status st = chain_upload(c, tokens, count, &op.ids);
  if (st != ETS_OK) return st;
  return chain_push(c, op);
}

ets_status ets_logit_chain_add_token_bias(ets_logit_chain* c, const int32_t* tokens, const float* bias, int32_t count) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_token_bias: null chain");
  c->last_error.clear();
  if (count < 0 || (count > 0 && (!tokens || !bias)))
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_token_bias: bad list");
  DeviceGuard g(c->device);
  ets::ChainOp op = {ets::kOpTokenBias, 0.0f, count, 0, nullptr, nullptr, 0, nullptr};
  // two additions to one entry do not commute with the rounding in between: keep list order then
  std::vector<int32_t> sorted(tokens, tokens + count);
  std::sort(sorted.begin(), sorted.end());
  for (int32_t j = 1; j < count; ++j) {
    if (sorted[j] == sorted[j - 1]) op.serial = 1;
  }
  ets_status st = chain_upload(c, tokens, count, &op.ids);
  if (st != ETS_OK) return st;
  st = chain_upload(c, bias, count, &op.values);
  if (st != ETS_OK) return st;
  return chain_push(c, op);
}

ets_status ets_logit_chain_add_repetition_penalty(ets_logit_chain* c, float penalty, const int32_t* d_history,
                                                  int64_t history_stride, const int32_t* d_history_len) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_repetition_penalty: null chain");
  c->last_error.clear();
  if (!d_history || !d_history_len || history_stride < 0)
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_repetition_penalty: bad history");
  if (!(penalty > 0.0f)) return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_add_repetition_penalty: penalty must be > 0");
  DeviceGuard g(c->device);
  ets::ChainOp op = {ets::kOpRepetition, penalty, 0, 0, d_history, nullptr, history_stride, d_history_len};
  ets_status st = chain_push(c, op);
  if (st == ETS_OK) c->repetition = true;
  return st;
}

ets_status ets_logit_chain_process(ets_logit_chain* c, void* d_logits, int32_t dtype, int32_t rank, const int64_t* sizes,
                                   void* hip_stream) {
  if (!c) return chain_fail(nullptr, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: null chain");
  c->last_error.clear();
  if (!d_logits || !sizes) return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: null pointer");
  if (dtype != ETS_DTYPE_FLOAT && dtype != ETS_DTYPE_HALF && dtype != ETS_DTYPE_BFLOAT16)
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: element type must be Float, Half or BFloat16");
  if (rank != 2 && rank != 3) return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: rank must be 2 or 3");
  for (int32_t d = 0; d < rank; ++d) {
    if (sizes[d] < 0) return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: negative extent");
  }
  const int64_t rows = sizes[0];
  const int64_t vocab = sizes[rank - 1];
  const int64_t seq = rank == 3 ? sizes[1] : 1;
  if (vocab > 0x7fffffff || rows > 65535)
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: at most 65535 rows of at most 2^31 - 1 entries");
  if (c->ops.empty() || rows == 0 || vocab == 0 || seq == 0) return ETS_OK;
  if (c->repetition && vocab > 1048576)
    return chain_fail(c, ETS_INVALID_ARGUMENT, "ets_logit_chain_process: the repetition penalty needs vocab <= 1048576");
  const int64_t row_pitch = seq * vocab;
  const int64_t row_offset = (seq - 1) * vocab;  // the last sequence position
  DeviceGuard g(c->device);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  switch (dtype) {
    case ETS_DTYPE_FLOAT:
      return chain_launch<ets::kDtypeFloat>(c, d_logits, row_pitch, row_offset, static_cast<int32_t>(vocab),
                                            static_cast<int32_t>(rows), stream);
    case ETS_DTYPE_HALF:
      return chain_launch<ets::kDtypeHalf>(c, d_logits, row_pitch, row_offset, static_cast<int32_t>(vocab),
                                           static_cast<int32_t>(rows), stream);
    default:
      return chain_launch<ets::kDtypeBFloat16>(c, d_logits, row_pitch, row_offset, static_cast<int32_t>(vocab),
                                               static_cast<int32_t>(rows), stream);
  }
}

ets_status ets_sampler_sample_batch_chain(ets_sampler* s, ets_logit_chain* c, void* d_logits, int32_t dtype, int32_t batch,
                                          int64_t row_stride_elems, int32_t* d_tokens, void* hip_stream) {
  if (!s) return fail(nullptr, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: null handle");
  s->last_error.clear();
  if (!c) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: null chain");
  if (!d_logits || !d_tokens) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: null pointer");
  if (dtype != ETS_DTYPE_FLOAT && dtype != ETS_DTYPE_HALF && dtype != ETS_DTYPE_BFLOAT16)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: element type must be Float, Half or BFloat16");
  if (batch < 0 || batch > s->max_batch)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: batch exceeds the handle's max_batch");
  if (row_stride_elems < s->vocab)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: row stride smaller than vocab_size");
  if (c->device != s->device) return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: chain and sampler live on different devices");
  if (c->repetition && s->vocab > 1048576)
    return fail(s, ETS_INVALID_ARGUMENT, "ets_sampler_sample_batch_chain: the repetition penalty needs vocab <= 1048576");
  if (batch == 0) return ETS_OK;
  DeviceGuard g(s->device);
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  // The chain's last processors, as far as they are biases and factors, are applied while the
  // sampler reads the logits -- when the rows take the path that can do that (the top-p draw with
  // several workgroups per row); everything in front of them runs in place first.
  const int32_t n_ops = static_cast<int32_t>(c->ops.size());
  ets::FusedOps fused = {};
  int32_t n_front = n_ops;
  const bool can_fuse = s->inv_temperature != 0.0f && !s->wb && draw_mode(s->vocab, s->topp, s->topk) == ets::kDrawTopP &&
                        use_split(s, d_logits, row_stride_elems, dtype, ets::kDrawTopP, 0);
  if (can_fuse) {
    while (n_front > 0 && fused.n < ets::kMaxFusedOps &&
           (c->ops[n_front - 1].kind == ets::kOpBias || c->ops[n_front - 1].kind == ets::kOpScale))
      --n_front, ++fused.n;
    for (int32_t k = 0; k < fused.n; ++k) {
      fused.scale[k] = c->ops[n_front + k].kind == ets::kOpScale ? 1 : 0;
      fused.value[k] = c->ops[n_front + k].value;
    }
  }
  if (n_front > 0) {
    ets_status st = ETS_OK;
    switch (dtype) {
      case ETS_DTYPE_FLOAT:
        st = chain_launch<ets::kDtypeFloat>(c, d_logits, row_stride_elems, 0, s->vocab, batch, stream, n_front);
        break;
      case ETS_DTYPE_HALF:
        st = chain_launch<ets::kDtypeHalf>(c, d_logits, row_stride_elems, 0, s->vocab, batch, stream, n_front);
        break;
      default:
        st = chain_launch<ets::kDtypeBFloat16>(c, d_logits, row_stride_elems, 0, s->vocab, batch, stream, n_front);
        break;
    }
    if (st != ETS_OK) return fail(s, st, std::string("ets_sampler_sample_batch_chain: ") + c->last_error);
  }
  int slot = -1;
  ets_status st = timing_begin(s, stream, batch, &slot);
  if (st != ETS_OK) return st;
  st = sample_device(s, d_logits, dtype, batch, row_stride_elems, d_tokens, nullptr, nullptr, stream,
                     fused.n > 0 ? &fused : nullptr);
  if (st != ETS_OK) return st;
  return timing_end(s, stream, slot);
}

const char* ets_logit_chain_last_error(const ets_logit_chain* c) {
  return c ? c->last_error.c_str() : g_thread_error.c_str();
}

}  // extern "C"
