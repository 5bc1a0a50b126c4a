/*
 * C++ drop-in for ExecuTorch's `extension/llm/sampler/sampler.h` and `util.h`, implemented over
 * the C ABI in et_sampler.h (the MI355X HIP sampler).  Same namespace, class name, constructors,
 * setters and `sample<T>` as the reference (sampler.h:37-83, aliases :89-102), so that
 * `extension/llm/runner/text_decoder_runner.h` compiles against it unchanged; link with
 * libet_sampler.so.
 *
 * Differences from the reference, all documented in et_sampler.h: arithmetic is fp32 on the
 * converted row for every T; exactly tied probabilities are ordered by token index; the caller's
 * logits buffer is not overwritten with probabilities.  `sample()` cannot report errors in the
 * reference; here it returns -1 and `last_status()` / `last_error()` say why.
 */
#pragma once

#include <cstdint>
#include <type_traits>
#include <utility>

#include "../et_sampler.h"

namespace executorch {
namespace extension {
namespace llm {

inline constexpr auto kTopp = 0.9f;  // sampler.h:29

template <typename T>
struct ProbIndex {  // sampler.h:31-35 (kept for source compatibility; unused by this implementation)
  T prob;
  int32_t index;
};

namespace detail {

// Maps a logits element type to its executorch ScalarType code.  float and uint16_t are known
// here; 2-byte types that identify themselves (ExecuTorch's Half / BFloat16 are recognised by
// name through the traits below) can be added by specialising EtsDtype.
template <typename T, typename = void>
struct EtsDtype;

template <>
struct EtsDtype<float> {
  static constexpr int32_t value = ETS_DTYPE_FLOAT;
};
template <>
struct EtsDtype<uint16_t> {
  static constexpr int32_t value = ETS_DTYPE_UINT16;
};

}  // namespace detail

/// Minimal stand-ins for the 16-bit element types, for callers that do not include the
/// ExecuTorch headers: plain 16-bit storage, bit-compatible with c10::Half / c10::BFloat16.
struct HalfBits {
  uint16_t x;
};
struct BFloat16Bits {
  uint16_t x;
};

namespace detail {
template <>
struct EtsDtype<HalfBits> {
  static constexpr int32_t value = ETS_DTYPE_HALF;
};
template <>
struct EtsDtype<BFloat16Bits> {
  static constexpr int32_t value = ETS_DTYPE_BFLOAT16;
};
}  // namespace detail

class Sampler {
 public:
  /// sampler.cpp:173-181
  Sampler(int32_t vocab_size, float temperature, float topp, unsigned long long rng_seed, int32_t max_batch = 1) {
    status_ = ets_sampler_create(vocab_size, temperature, topp, rng_seed, max_batch, &h_);
  }
  /// sampler.cpp:183-187: topp = kTopp, seed = time(nullptr)
  Sampler(int32_t vocab_size, float temperature) { status_ = ets_sampler_create_default(vocab_size, temperature, 1, &h_); }

  ~Sampler() { ets_sampler_destroy(h_); }
  Sampler(const Sampler&) = delete;
  Sampler& operator=(const Sampler&) = delete;
  Sampler(Sampler&& o) noexcept : h_(o.h_), status_(o.status_) { o.h_ = nullptr; }
  Sampler& operator=(Sampler&& o) noexcept {
    if (this != &o) {
      ets_sampler_destroy(h_);
      h_ = o.h_;
      status_ = o.status_;
      o.h_ = nullptr;
    }
    return *this;
  }

  /// sampler.h:48-53
  void set_temperature(float temperature) { status_ = ets_sampler_set_temperature(h_, temperature); }
  /// sampler.h:58-60
  void set_topk(int32_t topk) { status_ = ets_sampler_set_topk(h_, topk); }
  /// no counterpart: the reference fixes top-p at construction
  void set_topp(float topp) { status_ = ets_sampler_set_topp(h_, topp); }

  /// sampler.cpp:222-251.  `logits` points to vocab_size elements in host memory.
  template <typename T>
  int32_t sample(T* logits) {
    int32_t token = -1;
    status_ = ets_sampler_sample(h_, logits, detail::EtsDtype<std::remove_cv_t<T>>::value, &token);
    return status_ == ETS_OK ? token : -1;
  }

  /// Same with the element type given at run time (an executorch ScalarType value).
  int32_t sample(const void* logits, int32_t dtype) {
    int32_t token = -1;
    status_ = ets_sampler_sample(h_, logits, dtype, &token);
    return status_ == ETS_OK ? token : -1;
  }

  /// Batched entry over device-resident logits [batch, vocab] (no counterpart in the reference):
  /// `d_logits` and `d_tokens` are device pointers, `hip_stream` a hipStream_t (or nullptr).
  ets_status sample_batch(const void* d_logits, int32_t dtype, int32_t batch, int64_t row_stride_elems,
                          int32_t* d_tokens, void* hip_stream = nullptr) {
    status_ = ets_sampler_sample_batch(h_, d_logits, dtype, batch, row_stride_elems, d_tokens, hip_stream);
    return status_;
  }

  /// The same with one SamplingConfig per row (extension/llm/runner/llm_session.h:29-34;
  /// ets_sampling_config has its fields): `configs` is a host array of `batch` entries.
  ets_status sample_batch(const void* d_logits, int32_t dtype, int32_t batch, int64_t row_stride_elems,
                          const ets_sampling_config* configs, int32_t* d_tokens, void* hip_stream = nullptr) {
    status_ = ets_sampler_sample_batch_configs(h_, d_logits, dtype, batch, row_stride_elems, configs, d_tokens,
                                               nullptr, hip_stream);
    return status_;
  }

  ets_status last_status() const { return status_; }
  const char* last_error() const { return ets_sampler_last_error(h_); }
  ets_sampler* handle() const { return h_; }

 private:
  ets_sampler* h_ = nullptr;
  ets_status status_ = ETS_OK;
};

/// util.h:25-55.  Works with any tensor type that offers scalar_type() (convertible to the
/// executorch ScalarType code), dim(), size(d) and const_data_ptr() -- executorch::aten::Tensor
/// does.  Rank 3 samples the last position of batch 0; an unsupported dtype makes the reference
/// abort, here the call returns -1 with ETS_INVALID_ARGUMENT in sampler.last_status().
template <typename Tensor>
inline int32_t sample_from_logits(const Tensor& logits_tensor, Sampler& sampler) {
  const int32_t rank = static_cast<int32_t>(logits_tensor.dim());
  int64_t sizes[8] = {0};
  if (rank < 1 || rank > 8) return -1;
  for (int32_t d = 0; d < rank; ++d) sizes[d] = static_cast<int64_t>(logits_tensor.size(d));
  int32_t token = -1;
  const ets_status st = ets_sample_from_logits(sampler.handle(), logits_tensor.const_data_ptr(),
                                               static_cast<int32_t>(logits_tensor.scalar_type()), rank, sizes, &token);
  return st == ETS_OK ? token : -1;
}

/// The batched adapter (no counterpart: util.h:48-51 reads batch 0 of a host tensor): `logits_tensor`
/// describes a DEVICE-resident [batch, vocab] or [batch, seq, vocab] tensor (its const_data_ptr() is
/// a device pointer, as a delegate that skips the copy to the host leaves it); one token per batch
/// entry is written to the device array `d_tokens`, asynchronously on `hip_stream`.
template <typename Tensor>
inline ets_status sample_from_logits_batch(const Tensor& logits_tensor, Sampler& sampler, int32_t* d_tokens,
                                           void* hip_stream = nullptr) {
  const int32_t rank = static_cast<int32_t>(logits_tensor.dim());
  int64_t sizes[3] = {0, 0, 0};
  if (rank != 2 && rank != 3) return ETS_INVALID_ARGUMENT;
  for (int32_t d = 0; d < rank; ++d) sizes[d] = static_cast<int64_t>(logits_tensor.size(d));
  return ets_sample_from_logits_batch(sampler.handle(), logits_tensor.const_data_ptr(),
                                      static_cast<int32_t>(logits_tensor.scalar_type()), rank, sizes, d_tokens, hip_stream);
}

/// util.h:64-71
template <typename Tensor>
inline int32_t logits_to_token(const Tensor& logits_tensor, const float temperature = 0.0f) {
  const int32_t rank = static_cast<int32_t>(logits_tensor.dim());
  int64_t sizes[8] = {0};
  if (rank < 1 || rank > 8) return -1;
  for (int32_t d = 0; d < rank; ++d) sizes[d] = static_cast<int64_t>(logits_tensor.size(d));
  int32_t token = -1;
  const ets_status st = ets_logits_to_token(logits_tensor.const_data_ptr(), static_cast<int32_t>(logits_tensor.scalar_type()),
                                            rank, sizes, temperature, &token);
  return st == ETS_OK ? token : -1;
}

}  // namespace llm
}  // namespace extension
}  // namespace executorch

namespace torch {
namespace executor {
// the reference's deprecated aliases (sampler.h:89-96)
using ::executorch::extension::llm::ProbIndex;
using ::executorch::extension::llm::Sampler;
}  // namespace executor
}  // namespace torch

namespace executorch::llm {
using ::executorch::extension::llm::kTopp;  // sampler.h:98-102
}  // namespace executorch::llm
