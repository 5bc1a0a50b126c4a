// A decode loop with device-resident logits, shaped like the reference's generation loop
// (extension/llm/runner/text_token_generator.h:133-148: step -> apply_logit_processors ->
// logits_to_token -> the token goes back into the next step), written against the C ABI only:
//
//   "model step"   a fresh [batch, vocab] matrix of logits appears in DEVICE memory (a copy from a
//                  ring of synthetic matrices; a delegate that skips the copy of its outputs to the
//                  host leaves them like this, backends/cuda/runtime/cuda_backend.cpp:80-81)
//   processors     ets_logit_chain_process: repetition penalty over the tokens generated so far
//                  (a device-resident history) and a mask, in place, same stream
//   sampling       ets_sample_from_logits_batch on the same stream, tokens to a device array
//   feedback       the tokens are appended to the history on the device; 4 bytes per row go to the
//                  host (what a runner needs to detokenise and test for end of sequence)
//
// Prints the tokens of every step (the test compares them with the CPU oracle run over the same
// synthetic logits) and the sampler's device time per call from ets_sampler_get_stats().
//
//   decode_loop <vocab> <batch> <steps> <dtype 6|5|15> <temperature> <topp> <seed> <ring>
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <et_logit_processor.h>
#include <et_sampler.h>

#define HIP_OK(call)                                                                       \
  do {                                                                                     \
    hipError_t e_ = (call);                                                                \
    if (e_ != hipSuccess) {                                                                \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));               \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)
#define ETS_OK_OR_DIE(call, handle)                                                        \
  do {                                                                                     \
    ets_status s_ = (call);                                                                \
    if (s_ != ETS_OK) {                                                                    \
      std::fprintf(stderr, "%s failed: 0x%x %s\n", #call, s_, ets_sampler_last_error(handle)); \
      return 3;                                                                            \
    }                                                                                      \
  } while (0)

static uint64_t mix(uint64_t z) {  // splitmix64 finaliser
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// Logit (r, b, i): a multiple of 1/16 in [-8, 8), plus 6 at three positions per row -- exactly
// representable in bf16, fp16 and fp32, so every element type holds the same values.
static float logit_value(uint64_t seed, uint64_t row_id, uint64_t vocab, uint64_t i) {
  return (static_cast<int>(mix(seed + row_id * vocab + i) >> 56) - 128) / 16.0f;
}

static uint16_t to_bf16(float f) {  // exact for these values
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return static_cast<uint16_t>(u >> 16);
}

static uint16_t to_fp16(float f) {  // exact for multiples of 1/16 below 16 in magnitude
  if (f == 0.0f) return 0;
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const int exp = static_cast<int>((u >> 23) & 0xff) - 127 + 15;
  return static_cast<uint16_t>(sign | (static_cast<uint32_t>(exp) << 10) | ((u & 0x7fffffu) >> 13));
}

int main(int argc, char** argv) {
  if (argc != 9) {
    std::fprintf(stderr, "usage: decode_loop vocab batch steps dtype temperature topp seed ring\n");
    return 1;
  }
  const int64_t V = std::atoll(argv[1]), B = std::atoll(argv[2]);
  const int steps = std::atoi(argv[3]), dtype = std::atoi(argv[4]);
  const float temperature = static_cast<float>(std::atof(argv[5])), topp = static_cast<float>(std::atof(argv[6]));
  const uint64_t seed = std::strtoull(argv[7], nullptr, 10);
  const int ring = std::atoi(argv[8]);
  const size_t esz = dtype == ETS_DTYPE_FLOAT ? 4 : 2;

  // ---- the ring of synthetic logit matrices, in device memory
  std::vector<void*> d_ring(ring, nullptr);
  {
    std::vector<float> host(static_cast<size_t>(B * V));
    std::vector<uint16_t> host16(dtype == ETS_DTYPE_FLOAT ? 0 : host.size());
    for (int r = 0; r < ring; ++r) {
      for (int64_t b = 0; b < B; ++b) {
        const uint64_t row_id = static_cast<uint64_t>(r) * B + b;
        float* row = host.data() + b * V;
        for (int64_t i = 0; i < V; ++i) row[i] = logit_value(seed, row_id, V, i);
        for (int j = 0; j < 3; ++j) row[mix(seed + 0xABCDEFull + row_id * 3 + j) % V] += 6.0f;
      }
      const void* src = host.data();
      if (dtype != ETS_DTYPE_FLOAT) {
        for (size_t k = 0; k < host.size(); ++k) host16[k] = dtype == ETS_DTYPE_BFLOAT16 ? to_bf16(host[k]) : to_fp16(host[k]);
        src = host16.data();
      }
      HIP_OK(hipMalloc(&d_ring[r], host.size() * esz));
      HIP_OK(hipMemcpy(d_ring[r], src, host.size() * esz, hipMemcpyHostToDevice));
    }
  }
  void* d_logits = nullptr;  // what the "model" writes every step
  int32_t *d_tokens = nullptr, *d_history = nullptr, *d_len = nullptr, *h_tokens = nullptr;
  HIP_OK(hipMalloc(&d_logits, static_cast<size_t>(B * V) * esz));
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_tokens), sizeof(int32_t) * B));
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_history), sizeof(int32_t) * B * steps));
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&d_len), sizeof(int32_t) * B));
  HIP_OK(hipMemset(d_history, 0, sizeof(int32_t) * B * steps));
  HIP_OK(hipMemset(d_len, 0, sizeof(int32_t) * B));
  HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&h_tokens), sizeof(int32_t) * B * steps, hipHostMallocDefault));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // ---- the sampler the runner owns (text_decoder_runner.h:107) and its processors
  //      (text_token_generator.h:44-48)
  ets_sampler* sampler = nullptr;
  ETS_OK_OR_DIE(ets_sampler_create(static_cast<int32_t>(V), temperature, topp, seed, static_cast<int32_t>(B), &sampler), nullptr);
  ETS_OK_OR_DIE(ets_sampler_set_timing(sampler, 1), sampler);
  ets_logit_chain* chain = nullptr;
  ETS_OK_OR_DIE(ets_logit_chain_create(&chain), nullptr);
  ETS_OK_OR_DIE(ets_logit_chain_add_repetition_penalty(chain, 1.25f, d_history, steps, d_len), nullptr);
  int32_t banned[16];
  for (int k = 0; k < 16; ++k) banned[k] = 100 + k;
  ETS_OK_OR_DIE(ets_logit_chain_add_mask(chain, banned, 16), nullptr);

  const int64_t sizes[2] = {B, V};
  for (int t = 0; t < steps; ++t) {
    // the model step: fresh logits in device memory
    HIP_OK(hipMemcpyAsync(d_logits, d_ring[t % ring], static_cast<size_t>(B * V) * esz, hipMemcpyDeviceToDevice, stream));
    ETS_OK_OR_DIE(ets_logit_chain_process(chain, d_logits, dtype, 2, sizes, stream), nullptr);
    ETS_OK_OR_DIE(ets_sample_from_logits_batch(sampler, d_logits, dtype, 2, sizes, d_tokens, stream), sampler);
    // feedback on the device: history[b][t] = token[b], length = t + 1
    HIP_OK(hipMemcpy2DAsync(d_history + t, sizeof(int32_t) * steps, d_tokens, sizeof(int32_t), sizeof(int32_t), B,
                            hipMemcpyDeviceToDevice, stream));
    HIP_OK(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(d_len), t + 1, B, stream));
    // 4 bytes per row to the host
    HIP_OK(hipMemcpyAsync(h_tokens + static_cast<size_t>(t) * B, d_tokens, sizeof(int32_t) * B, hipMemcpyDeviceToHost, stream));
  }
  HIP_OK(hipStreamSynchronize(stream));
  ets_sampler_stats stats;
  ETS_OK_OR_DIE(ets_sampler_get_stats(sampler, &stats), sampler);
  for (int t = 0; t < steps; ++t) {
    std::printf("tokens %d:", t);
    for (int64_t b = 0; b < B; ++b) std::printf(" %d", h_tokens[static_cast<size_t>(t) * B + b]);
    std::printf("\n");
  }
  std::printf("stats calls %llu rows %llu us_per_call %.3f us_per_token %.3f\n", static_cast<unsigned long long>(stats.calls),
              static_cast<unsigned long long>(stats.rows), stats.aggregate_sampling_time_us / static_cast<double>(stats.calls),
              stats.aggregate_sampling_time_us / static_cast<double>(stats.rows));
  ets_logit_chain_destroy(chain);
  ets_sampler_destroy(sampler);
  return 0;
}
