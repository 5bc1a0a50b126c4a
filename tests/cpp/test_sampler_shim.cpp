// The reference's sampler tests (extension/llm/sampler/test/test_sampler.cpp:19-154 and the
// logits_to_token cases of extension/llm/runner/test/test_text_decoder_runner.cpp:83-140)
// written against the drop-in C++ class in include/executorch_amd/sampler.h.  Plain asserts, no
// gtest (not available here).  Needs a GPU to run; tests/test_cpp_shim.py builds it everywhere
// and runs it on the GPU box.
#include <executorch_amd/sampler.h>

#include <cstdio>
#include <cstdlib>
#include <random>
#include <set>
#include <vector>

using ::executorch::extension::llm::Sampler;

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      std::exit(1);                                                        \
    }                                                                      \
  } while (0)

// A tensor-like type with the four accessors the adapters use.
struct FakeTensor {
  std::vector<float> data;
  std::vector<int64_t> shape;
  int32_t scalar_type() const { return ETS_DTYPE_FLOAT; }
  int64_t dim() const { return static_cast<int64_t>(shape.size()); }
  int64_t size(int64_t d) const { return shape[d]; }
  const void* const_data_ptr() const { return data.data(); }
};

static uint16_t half_bits(float f) {  // round-to-nearest-even, normal range only (inputs are in [2^-14, 2))
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  const uint32_t exp = ((u >> 23) & 0xff) - 112;  // rebias 127 -> 15
  uint32_t man = u & 0x7fffff;
  uint32_t h = (exp << 10) | (man >> 13);
  const uint32_t rem = man & 0x1fff;
  if (rem > 0x1000 || (rem == 0x1000 && (h & 1))) ++h;
  return static_cast<uint16_t>(h);
}

int main() {
  std::mt19937 rng(0);
  std::uniform_real_distribution<float> uni(0.001f, 0.999f);
  {  // TestArgMax
    Sampler sampler{32000, 0.0f, 0.9f, 0};
    CHECK(sampler.last_status() == ETS_OK);
    std::vector<float> x(32000);
    for (auto& v : x) v = uni(rng);
    x[396] = 1.0f;
    CHECK(sampler.sample(x.data()) == 396);
  }
  {  // TestArgMaxWithFP16
    Sampler sampler{32000, 0.0f, 0.9f, 0};
    std::vector<executorch::extension::llm::HalfBits> x(32000);
    for (auto& v : x) v.x = half_bits(uni(rng));
    x[396].x = half_bits(1.0f);
    CHECK(sampler.sample(x.data()) == 396);
  }
  {  // TestTopKRestrictsToCandidates
    Sampler sampler{100, 1.0f, 0.0f, 42};
    sampler.set_topk(3);
    std::vector<float> x(100, -10.0f);
    x[7] = 5.0f, x[13] = 4.5f, x[42] = 4.0f;
    const std::set<int32_t> allowed = {7, 13, 42};
    for (int t = 0; t < 50; ++t) CHECK(allowed.count(sampler.sample(x.data())));
  }
  {  // TestTopKDisabledByZero
    Sampler sampler{50, 1.0f, 0.0f, 7};
    sampler.set_topk(0);
    std::vector<float> x(50, -10.0f);
    x[11] = 20.0f;
    int hits = 0;
    for (int t = 0; t < 20; ++t) hits += sampler.sample(x.data()) == 11;
    CHECK(hits >= 18);
  }
  {  // TestTopKEqualsOneIsArgmax
    Sampler sampler{100, 1.0f, 0.0f, 123};
    sampler.set_topk(1);
    std::vector<float> x(100);
    for (auto& v : x) v = uni(rng);
    x[57] = 100.0f;
    for (int t = 0; t < 10; ++t) CHECK(sampler.sample(x.data()) == 57);
  }
  {  // TestTopKTakesPrecedenceOverTopP
    Sampler sampler{100, 1.0f, 0.99f, 99};
    sampler.set_topk(2);
    std::vector<float> x(100, -10.0f);
    x[3] = 5.0f, x[8] = 4.5f, x[19] = 4.0f;
    const std::set<int32_t> allowed = {3, 8};
    for (int t = 0; t < 50; ++t) CHECK(allowed.count(sampler.sample(x.data())));
  }
  {  // logits_to_token: rank 2, rank 3 (last position), temperature > 0 stays in range
    FakeTensor t2{{0.1f, 0.2f, 0.8f, 0.4f}, {1, 4}};
    CHECK(executorch::extension::llm::logits_to_token(t2) == 2);
    FakeTensor t3{{0.8f, 0.1f, 0.1f, 0.1f, 0.1f, 0.2f, 0.8f, 0.4f}, {1, 2, 4}};
    CHECK(executorch::extension::llm::logits_to_token(t3) == 2);
    const int32_t tok = executorch::extension::llm::logits_to_token(t2, 1.0f);
    CHECK(tok >= 0 && tok < 4);
    Sampler injected{4, 0.0f};
    CHECK(executorch::extension::llm::sample_from_logits(t3, injected) == 2);
    torch::executor::Sampler alias{4, 0.0f, executorch::llm::kTopp, 1};  // deprecated aliases still resolve
    CHECK(alias.sample(t2.data.data()) == 2);
  }
  {  // the 4-logit known answer of the reference with seed 42: token 2
    Sampler sampler{4, 1.0f, 0.9f, 42};
    float x[4] = {0.1f, 0.2f, 0.8f, 0.4f};
    CHECK(sampler.sample(x) == 2);
    CHECK(x[2] == 0.8f);  // the buffer is left alone
  }
  std::printf("test_sampler_shim: all passed\n");
  return 0;
}
