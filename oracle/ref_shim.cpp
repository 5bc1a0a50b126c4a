// TEST INFRASTRUCTURE ONLY.  C-ABI wrapper around the *unmodified* reference
// Sampler (compiled from /root/reference/extension/llm/sampler/sampler.cpp by
// oracle/build_ref.sh into oracle/_ref/).  It exists so that the repo's own CPU
// restatement (sampler_oracle.cpp) can be A/B-checked bit-for-bit against the
// real thing inside the build container, and so golden vectors can be written.
// Nothing in the product path may load this library.
#include <executorch/extension/llm/sampler/sampler.h>

#include <cstdint>

using executorch::extension::llm::Sampler;

extern "C" {

void* ref_sampler_create(int32_t vocab, float temperature, float topp, unsigned long long seed) {
  return new Sampler(vocab, temperature, topp, seed);
}

void ref_sampler_destroy(void* h) { delete static_cast<Sampler*>(h); }

void ref_sampler_set_temperature(void* h, float t) { static_cast<Sampler*>(h)->set_temperature(t); }

void ref_sampler_set_topk(void* h, int32_t k) { static_cast<Sampler*>(h)->set_topk(k); }

// dtype codes follow executorch ScalarType: 6 Float, 5 Half, 15 BFloat16, 27 UInt16.
// The buffer is overwritten with probabilities exactly as the reference does.
int32_t ref_sampler_sample(void* h, void* logits, int32_t dtype) {
  Sampler* s = static_cast<Sampler*>(h);
  switch (dtype) {
    case 6:
      return s->sample(static_cast<float*>(logits));
    case 5:
      return s->sample(static_cast<executorch::aten::Half*>(logits));
    case 15:
      return s->sample(static_cast<executorch::aten::BFloat16*>(logits));
    case 27:
      return s->sample(static_cast<uint16_t*>(logits));
    default:
      return -1;
  }
}

}  // extern "C"
