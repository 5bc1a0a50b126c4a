// Host checks of two pieces of ets_seqsum_math.h that the ordered walks of the sampler rest on:
//
//  * next_event(): whatever flags a step computes -- including flags of lanes the walk has already
//    consumed, as a threshold below the starting sum, NaN or unsorted probabilities produce -- a walk
//    of the form  j = next_event(flags, from, n); ...; from = j + 1  ends after at most n steps;
//  * run_walk(): c copies of p added one after the other, in closed form, against the plain loop
//    (the sum behind the run and the copy behind which the sum first exceeds the threshold), over
//    binade changes, half-ulp ties, absorbed addends and thresholds in every position.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <random>

#include "ets_seqsum_math.h"

using namespace ets;

static uint32_t plain_walk(float& s, float p, uint32_t c, float T) {
  for (uint32_t k = 1; k <= c; ++k) {
    volatile float t = s + p;  // one fp32 add, rounded
    s = t;
    if (s > T) return k;
  }
  return 0;
}

int main() {
  std::mt19937_64 rng(2024);
  long bad = 0, cases = 0;
  // ---- next_event
  for (int rep = 0; rep < 200000; ++rep) {
    uint64_t flags = rng();
    if (rep % 3 == 0) flags &= rng();
    if (rep % 7 == 0) flags = 0;
    if (rep % 11 == 0) flags = ~0ull;
    const int count = 1 + static_cast<int>(rng() % 64);
    const int from = static_cast<int>(rng() % 70);
    const int j = next_event(flags, from, count);
    int want = count;
    for (int l = from; l < count && l < 64; ++l) {
      if ((flags >> l) & 1ull) {
        want = l;
        break;
      }
    }
    if (j != want) ++bad;
    ++cases;
  }
  // a walk whose flags are redrawn adversarially at every step (always flagging consumed lanes)
  for (int rep = 0; rep < 20000; ++rep) {
    int from = 0, steps = 0;
    const int count = 1 + static_cast<int>(rng() % 64);
    while (from < count) {
      const uint64_t flags = rng() | ((1ull << from) - 1ull) | (from ? 1ull : 0ull);
      const int j = next_event(flags, from, count);
      if (j < from) ++bad;
      if (j >= count) break;
      from = j + 1;
      if (++steps > 64) {
        ++bad;
        break;
      }
    }
    ++cases;
  }
  // ---- run_walk against the plain loop
  auto uni = [&](double lo, double hi) { return lo + (hi - lo) * (rng() >> 11) * (1.0 / 9007199254740992.0); };
  for (int rep = 0; rep < 60000; ++rep) {
    float s0, p;
    uint32_t c;
    const int kind = rep % 10;
    switch (kind) {
      case 0:  // small addend against a large sum: many copies per binade
        s0 = static_cast<float>(std::exp(uni(-8, 0)));
        p = s0 * static_cast<float>(std::exp(uni(-17, -9)));
        c = 1 + static_cast<uint32_t>(rng() % 65535);
        break;
      case 1:  // comparable sizes: a binade change every few copies
        s0 = static_cast<float>(std::exp(uni(-12, 0)));
        p = s0 * static_cast<float>(uni(0.01, 3.0));
        c = 1 + static_cast<uint32_t>(rng() % 200);
        break;
      case 2:  // half-ulp ties: p = (n0 + 1/2) ulp(s)
      case 3: {
        const int e = -static_cast<int>(rng() % 20);
        s0 = std::ldexp(static_cast<float>(8388608 + (rng() % 8388608)), e - 23);  // any parity
        p = std::ldexp(static_cast<float>(rng() % 64) + 0.5f, e - 23);
        c = 1 + static_cast<uint32_t>(rng() % 4000);
        break;
      }
      case 4:  // absorbed: below half an ulp
        s0 = static_cast<float>(uni(0.5, 1.0));
        p = s0 * static_cast<float>(std::exp(uni(-30, -17.5)));
        c = 1 + static_cast<uint32_t>(rng() % 65535);
        break;
      case 5:  // from zero
        s0 = 0.0f;
        p = static_cast<float>(std::exp(uni(-20, 0)));
        c = 1 + static_cast<uint32_t>(rng() % 3000);
        break;
      case 6:  // powers of two
        s0 = std::ldexp(1.0f, -static_cast<int>(rng() % 24));
        p = std::ldexp(1.0f, -static_cast<int>(rng() % 48));
        c = 1 + static_cast<uint32_t>(rng() % 65535);
        break;
      case 7:  // tiny sums (outside the shortcut's range)
        s0 = std::ldexp(static_cast<float>(uni(1, 2)), -80 - static_cast<int>(rng() % 60));
        p = s0 * static_cast<float>(uni(0.001, 2.0));
        c = 1 + static_cast<uint32_t>(rng() % 300);
        break;
      case 8:  // zero addend
        s0 = static_cast<float>(uni(0, 1));
        p = 0.0f;
        c = 1 + static_cast<uint32_t>(rng() % 1000);
        break;
      default:
        s0 = static_cast<float>(uni(0, 1));
        p = static_cast<float>(uni(0, 1e-4));
        c = 1 + static_cast<uint32_t>(rng() % 65535);
        break;
    }
    float end = s0;
    plain_walk(end, p, c, INFINITY);
    float thresholds[4] = {INFINITY, s0 + (end - s0) * static_cast<float>(uni(0, 1.1)), end, s0};
    for (float T : thresholds) {
      float a = s0, b = s0;
      const uint32_t ka = plain_walk(a, p, c, T);
      const uint32_t kb = run_walk(b, p, c, T);
      if (ka != kb || a != b) {
        if (bad < 10) std::printf("run_walk mismatch: s0=%a p=%a c=%u T=%a: plain (%u, %a) closed form (%u, %a)\n", s0, p, c, T, ka, a, kb, b);
        ++bad;
      }
      ++cases;
    }
  }
  std::printf("%ld cases, %ld mismatches\n", cases, bad);
  return bad ? 1 : 0;
}
