// Integer arithmetic behind the sequential-float-sum emulation.  No HIP dependency: the
// includer defines ETS_HD (function qualifiers), so the same code is unit-tested on the host.
#pragma once

#include <stdint.h>

#ifndef ETS_HD
#define ETS_HD inline
#endif

namespace ets {

constexpr uint32_t kSat = 1u << 26;  // saturation value of integer increments (> 2^24)

// ---- correctly rounded float division by a row constant ----------------------------------------
// fl(e / S) for e >= 0 and a normal S > 0, from r = double(1) / double(S) computed once per row:
// the double product e * r is within 2^-52 (relative) of the quotient, while the quotient of two
// 24-bit significands stays at least 2^-49 away from every rounding boundary of the NORMAL float
// grid (a boundary has a 25-bit odd significand M, and e = M * S would need 2^24 | significand(S)),
// so rounding the product to float rounds the quotient correctly.  On the subnormal grid exact
// ties do occur (e = 3 * 2^-149, S = 6), so results at or below 2^-126 take the division itself.
struct RowDivisor {
  float S;
  double recip;
};

ETS_HD RowDivisor row_divisor(float S) {
  RowDivisor d;
  d.S = S;
  d.recip = 1.0 / static_cast<double>(S);
  return d;
}

// The same quotient where only results above 2^-126 matter (comparisons against a threshold that
// is itself above 2^-126): exact there, and at most 2^-126 whenever the true result is.
ETS_HD float div_row_above(float e, const RowDivisor& d) {
  return static_cast<float>(static_cast<double>(e) * d.recip);
}

ETS_HD float div_row(float e, const RowDivisor& d) {
  const float p = static_cast<float>(static_cast<double>(e) * d.recip);
  if (p <= 1.17549435e-38f && e != 0.0f) return e / d.S;  // 2^-126 and below (also NaN-free: p >= 0)
  return p;
}

// The same for a numerator of either sign (logits divided by a temperature).
ETS_HD float div_row_signed(float x, const RowDivisor& d) {
  const float q = static_cast<float>(static_cast<double>(x) * d.recip);
  if (__builtin_fabsf(q) <= 1.17549435e-38f && x != 0.0f) return x / d.S;
  return q;
}

// ---- sequential float sums as an integer scan --------------------------------------------------
// A scalar loop `s += a[i]` (a[i] >= 0) rounds after every add.  While s stays inside one
// binade [2^k, 2^(k+1)) every partial sum is an integer multiple of u = ulp(s): writing
// s = S*u, adding a gives S + rne(a/u), where the tie case (a/u has fraction exactly 1/2)
// rounds so that the new S is even.  The increment therefore depends on the incoming state only
// through the PARITY of S, so a run of elements is summarised by two integers -- the total
// increment when entered with S even and with S odd -- and such summaries compose
// associatively.  That turns the loop into a parallel scan.  When a partial sum would leave the
// binade (S + inc >= 2^24) the summary stops being valid; the caller then lets one lane do the
// offending adds natively and restarts the scan behind it with the new u.

struct ParityInc {
  uint32_t even;  // total increment if the run is entered with S even
  uint32_t odd;   // ... with S odd
};

ETS_HD uint32_t sat_add(uint32_t a, uint32_t b) {
  const uint32_t c = a + b;
  return c < kSat ? c : kSat;
}

// a followed by b
ETS_HD ParityInc compose(ParityInc a, ParityInc b) {
  ParityInc c;
  c.even = sat_add(a.even, (a.even & 1u) ? b.odd : b.even);
  c.odd = sat_add(a.odd, ((a.odd + 1u) & 1u) ? b.odd : b.even);
  return c;
}

// Which lane (or slot) an ordered walk works on next: the first one flagged in `events` at or
// after `from`, or `count` when there is none.  Every ordered walk of the sampler advances with
//   j = next_event(events, from, 64); ...; from = j + 1;
// so it takes at most `count` steps whatever the flags say -- also on data that is not what the
// walk was written for (probabilities that are not sorted, a threshold below the starting sum,
// NaN), where flags of lanes already consumed could otherwise call the walk back for good.
ETS_HD int next_event(uint64_t events, int from, int count) {
  if (from >= 64) return count;
  const uint64_t ahead = events & (~0ull << from);
  if (!ahead) return count;
  const int j = __builtin_ctzll(ahead);
  return j < count ? j : count;
}

// Integer view of the running sum: s = S * 2^(kb - 150) with kb the biased exponent (>= 1).
struct SumState {
  uint32_t S;
  int kb;
};

ETS_HD SumState sum_state(float s) {
  const uint32_t b = __builtin_bit_cast(uint32_t, s);
  SumState st;
  const uint32_t e = b >> 23;  // s >= 0, so no sign bit
  st.kb = e ? static_cast<int>(e) : 1;
  st.S = e ? ((b & 0x7fffffu) | 0x800000u) : b;
  return st;
}

// Inverse of sum_state for S' <= 2^24 (the implicit bit carries into the exponent field).
ETS_HD float sum_value(uint32_t S, int kb) {
  return __builtin_bit_cast(float, (static_cast<uint32_t>(kb - 1) << 23) + S);
}

// Fold element `abits` (float bits, finite, >= 0) into a lane's summary.
ETS_HD void fold_elem(ParityInc& acc, uint32_t abits, int kb) {
  uint32_t ea = abits >> 23;
  uint32_t M = abits & 0x7fffffu;
  if (ea) {
    M |= 0x800000u;
  } else {
    ea = 1;
  }
  const int sh = kb - static_cast<int>(ea);
  uint32_t n0, up = 0, tie = 0;
  if (sh <= 0) {
    n0 = (sh < -2) ? kSat : (M << (-sh));  // a >= 2^k: certainly leaves the binade
  } else if (sh >= 25) {
    n0 = 0;  // a < u/2: absorbed
  } else {
    n0 = M >> sh;
    const uint32_t rem = M & ((1u << sh) - 1u);
    const uint32_t half = 1u << (sh - 1);
    up = rem > half ? 1u : 0u;
    tie = rem == half ? 1u : 0u;
  }
  const uint32_t base = n0 + up;
  const uint32_t inc_even = base + (tie & ((acc.even + n0) & 1u));
  const uint32_t inc_odd = base + (tie & ((acc.odd + n0 + 1u) & 1u));
  acc.even = sat_add(acc.even, inc_even);
  acc.odd = sat_add(acc.odd, inc_odd);
}

// fold_elem for running sums with biased exponent kb >= 64, where a / ulp(s) is an exact
// power-of-two scaling in float: `scale` = 2^(150 - kb).  Same result as fold_elem.
ETS_HD void fold_elem_scaled(ParityInc& acc, float a, float scale) {
  float t = a * scale;
  t = t < 67108864.0f ? t : 67108864.0f;  // 2^26 == kSat
  const float fl = __builtin_floorf(t);
  const float frac = t - fl;  // exact
  const uint32_t n0 = static_cast<uint32_t>(fl);
  const uint32_t up = frac > 0.5f ? 1u : 0u;
  const uint32_t tie = frac == 0.5f ? 1u : 0u;
  const uint32_t base = n0 + up;
  const uint32_t inc_even = base + (tie & ((acc.even + n0) & 1u));
  const uint32_t inc_odd = base + (tie & ((acc.odd + n0 + 1u) & 1u));
  acc.even = sat_add(acc.even, inc_even);
  acc.odd = sat_add(acc.odd, inc_odd);
}

// Order-free shortcut used while a whole chunk stays inside the binade of s (biased exponent
// kb >= 64) and no element sits on a half-ulp tie: the increment of `abits` is rne(a / ulp(s)),
// computed with an exact power-of-two scaling in float.  Sets `tie` when the fraction is exactly
// 1/2 (the caller must then fall back to the ordered scan) and saturates at kSat.
ETS_HD uint32_t fast_inc(uint32_t abits, int kb, bool& tie) {
  const float scale = __builtin_bit_cast(float, static_cast<uint32_t>(277 - kb) << 23);  // 2^(150 - kb)
  float t = __builtin_bit_cast(float, abits) * scale;
  t = t < 67108864.0f ? t : 67108864.0f;
  const float r = __builtin_rintf(t);
  tie = tie || (__builtin_fabsf(t - r) == 0.5f);
  return static_cast<uint32_t>(r);
}

// ---- runs of equal addends ----------------------------------------------------------------------
// c copies of p are added to s one after the other (s = s + p in fp32); the walk stops behind the
// first copy that takes s above T.  Returns that copy's number (1-based), or 0 when all c copies
// were added without exceeding T.  One lane.
ETS_HD uint32_t run_walk(float& s, float p, uint32_t c, float T) {
  uint32_t left = c, done = 0u;
  while (left > 0u) {
    const SumState ss = sum_state(s);
    const float scale = ss.kb >= 64 && ss.kb <= 250 ? __builtin_bit_cast(float, static_cast<uint32_t>(277 - ss.kb) << 23) : 0.0f;
    const float t = p * scale;
    if (scale == 0.0f || !(t < 16777216.0f)) {  // out of the shortcut's range: one native add
      s = s + p;
      --left;
      ++done;
      if (s > T) return done;
      continue;
    }
    const float r = __builtin_rintf(t);
    uint32_t n = static_cast<uint32_t>(r);
    uint32_t S = ss.S;
    if (__builtin_fabsf(t - r) == 0.5f) {
      // a half-ulp tie: the first add goes natively and leaves an even integer; from an even integer
      // every further copy adds floor(t), or one more if that is odd
      s = s + p;
      --left;
      ++done;
      if (s > T) return done;
      const SumState s2 = sum_state(s);
      if (s2.kb != ss.kb) continue;
      const uint32_t n0 = static_cast<uint32_t>(__builtin_floorf(t));
      n = n0 + (n0 & 1u);
      S = s2.S;
    }
    if (n == 0u) return 0u;  // absorbed: no copy changes the sum
    // s' > T  <=>  S' >= floor(T / ulp) + 1; the sum must also stay below 2^24 ulps
    const float tt = T * scale;
    uint32_t limit = 1u << 24;
    if (tt < 16777216.0f) {
      const uint32_t Tn = tt >= 0.0f ? static_cast<uint32_t>(__builtin_floorf(tt)) + 1u : 0u;
      limit = Tn < limit ? Tn : limit;
    }
    if (S >= limit) {  // (cannot happen: the walk would have stopped) one native add
      s = s + p;
      --left;
      ++done;
      if (s > T) return done;
      continue;
    }
    const uint32_t stay = (limit - S - 1u) / n;  // copies after which the integer is still below `limit`
    if (stay >= left) {
      s = sum_value(S + left * n, ss.kb);
      return 0u;
    }
    s = sum_value(S + stay * n, ss.kb);
    left -= stay;
    done += stay;
    s = s + p;  // the copy that reaches the limit, natively
    --left;
    ++done;
    if (s > T) return done;
  }
  return 0u;
}

}  // namespace ets
