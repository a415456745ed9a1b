// Exact emulation of a left-to-right fp32 summation as an associative scan.
//
// The reference accumulates exp() values into a float strictly in sequence
// (LogSoftMax src/softmax.h:36-41, FindNucleus src/sampling_distribution.h:164-174, the probability
// sums :252-256,288-292).  The float it ends with depends on that order, and discrete decisions hang
// on it (nucleus cut-off, beam ranking), so a tree reduction is not good enough.  Observation: while
// the running sum s stays inside one binade, s = n * ulp with an integer n in [2^23, 2^24), and
// adding a non-negative float e rounds to n + a + r, where a = floor(e/ulp) and r in {0,1} depends
// only on the fraction of e/ulp and -- for an exact tie -- on the parity of n + a.  Every addend is
// therefore a function  n -> n + d[n & 1]  given by two integers (d[0], d[1]); such functions are
// closed under composition, so prefix sums are an ordinary parallel scan over pairs of integers.
// When a prefix would reach 2^24 the sum leaves the binade: that single addition is done with a real
// float add and the scan restarts behind it.  There are at most ~280 binades, in practice < 30.
//
// This header is host/device neutral so the integer logic can be fuzzed on the CPU against real
// float additions (tests/seq_scan_check.cpp).
#pragma once
#include <stdint.h>
#include "exact_math.h"

namespace ms {

struct Step {
  uint32_t d0, d1;  // increment applied to an even / odd mantissa integer
};

constexpr uint32_t kStepSat = 1u << 30;   // increments saturate here (anything >= 2^24 means "left the binade")
constexpr uint32_t kMantLimit = 1u << 24;

EM_HD uint32_t step_sat_add(uint32_t a, uint32_t b) {
  const uint32_t s = a + b;  // a, b <= 2^30: no wrap
  return s > kStepSat ? kStepSat : s;
}

// Apply f, then g.
EM_HD Step step_compose(Step f, Step g) {
  Step r;
  r.d0 = step_sat_add(f.d0, (f.d0 & 1u) ? g.d1 : g.d0);
  r.d1 = step_sat_add(f.d1, ((f.d1 + 1u) & 1u) ? g.d1 : g.d0);
  return r;
}

EM_HD uint32_t step_apply(uint32_t n, Step f) { return step_sat_add(n, (n & 1u) ? f.d1 : f.d0); }

// A non-negative finite float s as n * 2^(se-150): se = biased exponent (subnormals use 1), n < 2^24.
struct SeqState {
  uint32_t n;
  int se;
};

EM_HD SeqState seq_decompose(float s) {
  const uint32_t b = em::as_u32(s) & 0x7fffffffu;
  const uint32_t er = b >> 23;
  SeqState st;
  st.n = er ? ((b & 0x7fffffu) | 0x800000u) : (b & 0x7fffffu);
  st.se = er ? static_cast<int>(er) : 1;
  return st;
}

// Inverse of seq_decompose for n < 2^24 (n < 2^23 only occurs with se == 1).
EM_HD float seq_recompose(uint32_t n, int se) {
  if (n < 0x800000u) return em::as_float(n);
  return em::as_float((static_cast<uint32_t>(se) << 23) | (n & 0x7fffffu));
}

// The step function of adding e (finite, >= 0) to a running sum whose unit is 2^(se-150).
EM_HD Step seq_make_step(float e, int se) {
  const uint32_t b = em::as_u32(e) & 0x7fffffffu;
  const uint32_t er = b >> 23;
  const uint32_t m = er ? ((b & 0x7fffffu) | 0x800000u) : (b & 0x7fffffu);
  const int ee = er ? static_cast<int>(er) : 1;
  const int shift = se - ee;  // e = m * 2^(-shift) units
  Step f;
  if (m == 0u) {
    f.d0 = f.d1 = 0u;
  } else if (shift <= 0) {
    const uint32_t a = (-shift >= 6) ? kStepSat : (m << (-shift));  // m < 2^24, so m << 5 < 2^29
    f.d0 = f.d1 = a > kStepSat ? kStepSat : a;
  } else if (shift > 25) {
    f.d0 = f.d1 = 0u;  // below half a unit
  } else {
    const uint32_t a = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half) {
      f.d0 = f.d1 = a + 1u;
    } else if (rem < half) {
      f.d0 = f.d1 = a;
    } else {  // tie: round to even
      f.d0 = a + (a & 1u);
      f.d1 = a + ((a & 1u) ^ 1u);
    }
  }
  return f;
}

}  // namespace ms
