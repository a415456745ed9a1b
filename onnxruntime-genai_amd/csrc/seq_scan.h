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
// The two increments are read off real float additions: inside a binade consecutive floats have
// consecutive bit patterns one unit apart, so adding e to the binade's first even value (mantissa
// integer 2^23) and to its first odd one (2^23 + 1) and subtracting the bit patterns gives the
// rounded increments for even and odd sums -- round-to-nearest-even included, done by the adder
// itself.  If such a sum lands in a higher binade the increment is at least 2^23 - 1 units, which
// takes every sum of that parity to 2^24 or beyond: it is reported as saturated ("left the binade")
// and the caller performs that addition for real.
EM_HD Step seq_make_step(float e, int se) {
  const uint32_t b0 = static_cast<uint32_t>(se) << 23;
  const uint32_t b1 = b0 | 1u;
  const uint32_t r0 = em::as_u32(em::as_float(b0) + e);
  const uint32_t r1 = em::as_u32(em::as_float(b1) + e);
  const uint32_t lim = b0 + 0x800000u;  // first bit pattern of the next binade
  Step f;
  f.d0 = r0 < lim ? r0 - b0 : kStepSat;
  f.d1 = r1 < lim ? r1 - b1 : kStepSat;
  return f;
}

// The composition of the step functions of e[0..count) (finite, >= 0) under the unit 2^(se-150), read off real
// float additions in one go: within a binade the rounding of an addition depends only on the addend and on the
// parity of the sum's mantissa integer, so all even sums of the binade run through the same sequence of
// parities and increments as its first even value does, and all odd ones as its first odd value does.  The two
// are added up for real; where such a sum lands in a higher binade (it cannot come back: the addends are not
// negative) the composition is reported as saturated, which the composition of the single steps would carry to
// 2^24 or beyond from every start of that parity as well.
EM_HD Step seq_compose_run(const float* e, int count, int se) {
  const uint32_t b0 = static_cast<uint32_t>(se) << 23;
  const uint32_t b1 = b0 | 1u;
  float f0 = em::as_float(b0), f1 = em::as_float(b1);
#pragma unroll
  for (int j = 0; j < count; ++j) {
    f0 = f0 + e[j];
    f1 = f1 + e[j];
  }
  const uint32_t r0 = em::as_u32(f0), r1 = em::as_u32(f1);
  const uint32_t lim = b0 + 0x800000u;  // first bit pattern of the next binade
  Step f;
  f.d0 = r0 < lim ? r0 - b0 : kStepSat;
  f.d1 = r1 < lim ? r1 - b1 : kStepSat;
  return f;
}

}  // namespace ms
