// Bit-reproducible single-precision exp/log shared by host and device code.
//
// The reference CPU path evaluates std::exp / std::log on float
// (src/sampling_distribution.h:165,254,290; src/softmax.h:14,40,44), i.e. glibc's expf/logf.
// glibc (>= 2.28) implements both with the table-driven double-precision algorithms of the
// ARM optimized-routines project.  Those algorithms use only IEEE-754 double add/mul/fma and
// one final double->float rounding, so restating them with explicit fma() calls yields the same
// float for every input on any IEEE machine -- an x86 host or a CDNA4 device alike.  The sampling
// kernels therefore produce probabilities that are bit-identical to the host libm results, which
// is what makes the nucleus cut-off and the categorical draw bit-exact.
//
// EM_CONTRACT selects how a*b+c is evaluated: 1 = fused (matches the FMA ifunc variants glibc
// picks on every x86-64 CPU with AVX2+FMA), 0 = separately rounded.  tests/test_exact_math.py
// compares both against the running host's libm.
#pragma once
#include <stdint.h>
#include <string.h>
#include <math.h>

#if defined(__HIPCC__)
#define EM_HD __host__ __device__ inline
#else
#define EM_HD inline
#endif

#ifndef EM_CONTRACT
#define EM_CONTRACT 1
#endif

namespace em {

EM_HD double as_double(uint64_t u) {
  double d;
  memcpy(&d, &u, sizeof(d));
  return d;
}
EM_HD uint64_t as_u64(double d) {
  uint64_t u;
  memcpy(&u, &d, sizeof(u));
  return u;
}
EM_HD float as_float(uint32_t u) {
  float f;
  memcpy(&f, &u, sizeof(f));
  return f;
}
EM_HD uint32_t as_u32(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof(u));
  return u;
}

// a*b+c with the rounding behaviour selected by EM_CONTRACT.
EM_HD double mad(double a, double b, double c) {
#if EM_CONTRACT
  return fma(a, b, c);
#else
  volatile double p = a * b;  // volatile: forbid the compiler from fusing the two roundings
  return p + c;
#endif
}

// 2^(i/32) for i = 0..31 as IEEE doubles with i<<47 subtracted from the bit pattern, so that adding
// (k << 47) for the integer k = round(32*x/ln2) yields 2^(k/32) directly.
EM_HD uint64_t exp2_tab(uint32_t i) {
  const uint64_t tab[32] = {
      0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
      0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
      0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
      0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
      0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
      0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
      0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
      0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL,
  };
  return tab[i];
}

// expf(x), bit-identical to glibc's.  `tab(i)` must return exp2_tab(i); callers that already hold the
// table in registers or LDS pass their own accessor.
template <typename Tab>
EM_HD float expf_core(float x, Tab tab) {
  const uint32_t ix = as_u32(x);
  const uint32_t abstop = (ix >> 20) & 0x7ff;
  const double N = 32.0;
  const double inv_ln2_n = 0x1.71547652b82fep+0 * N;
  const double shift = 0x1.8p+52;
  const double c0 = 0x1.c6af84b912394p-5 / N / N / N;
  const double c1 = 0x1.ebfce50fac4f3p-3 / N / N;
  const double c2 = 0x1.62e42ff0c52d6p-1 / N;
  const double xd = (double)x;
  double z = inv_ln2_n * xd;
  double kd = z + shift;
  const uint64_t ki = as_u64(kd);
  kd -= shift;
#if EM_CONTRACT
  const double r = fma(inv_ln2_n, xd, -kd);  // the product feeding z - kd is fused in glibc's FMA build
#else
  const double r = z - kd;
#endif
  uint64_t t = tab((uint32_t)(ki % 32));
  t += ki << (52 - 5);
  const double s = as_double(t);
  z = mad(c0, r, c1);
  const double r2 = r * r;
  double y = mad(c2, r, 1.0);
  y = mad(z, r2, y);
  y = y * s;
  float res = (float)y;
  if (abstop >= 0x42b) {  // |x| >= 88 or NaN/Inf
    if (ix == 0xff800000u) res = 0.0f;
    else if (abstop >= 0x7f8) res = x + x;
    else if (x > 0x1.62e42ep6f) res = as_float(0x7f800000u);  // overflow
    else if (x < -0x1.9fe368p6f) res = 0.0f;                  // underflow to zero
  }
  return res;
}

struct DefaultExp2Tab {
  EM_HD uint64_t operator()(uint32_t i) const { return exp2_tab(i); }
};

EM_HD float expf_exact(float x) { return expf_core(x, DefaultExp2Tab{}); }

struct LogTab {
  double invc, logc;
};

EM_HD LogTab log_tab(uint32_t i) {
  const LogTab tab[16] = {
      {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
      {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
      {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
      {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
      {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
      {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
      {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
      {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2},
  };
  return tab[i];
}

// logf(x), bit-identical to glibc's.
EM_HD float logf_exact(float x) {
  uint32_t ix = as_u32(x);
  if (ix == 0x3f800000u) return 0.0f;
  if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
    if (ix * 2 == 0) return as_float(0xff800000u);            // log(+-0) = -inf
    if (ix == 0x7f800000u) return x;                          // log(inf) = inf
    if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return as_float(0x7fc00000u);  // NaN
    ix = as_u32(x * 0x1p23f);                                 // subnormal: normalise
    ix -= 23u << 23;
  }
  const double ln2 = 0x1.62e42fefa39efp-1;
  const double a0 = -0x1.00ea348b88334p-2, a1 = 0x1.5575b0be00b6ap-2, a2 = -0x1.ffffef20a4123p-2;
  const uint32_t tmp = ix - 0x3f330000u;
  const uint32_t i = (tmp >> (23 - 4)) % 16;
  const int32_t k = (int32_t)tmp >> 23;
  const uint32_t iz = ix - (tmp & 0xff800000u);
  const LogTab t = log_tab(i);
  const double z = (double)as_float(iz);
  const double r = mad(z, t.invc, -1.0);
  const double y0 = mad((double)k, ln2, t.logc);
  const double r2 = r * r;
  double y = mad(a1, r, a2);
  y = mad(a0, r2, y);
  y = mad(y, r2, y0 + r);
  return (float)y;
}

}  // namespace em
