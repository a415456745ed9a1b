// Compares the library's bit-reproducible expf/logf (csrc/exact_math.h, host build) with the running
// host's libm over every float bit pattern.  Prints "<exp mismatches> <log mismatches>".
#include <cmath>
#include <cstdio>
#include "exact_math.h"
int main() {
  unsigned long long bad_e = 0, bad_l = 0;
#pragma omp parallel for reduction(+ : bad_e, bad_l) schedule(static)
  for (long long b = 0; b < (1LL << 32); b++) {
    const uint32_t u = (uint32_t)b;
    const float x = em::as_float(u);
    const float a = expf(x), m = em::expf_exact(x);
    if (em::as_u32(a) != em::as_u32(m) && !(a != a && m != m)) bad_e++;
    const float la = logf(x), lm = em::logf_exact(x);
    if (em::as_u32(la) != em::as_u32(lm) && !(la != la && lm != lm)) bad_l++;
  }
  printf("%llu %llu\n", bad_e, bad_l);
  return 0;
}
