// CPU fuzz of csrc/seq_scan.h: the integer emulation of left-to-right fp32 summation must equal real
// float additions for every prefix.  Prints the number of mismatches (0 expected).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
#include "seq_scan.h"
using namespace ms;

// Windowed emulation, as the device code organises it: within a window, prefixes are compositions of
// step functions; a prefix that would leave the binade is redone as a real float add.
static bool run_case(const std::vector<float>& e, float s0, int window, bool tree) {
  const int n = (int)e.size();
  std::vector<float> want(n);
  {
    volatile float s = s0;
    for (int i = 0; i < n; ++i) { s = s + e[i]; want[i] = s; }
  }
  float s = s0;
  int i0 = 0;
  while (i0 < n) {
    const int cnt = std::min(window, n - i0);
    const SeqState st = seq_decompose(s);
    std::vector<Step> f(cnt), pre(cnt);
    for (int j = 0; j < cnt; ++j) f[j] = seq_make_step(e[i0 + j], st.se);
    if (!tree) {
      Step acc{0, 0};
      for (int j = 0; j < cnt; ++j) { acc = step_compose(acc, f[j]); pre[j] = acc; }
    } else {  // Hillis-Steele style inclusive scan: exercises associativity
      pre = f;
      for (int d = 1; d < cnt; d <<= 1) {
        std::vector<Step> nxt = pre;
        for (int j = d; j < cnt; ++j) nxt[j] = step_compose(pre[j - d], pre[j]);
        pre.swap(nxt);
      }
    }
    int cross = -1;
    for (int j = 0; j < cnt; ++j) {
      const uint32_t na = step_apply(st.n, pre[j]);
      if (na >= kMantLimit) { cross = j; break; }
      if (em::as_u32(seq_recompose(na, st.se)) != em::as_u32(want[i0 + j])) return false;
    }
    if (cross < 0) {
      s = seq_recompose(step_apply(st.n, pre[cnt - 1]), st.se);
      i0 += cnt;
    } else {
      const float sb = cross ? seq_recompose(step_apply(st.n, pre[cross - 1]), st.se) : s;
      volatile float t = sb + e[i0 + cross];
      s = t;
      if (em::as_u32(s) != em::as_u32(want[i0 + cross])) return false;
      i0 += cross + 1;
    }
  }
  return true;
}

// The same with every `group` consecutive addends turned into one step function by seq_compose_run (real float
// additions from the binade's first even and first odd value), as the kernels that only need a thread's aggregate do:
// checked where a group ends; a group in which the sum leaves the binade is added element by element.
static bool run_case_groups(const std::vector<float>& e, float s0, int window, int group) {
  const int n = (int)e.size();
  std::vector<float> want(n);
  {
    volatile float s = s0;
    for (int i = 0; i < n; ++i) { s = s + e[i]; want[i] = s; }
  }
  float s = s0;
  int i0 = 0;
  while (i0 < n) {
    const int cnt = std::min(window * group, n - i0);
    const int groups = (cnt + group - 1) / group;
    const SeqState st = seq_decompose(s);
    Step acc{0, 0};
    int cross = -1;
    uint32_t before = st.n;
    for (int g = 0; g < groups; ++g) {
      const int len = std::min(group, cnt - g * group);
      acc = step_compose(acc, seq_compose_run(&e[i0 + g * group], len, st.se));
      const uint32_t na = step_apply(st.n, acc);
      if (na >= kMantLimit) { cross = g; break; }
      if (em::as_u32(seq_recompose(na, st.se)) != em::as_u32(want[i0 + g * group + len - 1])) return false;
      before = na;
    }
    if (cross < 0) {
      s = seq_recompose(before, st.se);
      i0 += cnt;
    } else {
      volatile float t = cross ? seq_recompose(before, st.se) : s;
      const int len = std::min(group, cnt - cross * group);
      for (int j = 0; j < len; ++j) t = t + e[i0 + cross * group + j];
      s = t;
      if (em::as_u32(s) != em::as_u32(want[i0 + cross * group + len - 1])) return false;
      i0 += cross * group + len;
    }
  }
  return true;
}

int main() {
  std::mt19937_64 rng(12345);
  std::normal_distribution<float> nd(0.f, 1.f);
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  long bad = 0, cases = 0;
  for (int rep = 0; rep < 6000; ++rep) {
    const int kind = rep % 8;
    const int n = 1 + (int)(rng() % 3000);
    std::vector<float> e(n);
    float s0 = 0.f;
    for (int i = 0; i < n; ++i) {
      switch (kind) {
        case 0: e[i] = std::exp(nd(rng) * 3.f - 8.f); break;                 // softmax-like
        case 1: e[i] = ud(rng); break;
        case 2: e[i] = std::ldexp((float)(rng() % 8), -24 - (int)(rng() % 4)); break;  // exact ties
        case 3: e[i] = std::ldexp(ud(rng), -140 + (int)(rng() % 20)); break;           // subnormal range
        case 4: e[i] = (rng() % 50 == 0) ? std::ldexp(ud(rng), (int)(rng() % 40)) : ud(rng) * 1e-6f; break;
        case 5: e[i] = std::exp(-(float)i * 0.01f); break;                   // sorted descending
        case 6: e[i] = (rng() % 3 == 0) ? 0.f : std::ldexp(1.f, -(int)(rng() % 30)); break;
        default: e[i] = std::ldexp((float)(1 + rng() % 0xffffff), -(int)(rng() % 60)); break;
      }
    }
    if (kind == 2 || kind == 6) s0 = 1.0f;
    if (kind == 7) s0 = std::ldexp(ud(rng), (int)(rng() % 10));
    const int window = 1 + (int)(rng() % 700);
    bad += !run_case(e, s0, window, false);
    bad += !run_case(e, s0, window, true);
    bad += !run_case_groups(e, s0, 1 + window % 64, rep % 3 == 0 ? 16 : 1 + (int)(rng() % 40));
    cases += 3;
  }
  printf("%ld %ld\n", bad, cases);
  return 0;
}
