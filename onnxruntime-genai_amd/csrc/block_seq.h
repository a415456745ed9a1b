// Block-wide drivers built on seq_scan.h: an exact left-to-right fp32 sum (with an optional
// "first index where a predicate on the running prefix holds" search), a double-precision CDF search,
// an in-place bitonic sort, and the exact sampling epilogue shared by the nucleus and general paths.
#pragma once
#include "device_utils.h"
#include "seq_scan.h"

namespace ms {

constexpr int kIntMax = 0x7fffffff;

struct SeqShared {
  Step wave_tot[16];
  int red_a[16];
  int red_b[16];
  double dred[16];
  double dscan[16];
  float s_before, e_cross, result;
  uint32_t n_last;
  int bcast_i;
  double bcast_d;
};

__device__ __forceinline__ Step shfl_up_step(Step x, int d) {
  Step y;
  y.d0 = __shfl_up(x.d0, d, 64);
  y.d1 = __shfl_up(x.d1, d, 64);
  return y;
}

__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const int o = __shfl_xor(v, m, 64);
    v = o < v ? o : v;
  }
  return v;
}

// Minimum of two ints over the block (both reduced at once).  Contains two barriers.
__device__ __forceinline__ void block_min2(int& a, int& b, SeqShared& sh) {
  a = wave_min_i(a);
  b = wave_min_i(b);
  const int lane = lane_id(), wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if (lane == 0) {
    sh.red_a[wave] = a;
    sh.red_b[wave] = b;
  }
  __syncthreads();
  int ra = sh.red_a[0], rb = sh.red_b[0];
  for (int w = 1; w < nw; ++w) {
    ra = sh.red_a[w] < ra ? sh.red_a[w] : ra;
    rb = sh.red_b[w] < rb ? sh.red_b[w] : rb;
  }
  __syncthreads();
  a = ra;
  b = rb;
}

struct NoStop {
  __device__ bool operator()(float, float, int) const { return false; }
};

// Exact value of (((s0 + e(0)) + e(1)) + ... ) in fp32 over i < n, computed by the whole block
// (every thread must call with identical arguments; every thread gets the result).
// If stop(prefix_i, e(i), i) holds for some i -- prefix_i being the sum including e(i) -- the scan
// ends at the first such i: *stop_index = i and the returned value is prefix_i.  Otherwise
// *stop_index = -1 and the value is the full sum.  e(i) must be finite and >= 0.
template <int ITEMS, typename GetE, typename StopFn>
__device__ float block_seq_sum(float s0, int n, GetE get, StopFn stop, int* stop_index, SeqShared& sh) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  float s = s0;
  int i0 = 0, found = -1;
  // Items per thread in the current window.  A window is redone from the element behind a binade
  // change, and those cluster at the start of a sum, so windows start small and double while no
  // change occurs.
  int items = 1;
  while (i0 < n) {
    const SeqState st = seq_decompose(s);
    const int span = static_cast<int>(blockDim.x) * items;
    const int base = i0 + tid * items;
    const int window_end = (n - i0 < span) ? n : i0 + span;
    float ev[ITEMS];
    Step f[ITEMS];
    Step agg{0u, 0u};
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int idx = base + j;
      const bool on = j < items && idx < window_end;
      ev[j] = on ? get(idx) : 0.0f;
      f[j] = seq_make_step(ev[j], st.se);
      agg = step_compose(agg, f[j]);
    }
    Step x = agg;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const Step y = shfl_up_step(x, d);
      if (lane >= d) x = step_compose(y, x);
    }
    if (lane == 63) sh.wave_tot[wave] = x;
    __syncthreads();
    Step ex = shfl_up_step(x, 1);
    if (lane == 0) ex = Step{0u, 0u};
    Step wp{0u, 0u};
    for (int w = 0; w < wave; ++w) wp = step_compose(wp, sh.wave_tot[w]);
    ex = step_compose(wp, ex);
    uint32_t nn = step_apply(st.n, ex);
    int lc = kIntMax, ls = kIntMax;
    float lpf = 0.0f;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int idx = base + j;
      if (j < items && idx < window_end) {
        const uint32_t nn2 = step_apply(nn, f[j]);
        if (nn2 >= kMantLimit) {
          if (nn < kMantLimit) {  // the one addition that leaves the binade
            sh.s_before = seq_recompose(nn, st.se);
            sh.e_cross = ev[j];
          }
          lc = idx < lc ? idx : lc;
        } else {
          const float pf = seq_recompose(nn2, st.se);
          if (ls == kIntMax && stop(pf, ev[j], idx)) {
            ls = idx;
            lpf = pf;
          }
          if (idx == window_end - 1) sh.n_last = nn2;
        }
        nn = nn2;
      }
    }
    int gc = lc, gs = ls;
    block_min2(gc, gs, sh);
    if (gs < gc) {  // predicate satisfied before any binade change
      if (ls == gs) sh.result = lpf;
      __syncthreads();
      s = sh.result;
      found = gs;
      __syncthreads();
      break;
    }
    if (gc == kIntMax) {
      s = seq_recompose(sh.n_last, st.se);
      i0 = window_end;
      if (items < ITEMS) items *= 2;
    } else {
      items = 1;
      const float e_cross = sh.e_cross;
      s = sh.s_before + e_cross;
      if (stop(s, e_cross, gc)) {
        found = gc;
        __syncthreads();
        break;
      }
      i0 = gc + 1;
    }
    __syncthreads();
  }
  *stop_index = found;
  return s;
}

// Position std::discrete_distribution would return for weights w(0..n-1) and canonical draw u
// (libstdc++ random.tcc: normalise by the double sum, partial sums in double, last forced to 1,
// lower_bound).  The reference accumulates those doubles sequentially; here they are reduced and
// scanned in parallel, which can move a cumulative value by at most a few n*2^-53.  If u lies that
// close to any cumulative value the answer is recomputed sequentially, so the result always equals
// the sequential one.
template <int ITEMS, typename GetW>
__device__ int block_discrete_draw(int n, GetW w, double u, SeqShared& sh) {
  if (n < 2) return 0;
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6, nw = blockDim.x >> 6;
  const int span = static_cast<int>(blockDim.x) * ITEMS;
  // total
  double part = 0.0;
  for (int i = tid; i < n; i += blockDim.x) part += static_cast<double>(w(i));
  part = wave_sum<double>(part);
  if (lane == 0) sh.dred[wave] = part;
  __syncthreads();
  double total = 0.0;
  for (int k = 0; k < nw; ++k) total += sh.dred[k];
  __syncthreads();
  const double guard = 16.0 * static_cast<double>(n) * 1.1102230246251565e-16;
  double carry = 0.0;
  int first = kIntMax;
  int risky = 0;
  for (int i0 = 0; i0 < n; i0 += span) {
    const int base = i0 + tid * ITEMS;
    double pv[ITEMS];
    double loc = 0.0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int idx = base + j;
      pv[j] = idx < n ? static_cast<double>(w(idx)) / total : 0.0;
      loc += pv[j];
    }
    double inc = loc;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const double y = __shfl_up(inc, d, 64);
      if (lane >= d) inc += y;
    }
    if (lane == 63) sh.dscan[wave] = inc;
    __syncthreads();
    double wp = carry;
    for (int k = 0; k < wave; ++k) wp += sh.dscan[k];
    double block_total = 0.0;
    for (int k = 0; k < nw; ++k) block_total += sh.dscan[k];
    double run = wp + (inc - loc);
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int idx = base + j;
      if (idx < n) {
        run += pv[j];
        const double cp = (idx == n - 1) ? 1.0 : run;
        if (idx != n - 1 && fabs(cp - u) <= guard) risky = 1;
        if (cp >= u && idx < first) first = idx;
      }
    }
    carry += block_total;
    __syncthreads();
  }
  int a = first, b = risky ? 0 : 1;
  block_min2(a, b, sh);
  if (b != 0) return a;
  // Sequential replay (reached with probability ~ n^2 * 1e-15 per draw).
  if (tid == 0) {
    double sum = 0.0;
    for (int i = 0; i < n; ++i) sum += static_cast<double>(w(i));
    double cp = 0.0;
    int pos = n - 1;
    for (int i = 0; i < n - 1; ++i) {
      cp += static_cast<double>(w(i)) / sum;
      if (cp >= u) {
        pos = i;
        break;
      }
    }
    sh.bcast_i = pos;
  }
  __syncthreads();
  const int pos = sh.bcast_i;
  __syncthreads();
  return pos;
}

// In-place bitonic sort, descending, of n (a power of two) keys in LDS or global memory.
__device__ __forceinline__ void block_sort_desc(u64* a, int n) {
  for (int k = 2; k <= n; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < (n >> 1); t += blockDim.x) {
        const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        const int hi = lo | j;
        const bool desc = (lo & k) == 0;
        const u64 x = a[lo], y = a[hi];
        if ((x < y) == desc) {
          a[lo] = y;
          a[hi] = x;
        }
      }
      __syncthreads();
    }
  }
}

struct RowOutputs {
  int32_t* token;
  int32_t* kept_count;
  int32_t* kept_ids;
  float* kept_probs;
  int kept_capacity;
};

// The reference's ComputeSampledCategorical + SampleCategoricalToken
// (src/sampling_distribution.h:218-297) on a row whose elements are available in rank order:
// sorted(i) returns the key64 of the i-th best element for i < n_sorted.  exps(i) must return
// exp((score_i - score_0) * inv_temp) as a float (callers may cache it).  Returns false -- without
// writing outputs -- when the nucleus does not end inside the n_sorted available elements.
template <int ITEMS, typename Sorted, typename Exps>
__device__ bool block_sample_epilogue(Sorted sorted, Exps exps, int n_sorted, int vocab,
                                      mi355x_sample_params prm, double u, const RowOutputs& out,
                                      SeqShared& sh) {
  int keep;
  float scale;     // kept probability j = base_j * scale, base_j = exps(j) or exps(j)/sum
  float sum = 1.0f;
  bool divide_by_sum = false;
  int idx_dummy;
  if (prm.k > 1) {
    const int m = prm.k < vocab ? prm.k : vocab;
    if (m > n_sorted) return false;
    sum = block_seq_sum<ITEMS>(0.0f, m, exps, NoStop{}, &idx_dummy, sh);
    divide_by_sum = sum > 0.0f;
    const float ssum = sum;
    const bool dv = divide_by_sum;
    auto pr = [=](int i) {
      const float e = exps(i);
      return dv ? e / ssum : e;
    };
    keep = m;
    float keep_sum;
    if (prm.p > 0.0f && prm.p < 1.0f) {
      const float p = prm.p;
      int si;
      keep_sum = block_seq_sum<ITEMS>(0.0f, m, pr, [=](float pf, float, int) { return pf >= p; }, &si, sh);
      if (si >= 0) keep = si + 1;
    } else {
      keep_sum = block_seq_sum<ITEMS>(0.0f, m, pr, NoStop{}, &idx_dummy, sh);
    }
    scale = keep_sum > 0.0f ? 1.0f / keep_sum : 0.0f;
  } else {
    const float p = prm.p;
    const int limit = n_sorted < vocab ? n_sorted : vocab;
    int si;
    const int V = vocab;
    float prefix = block_seq_sum<ITEMS>(
        0.0f, limit, exps,
        [=](float pf, float e, int i) {
          const float tail = static_cast<float>(V - i - 1) * e;
          return pf >= p * (pf + tail);
        },
        &si, sh);
    int cutoff;
    if (si >= 0) {
      cutoff = si + 1;
    } else if (limit == vocab) {
      cutoff = vocab;
    } else {
      return false;
    }
    if (vocab <= 64) {  // exact-partition override, src/sampling_distribution.h:186-203
      if (n_sorted < vocab) return false;
      const float global = block_seq_sum<ITEMS>(0.0f, vocab, exps, NoStop{}, &idx_dummy, sh);
      int sj;
      const float c = block_seq_sum<ITEMS>(0.0f, vocab, exps,
                                           [=](float pf, float, int) { return pf >= p * global; }, &sj, sh);
      (void)c;
      if (sj >= 0) {
        cutoff = sj + 1;
        si = -1;
      }
    }
    if (si < 0 || cutoff != si + 1) prefix = block_seq_sum<ITEMS>(0.0f, cutoff, exps, NoStop{}, &idx_dummy, sh);
    keep = cutoff;
    scale = prefix > 0.0f ? 1.0f / prefix : 0.0f;
  }
  const float fsum = sum;
  const bool dv2 = divide_by_sum;
  const float fscale = scale;
  auto q = [=](int i) {
    const float e = exps(i);
    const float b = dv2 ? e / fsum : e;
    return b * fscale;
  };
  if (out.kept_count && threadIdx.x == 0) *out.kept_count = keep;
  if (out.kept_ids) {
    const int lim = keep < out.kept_capacity ? keep : out.kept_capacity;
    for (int i = threadIdx.x; i < lim; i += blockDim.x) {
      out.kept_ids[i] = static_cast<int32_t>(key64_index(sorted(i)));
      if (out.kept_probs) out.kept_probs[i] = q(i);
    }
  }
  const int pos = block_discrete_draw<ITEMS>(keep, q, u, sh);
  if (threadIdx.x == 0) *out.token = static_cast<int32_t>(key64_index(sorted(pos)));
  return true;
}

}  // namespace ms
