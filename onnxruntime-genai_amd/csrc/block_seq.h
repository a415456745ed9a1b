// Block-wide drivers built on seq_scan.h: an exact left-to-right fp32 sum (with an optional
// "first index where a predicate on the running prefix holds" search), a double-precision CDF search,
// an in-place bitonic sort, and the exact sampling epilogue shared by the nucleus and general paths.
#pragma once
#include <type_traits>
#include <utility>
#include "device_utils.h"
#include "seq_scan.h"
#include "wave_select.h"

namespace ms {

constexpr int kIntMax = 0x7fffffff;

struct SeqShared {
  // block_seq_sum: double-buffered by pass parity so a pass needs two barriers only
  Step wave_tot[2][16];
  uint32_t ev_key[2][16];
  float ev_a[2][16], ev_b[2][16];
  uint32_t n_last[2];
  float head_sum;
  int head_found, head_n;
  // block_discrete_draw / block_min2
  int red_a[16];
  int red_b[16];
  double dred[16];
  double dscan[16];
  int bcast_i;
  double bcast_d;
};

__device__ __forceinline__ int wave_min_i(int v) { return -1 - wave_max<int>(-1 - v); }  // ~v reverses the order of ints

// Minimum of two ints over the block (both reduced at once).  Contains two barriers; the second one lets the next
// call follow at once, and a caller that has no next call before another barrier saves it (reuse_at_once = false).
__device__ __forceinline__ void block_min2(int& a, int& b, SeqShared& sh, bool reuse_at_once = true) {
  a = wave_min_i(a);
  b = wave_min_i(b);
  const int lane = lane_id(), wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if (lane == 0) {
    sh.red_a[wave] = a;
    sh.red_b[wave] = b;
  }
  __syncthreads();
  // lane w looks at wave w's pair (at most sixteen waves); ~v reverses the order of ints
  const int ra = -1 - row16_max<int>(-1 - (lane < nw ? sh.red_a[lane] : kIntMax));
  const int rb = -1 - row16_max<int>(-1 - (lane < nw ? sh.red_b[lane] : kIntMax));
  if (reuse_at_once) __syncthreads();
  a = ra;
  b = rb;
}

// Value of the lane `d` below (row_shr inside a row of 16, then the row broadcasts), 0 where there
// is no such lane: 0/0 is the identity Step, so the scan below needs no lane tests.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ Step step_from_below(Step x) {
  Step y;
  y.d0 = __builtin_amdgcn_update_dpp(0u, x.d0, CTRL, ROW_MASK, 0xf, false);
  y.d1 = __builtin_amdgcn_update_dpp(0u, x.d1, CTRL, ROW_MASK, 0xf, false);
  return y;
}

// Inclusive scan of Steps over the wave (lane order), data-parallel-primitive moves only.
__device__ __forceinline__ Step wave_scan_steps(Step x) {
  x = step_compose(step_from_below<0x111, 0xf>(x), x);  // row_shr:1
  x = step_compose(step_from_below<0x112, 0xf>(x), x);  // row_shr:2
  x = step_compose(step_from_below<0x114, 0xf>(x), x);  // row_shr:4
  x = step_compose(step_from_below<0x118, 0xf>(x), x);  // row_shr:8
  x = step_compose(step_from_below<0x142, 0xa>(x), x);  // row_bcast:15 into rows 1 and 3
  x = step_compose(step_from_below<0x143, 0xc>(x), x);  // row_bcast:31 into rows 2 and 3
  return x;
}

// The same scan, starting afresh at the lanes that hold their own index in h (the others hold -1; lane 0 must
// start a run): x ends as the composition from the run's first lane up to this lane, h as that first lane.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void segscan_level(Step& x, int& h) {
  const Step below = step_from_below<CTRL, ROW_MASK>(x);
  const int h_below = dpp_from_below_or<CTRL, ROW_MASK, int>(-1, h);
  const Step joined = step_compose(below, x);
  const bool starts = h >= 0;  // the lanes covered so far already hold a run's first lane
  x.d0 = starts ? x.d0 : joined.d0;
  x.d1 = starts ? x.d1 : joined.d1;
  h = starts ? h : h_below;
}
__device__ __forceinline__ void wave_segscan_steps(Step& x, int& h) {
  segscan_level<0x111, 0xf>(x, h);  // row_shr:1
  segscan_level<0x112, 0xf>(x, h);  // row_shr:2
  segscan_level<0x114, 0xf>(x, h);  // row_shr:4
  segscan_level<0x118, 0xf>(x, h);  // row_shr:8
  segscan_level<0x142, 0xa>(x, h);  // row_bcast:15 into rows 1 and 3
  segscan_level<0x143, 0xc>(x, h);  // row_bcast:31 into rows 2 and 3
}

// Composition over groups of four lanes: lanes 3, 7, 11, ... end with the composition of their group.
__device__ __forceinline__ Step quad_scan_steps(Step x) {
  x = step_compose(step_from_below<0x111, 0xf>(x), x);  // row_shr:1
  x = step_compose(step_from_below<0x112, 0xf>(x), x);  // row_shr:2
  return x;
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) { return ~wave_max<uint32_t>(~v); }

// Fetches the ITEMS consecutive addends thread t owns in the window [w0, wend): indices
// w0 + t*ITEMS + j.  Asking get() for them directly makes every lane walk its own 4*ITEMS-byte strip of
// global memory, which wastes most of every cache line fetched; with a staging buffer in LDS
// (blockDim * ITEMS floats) the window is read with consecutive lanes on consecutive indices and
// transposed through LDS instead.  Contains one barrier when staging; the caller's next barrier
// separates these LDS reads from the next window's writes.
template <int ITEMS, typename GetE>
__device__ __forceinline__ void window_fetch(float (&ev)[ITEMS], int w0, int wend, GetE get, float* stage) {
  const int tid = threadIdx.x, bd = static_cast<int>(blockDim.x);
  if (stage == nullptr) {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) ev[j] = (w0 + tid * ITEMS + j < wend) ? get(w0 + tid * ITEMS + j) : 0.0f;
    return;
  }
  float tmp[ITEMS];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) tmp[j] = (w0 + j * bd + tid < wend) ? get(w0 + j * bd + tid) : 0.0f;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) stage[j * bd + tid] = tmp[j];
  __syncthreads();
  if constexpr (ITEMS % 4 == 0) {
#pragma unroll
    for (int j = 0; j < ITEMS; j += 4) {
      const float4 q = *reinterpret_cast<const float4*>(stage + tid * ITEMS + j);
      ev[j] = q.x, ev[j + 1] = q.y, ev[j + 2] = q.z, ev[j + 3] = q.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) ev[j] = stage[tid * ITEMS + j];
  }
}

// Serial prefix over lanes: out[l] = ((x[0] + x[1]) + ...) + x[l], additions in lane order, as the
// reference's scalar loops do.  One DPP-shifted add per element (wave_shr:1, lane 0 reads 0).
// Steps run in unrolled groups of 8: a step past `count` leaves lanes below `count` unchanged.
__device__ __forceinline__ float wave_serial_prefix(float x, int count) {
  float s = 0.0f;
  for (int t = 0; t < count; t += 8) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float prev = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(s), 0x138, 0xf, 0xf, false));
      s = prev + x;
    }
  }
  return s;
}

__device__ __forceinline__ double wave_serial_prefix(double x, int count) {
  double s = 0.0;
  for (int t = 0; t < count; t += 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const u64 b = static_cast<u64>(__double_as_longlong(s));
      const uint32_t lo = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b), 0x138, 0xf, 0xf, false);
      const uint32_t hi = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b >> 32), 0x138, 0xf, 0xf, false);
      const double prev = __longlong_as_double(static_cast<long long>((static_cast<u64>(hi) << 32) | lo));
      s = prev + x;
    }
  }
  return s;
}

struct NoStop {
  __device__ bool operator()(float, float, int) const { return false; }
};

// A stop predicate may also say that it holds nowhere in a run of consecutive addends, judged at the run's last
// element: bool nowhere_in_run_ending(prefix, addend, index).  It must only say so when that is certain.
template <typename StopFn, typename = void>
struct StopSettlesRuns : std::false_type {};
template <typename StopFn>
struct StopSettlesRuns<StopFn, decltype(void(std::declval<const StopFn&>().nowhere_in_run_ending(0.0f, 0.0f, 0)))>
    : std::true_type {};

// Stops at the first prefix that reaches a fixed mass.  Prefixes do not decrease, so a run whose last prefix is
// below the mass holds no stop.
struct StopAtMass {
  float mass;
  __device__ __forceinline__ bool operator()(float pf, float, int) const { return pf >= mass; }
  __device__ __forceinline__ bool nowhere_in_run_ending(float pf, float, int) const { return pf < mass; }
};

// FindNucleus' stop (src/sampling_distribution.h:164-174) over addends in descending order: the prefix reaches
// p times (prefix + the bound (vocab - i - 1) * addend on what follows).  In exact arithmetic prefix - p * (prefix +
// bound) does not decrease along the row (prefixes do not decrease, addends and counts do not increase); the
// float evaluation is within a few 2^-24 of it, so a run whose last element misses the stop by more than 2^-18 of
// the right-hand side holds none.
struct StopAtNucleus {
  float p;
  int vocab, offset;  // the addend's rank in the row is its index + offset
  __device__ __forceinline__ bool operator()(float pf, float e, int i) const {
    const float tail = static_cast<float>(vocab - (i + offset) - 1) * e;
    return pf >= p * (pf + tail);
  }
  __device__ __forceinline__ bool nowhere_in_run_ending(float pf, float e, int i) const {
    const float tail = static_cast<float>(vocab - (i + offset) - 1) * e;
    return pf < (p * (pf + tail)) * 0.99999619f;  // 1 - 2^-18
  }
};

// Exact value of (((s0 + e(0)) + e(1)) + ... ) in fp32 over i < n, computed by the whole block
// (every thread must call with identical arguments; every thread gets the result).
// If stop(prefix_i, e(i), i) holds for some i -- prefix_i being the sum including e(i) -- the scan
// ends at the first such i: *stop_index = i and the returned value is prefix_i.  Otherwise
// *stop_index = -1 and the value is the full sum.  e(i) must be finite and >= 0.
//
// The addends of a window (blockDim * ITEMS elements) are evaluated once and kept in registers.  A
// pass scans the part of the window not yet folded into the sum under the sum's current binade and
// finds the first event: the addition that leaves the binade (done with a real float add, after
// which the rest of the window is scanned again under the new binade) or the first index where the
// predicate holds.  Passes cost two barriers; there is one per window plus one per binade change.
template <int ITEMS, typename GetE, typename StopFn>
__device__ float block_seq_sum(float s0, int n, GetE get, StopFn stop, int* stop_index, SeqShared& sh,
                               float* stage = nullptr, int head = 0, bool synced = false) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6, nw = static_cast<int>(blockDim.x) >> 6;
  const int span = static_cast<int>(blockDim.x) * ITEMS;
  constexpr uint32_t kNone = 0xffffffffu;
  float s = s0;
  int found = -1;
  int par = 0;
  if (!synced) __syncthreads();  // a previous call's readers are done with the parity-0 buffers (synced: the caller vouches)
  // A sum that starts from nothing changes binade every few additions, and each change costs a pass
  // of the scan below.  The first `head` elements are therefore added for real, 64 at a time, by a
  // chain of lane-shifted float additions in wave 0 (about ten cycles per element).  The head ends early once 64
  // elements have added less than an eighth to the sum: from there on a binade is left rarely, and the other waves
  // wait while the head runs.
  int n_head = 0;
  if (head > 0) {
    n_head = head < n ? head : n;
    if (wave == 0) {
      float carry = s0;
      int fnd = -1, done = n_head;
      float x_next = lane < n_head ? get(lane) : 0.0f;
      for (int r0 = 0; r0 < n_head && fnd < 0; r0 += 64) {
        const float x = x_next;
        const int idx = r0 + lane;
        x_next = idx + 64 < n_head ? get(idx + 64) : 0.0f;  // in flight during the chain of the current 64 elements
        const float sp = wave_serial_prefix(lane == 0 ? carry + x : x, 64);
        const unsigned long long hit = __ballot(idx < n_head && stop(sp, x, idx));
        if (hit != 0ull) {
          const int l = __ffsll(static_cast<long long>(hit)) - 1;
          fnd = r0 + l;
          carry = wave_read_lane(sp, l);
        } else {
          const float before = carry;
          carry = wave_read_lane(sp, 63);  // lanes past the end added zeros
          if (carry - before <= 0.125f * carry && r0 + 64 < n_head) {
            done = r0 + 64;
            break;
          }
        }
      }
      if (lane == 0) {
        sh.head_sum = carry;
        sh.head_found = fnd;
        sh.head_n = done;
      }
    }
    __syncthreads();
    s = sh.head_sum;
    found = sh.head_found;
    n_head = sh.head_n;
  }
  for (int w0 = n_head; w0 < n && found < 0; w0 += span) {
    const int base = w0 + tid * ITEMS;
    const int wend = (n - w0 < span) ? n : w0 + span;
    float ev[ITEMS];
    window_fetch<ITEMS>(ev, w0, wend, get, stage);
    int start = w0;  // first index not yet folded into s
    while (true) {
      const SeqState st = seq_decompose(s);
      // the thread's addends that are still to be folded in (the others count as zeros), composed into one step
      float live[ITEMS];
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) live[j] = (base + j >= start && base + j < wend) ? ev[j] : 0.0f;
      const Step agg = seq_compose_run(live, ITEMS, st.se);
      const Step inc = wave_scan_steps(agg);
      if (lane == 63) sh.wave_tot[par][wave] = inc;
      __syncthreads();
      Step ex = step_from_below<0x138, 0xf>(inc);  // wave_shr:1, identity into lane 0
      // composition of the waves before this one: lane l takes wave l's total, four scan levels cover the at most
      // 16 waves, and this wave reads lane wave - 1
      Step wt = lane < nw ? sh.wave_tot[par][lane] : Step{0u, 0u};
      wt = step_compose(step_from_below<0x111, 0xf>(wt), wt);  // row_shr:1
      wt = step_compose(step_from_below<0x112, 0xf>(wt), wt);  // row_shr:2
      wt = step_compose(step_from_below<0x114, 0xf>(wt), wt);  // row_shr:4
      wt = step_compose(step_from_below<0x118, 0xf>(wt), wt);  // row_shr:8
      Step wp{0u, 0u};
      if (wave > 0) {
        wp.d0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wt.d0), wave - 1));
        wp.d1 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wt.d1), wave - 1));
      }
      ex = step_compose(wp, ex);
      uint32_t nn = step_apply(st.n, ex);
      uint32_t key = kNone;
      float pa = 0.0f, pb = 0.0f;
      // Without a stop predicate only a binade change is of interest, and a thread whose last
      // prefix is still inside the binade (prefixes never decrease) has none among its elements.
      constexpr bool kPlain = std::is_same<StopFn, NoStop>::value;
      const uint32_t nn_end = step_apply(nn, agg);
      bool walk = true;
      if (nn_end < kMantLimit) {
        if constexpr (kPlain) {
          nn = nn_end;
          walk = false;
        } else if constexpr (StopSettlesRuns<StopFn>::value) {
          // A thread whose addends are all live and stay inside the binade asks its predicate about the run as a
          // whole: nowhere true (judged at the run's last element), or true at its first element already, which
          // is then the thread's event; only the thread in which the predicate turns true walks its elements.
          if (base >= start && base + ITEMS <= wend) {
            if (stop.nowhere_in_run_ending(seq_recompose(nn_end, st.se), ev[ITEMS - 1], base + ITEMS - 1)) {
              nn = nn_end;
              walk = false;
            } else {
              const float p1 = seq_recompose(step_apply(nn, seq_make_step(ev[0], st.se)), st.se);
              if (stop(p1, ev[0], base)) {
                key = static_cast<uint32_t>(base) << 1;
                pa = p1;
                nn = nn_end;
                walk = false;
              }
            }
          }
        }
      }
      if (walk) {
        // From the exact prefix in front of the thread's elements the walk is the reference's own loop: real float
        // additions, one per element (the step functions exist to compose runs in parallel; a thread that walks has
        // its start).  A sum whose bit pattern reaches the next binade's first has left the binade.
        const uint32_t lim = (static_cast<uint32_t>(st.se) << 23) + 0x800000u;
        bool gone = nn >= kMantLimit;  // an earlier thread's element left the binade already
        float s_run = seq_recompose(gone ? 0u : nn, st.se);
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
          const int idx = base + j;
          if (idx >= start && idx < wend) {
            const float s_next = s_run + ev[j];
            const bool leaves = gone || em::as_u32(s_next) >= lim;
            if (key == kNone) {
              if (leaves) {  // leaves the binade here (or an earlier thread's element did)
                key = (static_cast<uint32_t>(idx) << 1) | 1u;
                pa = s_run;
                pb = ev[j];
              } else if (!kPlain) {
                if (stop(s_next, ev[j], idx)) {
                  key = static_cast<uint32_t>(idx) << 1;
                  pa = s_next;
                }
              }
            }
            gone = leaves;
            s_run = s_next;
          }
        }
        nn = gone ? kStepSat : seq_decompose(s_run).n;
      }
      if (wend - 1 >= base && wend - 1 < base + ITEMS) sh.n_last[par] = nn;
      const uint32_t wkey = wave_min_u32(key);
      if (key == wkey && (key != kNone || lane == 0)) {
        sh.ev_key[par][wave] = key;
        sh.ev_a[par][wave] = pa;
        sh.ev_b[par][wave] = pb;
      }
      __syncthreads();
      // the first event of the block: lane l looks at wave l's (event keys are distinct: they carry the index)
      const uint32_t k2 = lane < nw ? sh.ev_key[par][lane] : kNone;
      const uint32_t gk = wave_min_u32(k2);
      const int from = __ffsll(static_cast<long long>(__ballot(k2 == gk))) - 1;  // 0 when there is no event
      const float ga = sh.ev_a[par][from], gb = sh.ev_b[par][from];
      const uint32_t n_last = sh.n_last[par];
      par ^= 1;
      if (gk == kNone) {  // the rest of the window stayed inside the binade
        s = seq_recompose(n_last, st.se);
        break;
      }
      const int at = static_cast<int>(gk >> 1);
      if ((gk & 1u) == 0u) {  // predicate satisfied before any binade change
        s = ga;
        found = at;
        break;
      }
      s = ga + gb;  // the one addition that leaves the binade
      if (stop(s, gb, at)) {
        found = at;
        break;
      }
      start = at + 1;
      if (start >= wend) break;
    }
  }
  *stop_index = found;
  return s;
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_from_below(double x) {
  const u64 b = static_cast<u64>(__double_as_longlong(x));
  const uint32_t lo = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b), CTRL, ROW_MASK, 0xf, false);
  const uint32_t hi = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b >> 32), CTRL, ROW_MASK, 0xf, false);
  return __longlong_as_double(static_cast<long long>((static_cast<u64>(hi) << 32) | lo));
}

// Inclusive prefix sums over the wave in tree order (lanes without a source add +0.0).
__device__ __forceinline__ double wave_scan_add(double x) {
  x += dpp_from_below<0x111, 0xf>(x);  // row_shr:1
  x += dpp_from_below<0x112, 0xf>(x);  // row_shr:2
  x += dpp_from_below<0x114, 0xf>(x);  // row_shr:4
  x += dpp_from_below<0x118, 0xf>(x);  // row_shr:8
  x += dpp_from_below<0x142, 0xa>(x);  // row_bcast:15 into rows 1 and 3
  x += dpp_from_below<0x143, 0xc>(x);  // row_bcast:31 into rows 2 and 3
  return x;
}

// Inclusive prefix sums inside every row of sixteen lanes (enough where only the first sixteen lanes hold values).
__device__ __forceinline__ double row_scan_add(double x) {
  x += dpp_from_below<0x111, 0xf>(x);  // row_shr:1
  x += dpp_from_below<0x112, 0xf>(x);  // row_shr:2
  x += dpp_from_below<0x114, 0xf>(x);  // row_shr:4
  x += dpp_from_below<0x118, 0xf>(x);  // row_shr:8
  return x;
}

// One thread's share of the search for the first cumulative value that reaches `target`: its weights pv follow a
// cumulative value of `before` and sum to `loc`.  first = the lowest index whose cumulative value reaches the target
// (the last index always does: its value is forced to 1); risky = some cumulative value other than the last lies
// within `guard` of the target.  Most threads lie entirely on one side of the target by more than the guard and
// settle that from their two end values: the additions of a thread's weights in another order differ from these
// by less than the guard (it counts sixteen roundings per weight of the whole distribution), hence the factor two.
template <int ITEMS>
__device__ __forceinline__ void draw_scan_thread(const double (&pv)[ITEMS], double before, double loc, int base, int n,
                                                 double target, double guard, int& first, int& risky) {
  if (base >= n) return;
  if (before + loc < target - 2.0 * guard) {  // all below the target
    if (base + ITEMS >= n && n - 1 < first) first = n - 1;
    return;
  }
  if (before > target + 2.0 * guard) {  // all above it
    if (base < first) first = base;
    return;
  }
  double run = before;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const int idx = base + j;
    if (idx < n) {
      run += pv[j];
      if (idx != n - 1 && fabs(run - target) <= guard) risky = 1;
      if ((idx == n - 1 || run >= target) && idx < first) first = idx;  // the last value is forced to 1
    }
  }
}

// Position std::discrete_distribution would return for weights w(0..n-1) and canonical draw u
// (libstdc++ random.tcc: normalise by the double sum, partial sums in double, last forced to 1,
// lower_bound).  The reference divides every weight by the sum and accumulates the quotients
// sequentially; here the raw weights are reduced and scanned in parallel and compared with u * sum,
// which differs from the reference's cumulative values by at most a few n*2^-53 (relative to the
// sum).  If u lies that close to any cumulative value the answer is recomputed sequentially with the
// reference's own operations, so the result always equals the sequential one.
template <int ITEMS, typename GetW>
__device__ int block_discrete_draw(int n, GetW w, double u, SeqShared& sh, float* stage = nullptr) {
  if (n < 2) return 0;
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6, nw = blockDim.x >> 6;
  const int span = static_cast<int>(blockDim.x) * ITEMS;
  // The total comes first unless the whole distribution fits one window: then the window's own scan supplies it
  // (any summation order will do: the guard band below covers the difference).
  const bool single = n <= span;
  double total = 0.0;
  if (!single) {
    double part = 0.0;
#pragma unroll 8
    for (int i = tid; i < n; i += blockDim.x) part += static_cast<double>(w(i));
    part = wave_sum<double>(part);
    if (lane == 0) sh.dred[wave] = part;
    __syncthreads();
    for (int k = 0; k < nw; ++k) total += sh.dred[k];
    __syncthreads();
    // A NaN weight (a row of -inf logits gives exp(-inf - -inf)) makes every quotient w/sum NaN; the
    // binary search of std::discrete_distribution over NaNs and the forced final 1.0 ends on 0.
    if (total != total) return 0;
  }
  double guard = 16.0 * static_cast<double>(n) * 1.1102230246251565e-16 * total;
  double target = u * total;
  double carry = 0.0;
  int first = kIntMax;
  int risky = 0;
  for (int i0 = 0; i0 < n; i0 += span) {
    const int base = i0 + tid * ITEMS;
    double pv[ITEMS];
    double loc = 0.0;
    {
      float wv[ITEMS];
      window_fetch<ITEMS>(wv, i0, (n - i0 < span) ? n : i0 + span, w, stage);
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) {
        pv[j] = static_cast<double>(wv[j]);
        loc += pv[j];
      }
    }
    const double inc = wave_scan_add(loc);  // lane-shifting additions: the general lane shuffles go through LDS
    if (lane == 63) sh.dscan[wave] = inc;
    __syncthreads();
    // sums of the waves before this one and of the whole window: lane k takes wave k's sum
    const double ws = row_scan_add(lane < nw ? sh.dscan[lane] : 0.0);
    const double block_total = wave_read_lane(ws, nw - 1);
    const double wp = carry + (wave > 0 ? wave_read_lane(ws, wave - 1) : 0.0);
    if (single) {
      total = block_total;
      if (total != total) return 0;  // NaN weights, as above (every thread holds the same total)
      guard = 16.0 * static_cast<double>(n) * 1.1102230246251565e-16 * total;
      target = u * total;
    }
    draw_scan_thread<ITEMS>(pv, wp + (inc - loc), loc, base, n, target, guard, first, risky);
    carry += block_total;
    if (i0 + span < n) __syncthreads();  // (the next window writes the waves' sums again; after the last one nothing does)
  }
  int a = first, b = risky ? 0 : 1;
  block_min2(a, b, sh, false);  // (the one reduction of a draw; the replay below has barriers of its own)
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
template <typename Key>
__device__ __forceinline__ void block_sort_desc(Key* a, int n) {
  for (int k = 2; k <= n; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < (n >> 1); t += blockDim.x) {
        const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        const int hi = lo | j;
        const bool desc = (lo & k) == 0;
        const Key x = a[lo], y = a[hi];
        if ((x < y) == desc) {
          a[lo] = y;
          a[hi] = x;
        }
      }
      __syncthreads();
    }
  }
}

// Compare-exchange of two keys held by one thread; `a` has the lower index.
__device__ __forceinline__ void key_cmpx(u64& a, u64& b, bool desc) {
  const bool sw = (a < b) == desc;
  const u64 t = sw ? b : a;
  b = sw ? a : b;
  a = t;
}

template <int M, int R>
__device__ __forceinline__ void wave_key_exchange(u64 (&x)[R], bool keep_max) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const u64 y = lane_xor64<M>(x[r]);
    x[r] = ((y > x[r]) == keep_max) ? y : x[r];
  }
}

// Bitonic sort, descending, of 1024*R keys in LDS by a block of 1024 threads, with the keys held in
// registers: thread t owns the keys of indices t*R .. t*R+R-1.  Exchange distances below R stay
// inside a thread, distances below 64*R cross lanes with data-parallel-primitive moves, and only the
// ten stages with larger distances go through LDS.
template <int R>
__device__ __noinline__ void block_sort_desc_regs(u64* lds) {
  constexpr int kT = 1024;
  const int t = threadIdx.x;
  u64 x[R];
#pragma unroll
  for (int r = 0; r < R; ++r) x[r] = lds[r * kT + t];  // any order of the unsorted input will do
  __syncthreads();
#pragma unroll
  for (int k = 2; k <= R; k <<= 1) {
#pragma unroll
    for (int j = k >> 1; j >= 1; j >>= 1) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if ((r & j) == 0) key_cmpx(x[r], x[r | j], k < R ? (r & k) == 0 : (t & 1) == 0);
    }
  }
  for (int kt = 2; kt <= kT; kt <<= 1) {
    const bool desc = (t & kt) == 0;
    for (int jt = kt >> 1; jt >= 1; jt >>= 1) {
      const bool keep_max = ((t & jt) == 0) == desc;
      if (jt >= 64) {
#pragma unroll
        for (int r = 0; r < R; ++r) lds[r * kT + t] = x[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const u64 y = lds[r * kT + (t ^ jt)];
          x[r] = ((y > x[r]) == keep_max) ? y : x[r];
        }
        __syncthreads();
      } else if (jt == 32) {
        wave_key_exchange<32, R>(x, keep_max);
      } else if (jt == 16) {
        wave_key_exchange<16, R>(x, keep_max);
      } else if (jt == 8) {
        wave_key_exchange<8, R>(x, keep_max);
      } else if (jt == 4) {
        wave_key_exchange<4, R>(x, keep_max);
      } else if (jt == 2) {
        wave_key_exchange<2, R>(x, keep_max);
      } else {
        wave_key_exchange<1, R>(x, keep_max);
      }
    }
#pragma unroll
    for (int j = R >> 1; j >= 1; j >>= 1) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if ((r & j) == 0) key_cmpx(x[r], x[r | j], desc);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) lds[t * R + r] = x[r];
  __syncthreads();
}

constexpr int kEpiHead = 256;  // elements of every epilogue sum added by the serial head

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
// writing outputs -- when the nucleus does not end inside the n_sorted available elements.  synced: every thread
// has passed a barrier since `sh` was last used, so the first sum need not begin with one.
template <int ITEMS, typename Sorted, typename Exps>
__device__ __forceinline__ bool block_sample_epilogue(Sorted sorted, Exps exps, int n_sorted, int vocab,
                                      mi355x_sample_params prm, double u, const RowOutputs& out,
                                      SeqShared& sh, bool synced = false) {
  int keep;
  float scale;     // kept probability j = base_j * scale, base_j = exps(j) or exps(j)/sum
  float sum = 1.0f;
  bool divide_by_sum = false;
  int idx_dummy;
  if (prm.k > 1) {
    const int m = prm.k < vocab ? prm.k : vocab;
    if (m > n_sorted) return false;
    sum = block_seq_sum<ITEMS>(0.0f, m, exps, NoStop{}, &idx_dummy, sh, nullptr, kEpiHead, synced);
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
      keep_sum = block_seq_sum<ITEMS>(0.0f, m, pr, StopAtMass{p}, &si, sh, nullptr, kEpiHead);
      if (si >= 0) keep = si + 1;
    } else {
      keep_sum = block_seq_sum<ITEMS>(0.0f, m, pr, NoStop{}, &idx_dummy, sh, nullptr, kEpiHead);
    }
    scale = keep_sum > 0.0f ? 1.0f / keep_sum : 0.0f;
  } else {
    const float p = prm.p;
    const int limit = n_sorted < vocab ? n_sorted : vocab;
    const int V = vocab;
    // The reference sorts in batches that end at 16, 64, 256, ... elements and recognises a stop
    // only when it lies strictly inside a batch (src/sampling_distribution.h:166-181): a stop
    // on the last element of a batch smaller than the row is missed and the search goes on in
    // the next batch with the running sum it has.
    int base = 0;
    int cutoff;
    float prefix = 0.0f;
    bool prefix_is_keep_sum = true;
    for (;;) {
      const int b = base;
      int si;
      prefix = block_seq_sum<ITEMS>(prefix, limit - b, [=](int i) { return exps(i + b); }, StopAtNucleus{p, V, b}, &si, sh,
                                    nullptr, b == 0 ? kEpiHead : 0, synced && b == 0);
      if (si < 0) {
        if (limit != vocab) return false;
        cutoff = vocab;
        break;
      }
      cutoff = b + si + 1;
      const bool batch_end = cutoff >= 16 && (cutoff & (cutoff - 1)) == 0 && ((__ffs(cutoff) - 1) & 1) == 0;
      if (!batch_end || cutoff >= vocab) break;
      if (cutoff >= limit) return false;
      base = cutoff;
    }
    if (vocab <= 64) {  // exact-partition override, src/sampling_distribution.h:186-203
      if (n_sorted < vocab) return false;
      const float global = block_seq_sum<ITEMS>(0.0f, vocab, exps, NoStop{}, &idx_dummy, sh, nullptr, kEpiHead);
      int sj;
      const float c = block_seq_sum<ITEMS>(0.0f, vocab, exps, StopAtMass{p * global}, &sj, sh, nullptr, kEpiHead);
      (void)c;
      if (sj >= 0) {
        cutoff = sj + 1;
        prefix_is_keep_sum = false;
      }
    }
    if (!prefix_is_keep_sum) prefix = block_seq_sum<ITEMS>(0.0f, cutoff, exps, NoStop{}, &idx_dummy, sh, nullptr, kEpiHead);
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
