// The launch that writes a segment's exponentials and its step record (see seqsum_kernels.hip), as a template so
// that a caller can give the workgroups something to do while they wait for the earlier segments' sums.
#pragma once
#include "kernels.h"
#include "block_seq.h"
#include "seg_io.h"
#include "wave_select.h"

namespace ms {

__device__ __forceinline__ float row_max_of_segments(const SeqSumArgs& a, int row, uint32_t* red) {
  uint32_t m = 0u;
  for (int s = threadIdx.x; s < a.segs; s += blockDim.x) {
    const uint32_t k = a.seg_max[static_cast<size_t>(row) * a.segs + s];
    m = k > m ? k : m;
  }
  return key_to_float(block_max<uint32_t>(m, red));
}

// A segment sum that has not been written yet: all bits set, a NaN no sum can be (sums of exponentials are
// finite, and a NaN that came in through the logits keeps zeros in its low bits when widened to double).  The
// buffer holds this value everywhere between launches: the walk puts it back.
constexpr unsigned long long kSumNotReady = ~0ull;

__device__ __forceinline__ unsigned long long load_sum_bits(const double* p) {
  return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_sum_bits(double* p, unsigned long long bits) {
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Expected relative distance between the float the reference holds after adding `count` non-negative
// terms one by one and their exact sum: roundings mostly cancel, so it grows like sqrt(count) * 2^-24
// (the worst case grows like count * 2^-24).  Only an estimate is needed: a segment classified on a
// wrong estimate fails the walk's check and is scanned.
__device__ __forceinline__ double seq_drift(int count) {
  return (8.0 * sqrt(static_cast<double>(count)) + 8.0) * 6.0e-8;
}

// Steps 2 and 3 in one launch.  A segment's workgroup writes its exponentials and publishes their double sum;
// then it waits for the sums of the row's earlier segments, which earlier workgroups of the same launch publish
// (workgroups start in index order and a row's segments are consecutive indices, so whatever a workgroup waits for
// is running or done), and goes on with its step record from the exponentials it still holds.  A wait that gives
// up only costs time: the segment is recorded as one whose parts the walk adds element by element.
//
// `between(v, seg, row)` runs, in all threads, after the sum is out and before the earlier sums are needed: work
// on the segment's elements v (as loaded: zeros past the end of the row) that would otherwise wait for a launch of
// its own.
// FULL: the segment lies inside the row (all but a row's last segment do), so nothing has to ask where the row ends.
// `Shared` is what it needs of LDS (declared once, by the kernel, for both forms of the body).
struct NothingBetween {
  struct Shared {};
  template <bool FULL>
  __device__ __forceinline__ void run(Shared&, const float (&)[kSegPer], int, int) const {}
};

struct ExpStepShared {
  uint32_t red[4];
  double dred[4];
  uint64_t exp_tab[32];  // the table of expf in LDS: a lookup per element from constant memory is a gather
  __align__(16) float stage[kSegElems];  // the segment's exponentials in element order
  Step wave_tot[4];
  double wave_parts[4];
};

template <typename InT, typename Between, bool FULL>
__device__ __forceinline__ void seqsum_exp_step_body(const SeqSumArgs& a, const Between& between, ExpStepShared& sh,
                                                     typename Between::Shared& between_sh) {
  uint32_t* const red = sh.red;
  double* const dred = sh.dred;
  uint64_t* const exp_tab = sh.exp_tab;
  float* const stage = sh.stage;
  Step* const wave_tot = sh.wave_tot;
  double* const wave_parts = sh.wave_parts;
  const int seg = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const InT* x = static_cast<const InT*>(a.x) + static_cast<size_t>(row) * a.row_stride;
  float v[kSegPer];
  seg_load<InT>(x, FULL ? (seg + 1) * kSegElems : a.vocab, seg, 0.0f, v);
  if (tid < 32) exp_tab[tid] = em::exp2_tab(static_cast<uint32_t>(tid));
  const float max_score = row_max_of_segments(a, row, red);  // its barriers also publish the table
  const uint64_t* const tab = exp_tab;
  auto lds_tab = [=](uint32_t i) { return tab[i]; };
  float* erow = a.e + static_cast<size_t>(row) * a.e_stride;
  const int first = seg * kSegElems;
  double part = 0.0;
  // four consecutive exponentials per store (the row of exponentials starts 16-byte aligned and a thread's ids come
  // in aligned groups of four); a group that crosses the end of the row is stored element by element
#pragma unroll
  for (int e0 = 0; e0 < kSegPer; e0 += 4) {
    const int idx = seg_index<InT>(seg, e0);
    float ex[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      ex[c] = (FULL || idx + c < a.vocab) ? em::expf_core((v[e0 + c] - max_score) * a.inv_temp, lds_tab) : 0.0f;
      part += static_cast<double>(ex[c]);
    }
    v4f q;
    q.x = ex[0], q.y = ex[1], q.z = ex[2], q.w = ex[3];
    *reinterpret_cast<v4f*>(stage + (idx - first)) = q;
    if (FULL || idx + 4 <= a.vocab) {
      *reinterpret_cast<v4f*>(erow + idx) = q;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (idx + c < a.vocab) erow[idx + c] = ex[c];
    }
  }
  part = wave_sum<double>(part);
  if (lane == 0) dred[wave] = part;
  __syncthreads();  // (the staged exponentials are complete, too)
  const double own = (dred[0] + dred[1]) + (dred[2] + dred[3]);
  double* sums = a.seg_sum + static_cast<size_t>(row) * a.segs;
  if (tid == 0) store_sum_bits(sums + seg, static_cast<unsigned long long>(__double_as_longlong(own)));
  between.template run<FULL>(between_sh, v, seg, row);
  // the sums of the segments before this one
  double before = 0.0;
  bool gave_up = false;
  for (int sg = tid; sg < seg; sg += kSegBlock) {
    unsigned long long bits = load_sum_bits(sums + sg);
    for (int spins = 0; bits == kSumNotReady && spins < a.poll_limit; ++spins) {
      __builtin_amdgcn_s_sleep(1);
      bits = load_sum_bits(sums + sg);
    }
    if (bits == kSumNotReady) gave_up = true;
    else before += __longlong_as_double(static_cast<long long>(bits));
  }
  gave_up = __syncthreads_or(gave_up ? 1 : 0) != 0;  // (also: every thread has read dred)
  before = wave_sum<double>(before);
  if (lane == 0) dred[wave] = before;
  __syncthreads();
  before = (dred[0] + dred[1]) + (dred[2] + dred[3]);
  const int n = FULL ? kSegElems : a.vocab - first;
  int4* rec = a.seg_step + static_cast<size_t>(row) * a.segs + seg;
  if (gave_up) {
    if (tid < kSegSubs) a.sub_se[(static_cast<size_t>(row) * a.segs + seg) * kSegSubs + tid] = -1;
    if (tid == 0) {
      *rec = make_int4(0, 0, -2, 0);
      atomicAdd(a.gave_up, 1u);
    }
    return;
  }
  const double lo = before * (1.0 - seq_drift(first));
  const double hi = (before + own) * (1.0 + seq_drift(first + n));
  const float lo_f = __double2float_rd(lo), hi_f = __double2float_ru(hi);
  const int se = seq_decompose(lo_f).se;
  const bool known = lo_f > 0.0f && hi_f < 3.0e38f && seq_decompose(hi_f).se == se;
  // thread t continues with elements 16 t .. 16 t + 15 of the segment (zeros past the end of the row)
  float ev[kSegPer];
#pragma unroll
  for (int j = 0; j < kSegPer; j += 4) {
    const float4 q = *reinterpret_cast<const float4*>(stage + tid * kSegPer + j);
    ev[j] = q.x, ev[j + 1] = q.y, ev[j + 2] = q.z, ev[j + 3] = q.w;
  }
  if (!known) {
    // Powers of two may fall inside the segment.  Each of its 64-element parts (four lanes of sixteen elements)
    // estimates the binade the sum has where the part begins, from the double sums of the parts before it, and
    // gets a composed step under that binade and one under the next: the walk applies the one that matches the
    // sum it holds, and adds a part element by element where the sum leaves its binade inside the part or the
    // estimate was wrong.
    constexpr int kPart = kSegElems / kSegSubs;
    static_assert(kPart == 4 * kSegPer && kSegBlock == kSegSubs * 4, "a part is four lanes");
    double mine = 0.0;
#pragma unroll
    for (int j = 0; j < kSegPer; ++j) mine += static_cast<double>(ev[j]);
    mine += __longlong_as_double(static_cast<long long>(lane_xor64<1>(static_cast<u64>(__double_as_longlong(mine)))));
    mine += __longlong_as_double(static_cast<long long>(lane_xor64<2>(static_cast<u64>(__double_as_longlong(mine)))));
    // (all four lanes of a part hold its sum)
    const int part_i = tid >> 2;
    // the sum of the parts before this one: a prefix over the wave's sixteen parts and the totals of the waves before
    const double upto = wave_prefix_sum<double>((lane & 3) == 0 ? mine : 0.0);
    if (lane == 63) wave_parts[wave] = upto;
    __syncthreads();
    double start = before;
    for (int w = 0; w < wave; ++w) start += wave_parts[w];
    start += upto - mine;
    const int p_first = first + part_i * kPart;
    const float plo = __double2float_rd(start * (1.0 - seq_drift(p_first)));
    const float phi = __double2float_ru((start + mine) * (1.0 + seq_drift(p_first + kPart)));
    int pse = seq_decompose(plo).se;
    if (!(plo > 0.0f && phi < 3.0e38f && seq_decompose(phi).se <= pse + 1)) pse = -1;  // the walk adds this part itself
    Step lo_step{0u, 0u}, hi_step{0u, 0u};
    if (pse >= 0) {
      lo_step = seq_compose_run(ev, kSegPer, pse);
      hi_step = seq_compose_run(ev, kSegPer, pse + 1);
    }
    lo_step = quad_scan_steps(lo_step);
    hi_step = quad_scan_steps(hi_step);
    if ((lane & 3) == 3) {
      const size_t at = (static_cast<size_t>(row) * a.segs + seg) * kSegSubs + part_i;
      a.sub_step[at] = make_int4(static_cast<int>(lo_step.d0), static_cast<int>(lo_step.d1), static_cast<int>(hi_step.d0),
                                 static_cast<int>(hi_step.d1));
      a.sub_se[at] = pse;
    }
    if (tid == 0) *rec = make_int4(0, 0, -2, 0);
    return;
  }
  const Step agg = seq_compose_run(ev, kSegPer, se);
  const Step inc = wave_scan_steps(agg);
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  if (tid == 0) {
    Step t = wave_tot[0];
    for (int w = 1; w < 4; ++w) t = step_compose(t, wave_tot[w]);
    *rec = make_int4(static_cast<int>(t.d0), static_cast<int>(t.d1), se, 0);
  }
}

template <typename InT, typename Between>
__global__ __launch_bounds__(kSegBlock) void seqsum_exp_step_kernel(const SeqSumArgs a, const Between between) {
  __shared__ ExpStepShared sh;
  __shared__ typename Between::Shared between_sh;
  if ((static_cast<int>(blockIdx.x) + 1) * kSegElems <= a.vocab)
    seqsum_exp_step_body<InT, Between, true>(a, between, sh, between_sh);
  else
    seqsum_exp_step_body<InT, Between, false>(a, between, sh, between_sh);
}

}  // namespace ms
