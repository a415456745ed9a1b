// Exact sequential-order sum of exp((x - max) / T) over long rows, spread over the whole GPU.
//
// The reference adds the exponentials of a row one by one into a float (LogSoftMax / Softmax,
// src/softmax.h:26-47); block_seq.h reproduces that with a scan of step functions, but one workgroup
// per row leaves most of the chip idle when there are few, long rows (beam search: 32 rows of 152K).
// Here a row is cut into segments of kSegElems elements and four small kernels share the work:
//   1. seqsum_max:   segment maxima.
//   2. seqsum_exp:   e_i = expf((x_i - rowmax) * inv_T) (exact), stored as fp32, plus the segment's
//                    sum in double.
//   3. seqsum_step:  from the double prefix sums a segment knows the binade its running sum will be
//                    in -- unless a power of two may fall inside it -- and composes the step functions
//                    of its elements under that binade into one (d0, d1) pair.
//   4. seqsum_walk:  one workgroup per row walks the segments in order: a composed step is applied
//                    after checking that the running sum really is in the assumed binade and stays
//                    in it (then the composition is exactly the sequential result); every other
//                    segment is summed with the exact in-order scan of block_seq.h.
// The check in step 4 makes the result independent of the estimate in step 3: a wrong guess only
// costs a scan.
#include "kernels.h"
#include "block_seq.h"
#include "seg_io.h"

namespace ms {

template <typename InT>
__global__ __launch_bounds__(kSegBlock) void seqsum_max_kernel(const SeqSumArgs a) {
  __shared__ uint32_t red[4];
  const int seg = blockIdx.x, row = blockIdx.y;
  const InT* x = static_cast<const InT*>(a.x) + static_cast<size_t>(row) * a.row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
  float v[kSegPer];
  seg_load<InT>(x, aligned, a.vocab, seg, -__builtin_inff(), v);
  float fm = -__builtin_inff();
#pragma unroll
  for (int e = 0; e < kSegPer; ++e) fm = fmaxf(fm, v[e]);
  const uint32_t m = block_max<uint32_t>(order_key(fm), red);
  if (threadIdx.x == 0) a.seg_max[static_cast<size_t>(row) * a.segs + seg] = m;
}

__device__ __forceinline__ float row_max_of_segments(const SeqSumArgs& a, int row, uint32_t* red) {
  uint32_t m = 0u;
  for (int s = threadIdx.x; s < a.segs; s += blockDim.x) {
    const uint32_t k = a.seg_max[static_cast<size_t>(row) * a.segs + s];
    m = k > m ? k : m;
  }
  return key_to_float(block_max<uint32_t>(m, red));
}

template <typename InT>
__global__ __launch_bounds__(kSegBlock) void seqsum_exp_kernel(const SeqSumArgs a) {
  __shared__ uint32_t red[4];
  __shared__ double dred[4];
  __shared__ uint64_t exp_tab[32];  // the table of expf in LDS: a lookup per element from constant memory is a gather
  const int seg = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
  const InT* x = static_cast<const InT*>(a.x) + static_cast<size_t>(row) * a.row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
  float v[kSegPer];
  seg_load<InT>(x, aligned, a.vocab, seg, 0.0f, v);
  if (tid < 32) exp_tab[tid] = em::exp2_tab(static_cast<uint32_t>(tid));
  const float max_score = row_max_of_segments(a, row, red);  // its barriers also publish the table
  const uint64_t* const tab = exp_tab;
  auto lds_tab = [=](uint32_t i) { return tab[i]; };
  float* erow = a.e + static_cast<size_t>(row) * a.e_stride;
  double part = 0.0;
#pragma unroll
  for (int e = 0; e < kSegPer; ++e) {
    const int idx = seg_index<InT>(seg, e);
    if (idx < a.vocab) {
      const float ex = em::expf_core((v[e] - max_score) * a.inv_temp, lds_tab);
      erow[idx] = ex;
      part += static_cast<double>(ex);
    }
  }
  part = wave_sum<double>(part);
  if ((tid & 63) == 0) dred[tid >> 6] = part;
  __syncthreads();
  if (tid == 0) a.seg_sum[static_cast<size_t>(row) * a.segs + seg] = (dred[0] + dred[1]) + (dred[2] + dred[3]);
}

// Expected relative distance between the float the reference holds after adding `count` non-negative
// terms one by one and their exact sum: roundings mostly cancel, so it grows like sqrt(count) * 2^-24
// (the worst case grows like count * 2^-24).  Only an estimate is needed: a segment classified on a
// wrong estimate fails the walk's check and is scanned.
__device__ __forceinline__ double seq_drift(int count) {
  return (8.0 * sqrt(static_cast<double>(count)) + 8.0) * 6.0e-8;
}

__global__ __launch_bounds__(kSegBlock) void seqsum_step_kernel(const SeqSumArgs a) {
  __shared__ double dred[4];
  __shared__ __align__(16) float stage[kSegElems];
  __shared__ Step wave_tot[4];
  const int seg = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const double* sums = a.seg_sum + static_cast<size_t>(row) * a.segs;
  double before = 0.0;
  for (int s = tid; s < seg; s += kSegBlock) before += sums[s];
  before = wave_sum<double>(before);
  if (lane == 0) dred[wave] = before;
  __syncthreads();
  before = (dred[0] + dred[1]) + (dred[2] + dred[3]);
  const int first = seg * kSegElems;
  const int n = a.vocab - first < kSegElems ? a.vocab - first : kSegElems;
  const double lo = before * (1.0 - seq_drift(first));
  const double hi = (before + sums[seg]) * (1.0 + seq_drift(first + n));
  const float lo_f = __double2float_rd(lo), hi_f = __double2float_ru(hi);
  const int se = seq_decompose(lo_f).se, se_hi = seq_decompose(hi_f).se;
  int4* rec = a.seg_step + static_cast<size_t>(row) * a.segs + seg;
  const bool in_range = lo_f > 0.0f && hi_f < 3.0e38f;
  const bool known = in_range && se_hi == se;
  if (!known && !(in_range && se_hi == se + 1)) {  // several powers of two may fall inside the segment: the walk scans it
    if (tid == 0) *rec = make_int4(0, 0, -1, 0);
    return;
  }
  const float* erow = a.e + static_cast<size_t>(row) * a.e_stride + first;
  float ev[kSegPer];
  window_fetch<kSegPer>(ev, 0, n, [=](int i) { return erow[i]; }, stage);
  if (!known) {
    // One power of two may fall inside the segment.  Each of its sixteen 256-element parts (sixteen lanes of
    // sixteen elements) gets a composed step under the binade before that power and one under the binade after
    // it: the walk applies the first kind up to the part where the sum leaves the binade, adds that part
    // element by element, and goes on with the second kind.
    static_assert(kSegSubs * 16 * kSegPer == kSegElems && kSegBlock == kSegSubs * 16, "a part is sixteen lanes");
    Step lo_step{0u, 0u}, hi_step{0u, 0u};
#pragma unroll
    for (int j = 0; j < kSegPer; ++j) {
      lo_step = step_compose(lo_step, seq_make_step(ev[j], se));
      hi_step = step_compose(hi_step, seq_make_step(ev[j], se + 1));
    }
    lo_step = row_scan_steps(lo_step);
    hi_step = row_scan_steps(hi_step);
    if ((lane & 15) == 15) {
      int4* sub = a.sub_step + (static_cast<size_t>(row) * a.segs + seg) * kSegSubs;
      sub[tid >> 4] = make_int4(static_cast<int>(lo_step.d0), static_cast<int>(lo_step.d1), static_cast<int>(hi_step.d0),
                                static_cast<int>(hi_step.d1));
    }
    if (tid == 0) *rec = make_int4(0, 0, -2, se);
    return;
  }
  Step agg{0u, 0u};
#pragma unroll
  for (int j = 0; j < kSegPer; ++j) agg = step_compose(agg, seq_make_step(ev[j], se));
  const Step inc = wave_scan_steps(agg);
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  if (tid == 0) {
    Step t = wave_tot[0];
    for (int w = 1; w < 4; ++w) t = step_compose(t, wave_tot[w]);
    *rec = make_int4(static_cast<int>(t.d0), static_cast<int>(t.d1), se, 0);
  }
}

constexpr int kWalkBlock = 256;

__global__ __launch_bounds__(kWalkBlock) void seqsum_walk_kernel(const SeqSumArgs a) {
  __shared__ SeqShared sh;
  __shared__ uint32_t red[16];
  __shared__ int4 recs[kMaxSegs];
  __shared__ int4 subs[kSegSubs];
  __shared__ __align__(16) float stage[kSegElems];
  const int row = blockIdx.x, tid = threadIdx.x;
  for (int s = tid; s < a.segs; s += kWalkBlock) recs[s] = a.seg_step[static_cast<size_t>(row) * a.segs + s];
  const float max_score = row_max_of_segments(a, row, red);  // its barriers also publish recs
  const float* erow = a.e + static_cast<size_t>(row) * a.e_stride;
  float s = 0.0f;
  for (int seg = 0; seg < a.segs; ++seg) {
    const int4 r = recs[seg];
    if (r.z >= 0) {
      const SeqState st = seq_decompose(s);
      if (st.se == r.z) {
        const uint32_t n2 = step_apply(st.n, Step{static_cast<uint32_t>(r.x), static_cast<uint32_t>(r.y)});
        if (n2 < kMantLimit) {  // stayed inside the binade: the composed step is the sequential result
          s = seq_recompose(n2, st.se);
          continue;
        }
      }
    }
    const int first = seg * kSegElems;
    const int n = a.vocab - first < kSegElems ? a.vocab - first : kSegElems;
    const float* e = erow + first;
    int dummy;
    if (r.z == -2) {
      // part by part: a part's composed step under the binade the sum is in, or -- where the sum leaves the
      // binade, or is in neither of the two binades the records were made for -- the part's elements one by one
      const int4* sub = a.sub_step + (static_cast<size_t>(row) * a.segs + seg) * kSegSubs;
      __syncthreads();  // the previous segment's readers of subs are done
      if (tid < kSegSubs) subs[tid] = sub[tid];
      __syncthreads();
      constexpr int kPart = kSegElems / kSegSubs;
      for (int j = 0; j * kPart < n; ++j) {
        const SeqState st = seq_decompose(s);
        const int4 q = subs[j];
        if (st.se == r.w || st.se == r.w + 1) {
          const Step f = st.se == r.w ? Step{static_cast<uint32_t>(q.x), static_cast<uint32_t>(q.y)}
                                      : Step{static_cast<uint32_t>(q.z), static_cast<uint32_t>(q.w)};
          const uint32_t n2 = step_apply(st.n, f);
          if (n2 < kMantLimit) {
            s = seq_recompose(n2, st.se);
            continue;
          }
        }
        const float* ep = e + j * kPart;
        const int np = n - j * kPart < kPart ? n - j * kPart : kPart;
        s = block_seq_sum<kPart / kWalkBlock>(s, np, [=](int i) { return ep[i]; }, NoStop{}, &dummy, sh, nullptr, kPart);  // one wave's chain
      }
      continue;
    }
    s = block_seq_sum<kSegElems / kWalkBlock>(s, n, [=](int i) { return e[i]; }, NoStop{}, &dummy, sh, stage,
                                                 seg == 0 ? 1024 : 0);
  }
  if (tid == 0) {
    a.out_sum[row] = s;
    a.out_max[row] = max_score;
  }
}

// Element-wise finish of Softmax / LogSoftMax (src/softmax.h:26-47) once a row's maximum and sum
// are known: log-softmax writes (x - max) * inv_T - log(sum); softmax writes e * (1 / sum), with e the
// stored exponential (left as is when the sum is zero).
template <bool LOG>
__global__ __launch_bounds__(kSegBlock) void softmax_apply_kernel(float* scores, int64_t row_stride, const SeqSumArgs a) {
  const int seg = blockIdx.x, row = blockIdx.y;
  float* x = scores + static_cast<size_t>(row) * row_stride;
  const float* erow = a.e + static_cast<size_t>(row) * a.e_stride;
  const float max_score = a.out_max[row], sum = a.out_sum[row];
  const float lse = LOG ? em::logf_exact(sum) : 0.0f;
  const float inv_sum = 1.0f / sum;
#pragma unroll
  for (int j = 0; j < kSegPer; ++j) {
    const int i = seg * kSegElems + j * kSegBlock + static_cast<int>(threadIdx.x);
    if (i < a.vocab) {
      if (LOG) {
        x[i] = (x[i] - max_score) * a.inv_temp - lse;
      } else {
        const float ex = erow[i];
        x[i] = sum > 0.0f ? ex * inv_sum : ex;
      }
    }
  }
}

}  // namespace ms

// have_seg_max != 0: the segment maxima in a->seg_max were already written by the caller's own kernel.
extern "C" hipError_t ms_launch_seqsum(const ms::SeqSumArgs* a, int dtype, int have_seg_max, hipStream_t stream) {
  const dim3 grid(a->segs, a->rows), block(ms::kSegBlock);
  if (dtype == MI355X_F16) {
    if (!have_seg_max) hipLaunchKernelGGL(ms::seqsum_max_kernel<uint16_t>, grid, block, 0, stream, *a);
    hipLaunchKernelGGL(ms::seqsum_exp_kernel<uint16_t>, grid, block, 0, stream, *a);
  } else {
    if (!have_seg_max) hipLaunchKernelGGL(ms::seqsum_max_kernel<float>, grid, block, 0, stream, *a);
    hipLaunchKernelGGL(ms::seqsum_exp_kernel<float>, grid, block, 0, stream, *a);
  }
  hipLaunchKernelGGL(ms::seqsum_step_kernel, grid, block, 0, stream, *a);
  hipLaunchKernelGGL(ms::seqsum_walk_kernel, dim3(a->rows), dim3(ms::kWalkBlock), 0, stream, *a);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_softmax_apply(float* scores, int64_t row_stride, const ms::SeqSumArgs* a,
                                              int log_softmax, hipStream_t stream) {
  const dim3 grid(a->segs, a->rows), block(ms::kSegBlock);
  if (log_softmax)
    hipLaunchKernelGGL(ms::softmax_apply_kernel<true>, grid, block, 0, stream, scores, row_stride, *a);
  else
    hipLaunchKernelGGL(ms::softmax_apply_kernel<false>, grid, block, 0, stream, scores, row_stride, *a);
  return hipGetLastError();
}
