// Exact sequential-order sum of exp((x - max) / T) over long rows, spread over the whole GPU.
//
// The reference adds the exponentials of a row one by one into a float (LogSoftMax / Softmax,
// src/softmax.h:26-47); block_seq.h reproduces that with a scan of step functions, but one workgroup
// per row leaves most of the chip idle when there are few, long rows (beam search: 32 rows of 152K).
// Here a row is cut into segments of kSegElems elements and three launches share the work:
//   1. seqsum_max:      segment maxima.
//   2. seqsum_exp_step: e_i = expf((x_i - rowmax) * inv_T) (exact), stored as fp32, plus the segment's
//                       sum in double; then, from the double sums of the segments before it, a segment
//                       knows the binade its running sum will be in -- unless a power of two may fall
//                       inside it -- and composes the step functions of its elements under that binade
//                       into one (d0, d1) pair.
//   3. seqsum_walk:     one wave per row walks the segments in order: composed steps are applied after
//                       checking that the running sum really is in the assumed binade and stays in it
//                       (then the composition is exactly the sequential result); a segment that may hold
//                       a power of two is walked through the composed steps of its 64 parts, and a
//                       part that fails the check is added element by element.
// The check in step 3 makes the result independent of the estimate in step 2: a wrong guess only
// costs a scan.
#include "kernels.h"
#include "block_seq.h"
#include "seg_io.h"
#include "seqsum_exp_step.h"

namespace ms {

template <typename InT>
__global__ __launch_bounds__(kSegBlock) void seqsum_max_kernel(const SeqSumArgs a) {
  __shared__ uint32_t red[4];
  const int seg = blockIdx.x, row = blockIdx.y;
  const InT* x = static_cast<const InT*>(a.x) + static_cast<size_t>(row) * a.row_stride;
  float v[kSegPer];
  seg_load<InT>(x, a.vocab, seg, -__builtin_inff(), v);
  float fm = -__builtin_inff();
#pragma unroll
  for (int e = 0; e < kSegPer; ++e) fm = fmaxf(fm, v[e]);
  const uint32_t m = block_max<uint32_t>(order_key(fm), red);
  if (threadIdx.x == 0) {
    a.seg_max[static_cast<size_t>(row) * a.segs + seg] = m;
    // This launch comes first in every sequence: it marks the segment's sum as not written, so that the look-back
    // of the next launch never takes a sum left by an earlier call for this one's (the walk puts the mark back too,
    // but a sequence that was cut short after its second launch would otherwise leave finite sums behind).
    store_sum_bits(a.seg_sum + static_cast<size_t>(row) * a.segs + seg, kSumNotReady);
  }
}

// ---- the walk: one wave per row walks, fifteen more prepare its way ------------------------------------
// Steps compose associatively as long as the sum stays in one binade, so the walking wave does not visit the
// segments one by one: lane l takes the record of segment seg + l, the compositions over lanes are scanned, and
// every lane checks whether the sum would still be inside the binade after its segment.  All lanes before the
// first one that fails are exact; the failing segment is handled through the records of its 64 parts in the same
// way, a part that fails is added element by element (a chain of lane-shifted float additions), and the wave goes
// on behind it with the binade the sum then has.
//
// Which records compose with which is known before the sum is: a record says for which binade it holds, so the
// lanes fall into runs of equal binade, and the composition of a run from its first lane up to every lane of it
// (a scan that starts afresh at every run) does not depend on the sum.  The workgroup's other waves prepare
// these scans -- one wave for the segments' records, one per segment whose parts are needed -- and fetch the
// elements of the parts that will most likely be added one by one, all at the same time; the walking wave then
// only applies a prepared composition to the sum it holds wherever it stands at the first lane of a run in the
// binade the run expects, and falls back to a scan of its own anywhere else.
constexpr Step kStepIdentity{0u, 0u};
constexpr Step kStepLeaves{kStepSat, kStepSat};  // composed with anything, it still says "left the binade"
constexpr int kWalkSpecials = 16;                 // segments per group of 64 whose part records are cached in LDS
constexpr int kWalkWaves = 16;

// Applies the steps f (one per lane; identity below `from`, kStepLeaves where no valid record exists) to the sum
// s in lane order and returns the number of leading lanes from `from` on, below `limit`, whose results are exact;
// s becomes the sum behind the last of them.
__device__ __forceinline__ int wave_apply_steps(float& s, Step f, int from, int limit) {
  const int lane = lane_id();
  const SeqState st = seq_decompose(s);
  const Step p = wave_scan_steps(f);
  const uint32_t n2 = step_apply(st.n, p);
  const unsigned long long bad = __ballot(lane >= from && lane < limit && n2 >= kMantLimit);
  const int stop = bad != 0ull ? __ffsll(static_cast<long long>(bad)) - 1 : limit;
  if (stop > from) s = seq_recompose(wave_read_lane(n2, stop - 1), st.se);
  return stop;
}

// A prepared run: `run` composes the steps from lane `head` up to this lane; `se` is the binade they hold for
// (negative: none).  Applied to the sum s standing at lane `from`: the number of leading lanes from `from` on that
// are exact (from itself if the run does not start there or expects another binade); s moves behind them.
// *same_run: the lane it stopped at belongs to the run too, so the sum leaves the binade inside that lane's share.
__device__ __forceinline__ int wave_apply_run(float& s, uint2 run, int head, int se, int from, int limit, bool* same_run) {
  const int lane = lane_id();
  const SeqState st = seq_decompose(s);
  const uint32_t n2 = step_apply(st.n, Step{run.x, run.y});
  const bool mine = lane >= from && lane < limit && head == from && se == st.se;
  const unsigned long long in_run = __ballot(mine);
  const unsigned long long not_good = ~__ballot(mine && n2 < kMantLimit) & (~0ull << from);
  const int stop = not_good != 0ull ? __ffsll(static_cast<long long>(not_good)) - 1 : 64;
  if (stop > from) s = seq_recompose(wave_read_lane(n2, stop - 1), st.se);
  *same_run = stop < 64 && ((in_run >> stop) & 1ull) != 0ull;
  return stop;
}

// Scan of steps that starts afresh at every lane whose `se` differs from the lane's below (and at every lane
// without a valid step): the composition from the run's first lane up to each lane, and that first lane.
__device__ __forceinline__ void wave_prepare_runs(Step st, int se, uint2* run, int* head) {
  const int lane = lane_id();
  const int below = dpp_from_below_or<0x138, 0xf, int>(-4, se);  // wave_shr:1; lane 0 sees a value no lane holds
  int h = (lane == 0 || se < 0 || se != below) ? lane : -1;
  wave_segscan_steps(st, h);
  *run = make_uint2(st.d0, st.d1);
  *head = h;
}

constexpr int kWalkAhead = 8;  // parts per cached segment whose elements are fetched ahead into LDS

__global__ __launch_bounds__(64 * kWalkWaves) void seqsum_walk_kernel(const SeqSumArgs a) {
  static_assert(kSegSubs == 64, "one part per lane");
  constexpr int kPart = kSegElems / kSegSubs;
  static_assert(kPart == 64, "a part is one round of the addition chain");
  __shared__ int4 part_rec[kWalkSpecials][kSegSubs];
  __shared__ int part_se[kWalkSpecials][kSegSubs];
  __shared__ uint2 part_run[kWalkSpecials][kSegSubs];
  __shared__ unsigned char part_head[kWalkSpecials][kSegSubs];
  __shared__ float ahead[kWalkSpecials][kWalkAhead][kPart];
  __shared__ int ahead_part[kWalkSpecials][kWalkAhead];
  __shared__ uint2 seg_run[64];
  __shared__ int seg_head[64];
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t rbase = static_cast<size_t>(row) * a.segs;
  float max_score = 0.0f;
  if (wave == 0) {
    uint32_t m = 0u;
    for (int sg = lane; sg < a.segs; sg += 64) {
      const uint32_t k = a.seg_max[rbase + sg];
      m = k > m ? k : m;
    }
    max_score = key_to_float(wave_max<uint32_t>(m));
  }
  // (the row's segment sums have served: back to "not written" for the next launch)
  for (int sg = static_cast<int>(threadIdx.x) - 64; sg >= 0 && sg < a.segs; sg += 64 * (kWalkWaves - 1))
    store_sum_bits(a.seg_sum + rbase + sg, kSumNotReady);
  const float* erow = a.e + static_cast<size_t>(row) * a.e_stride;
  float s = 0.0f;
  for (int g0 = 0; g0 < a.segs; g0 += 64) {  // groups of 64 segments, one per lane
    const int g_n = a.segs - g0 < 64 ? a.segs - g0 : 64;
    const int4 r = lane < g_n ? a.seg_step[rbase + g0 + lane] : make_int4(0, 0, -3, 0);
    const unsigned long long special = __ballot(lane < g_n && r.z == -2);
    const int n_special = __popcll(special) < kWalkSpecials ? __popcll(special) : kWalkSpecials;
    __syncthreads();  // the walk through the previous group is over
    // task 0: the runs of the segments' records; task 1 + slot: the parts of the slot-th segment that has part
    // records -- its runs and the elements of the parts that will most likely be added one by one (those whose
    // estimated binade differs from the next part's, and those without an estimate)
    for (int task = wave; task <= n_special; task += kWalkWaves) {
      if (task == 0) {
        uint2 run;
        int head;
        wave_prepare_runs(r.z >= 0 ? Step{static_cast<uint32_t>(r.x), static_cast<uint32_t>(r.y)} : kStepLeaves, r.z, &run,
                          &head);
        seg_run[lane] = run;
        seg_head[lane] = head;
        continue;
      }
      const int slot = task - 1;
      unsigned long long left = special;
      for (int i = 0; i < slot; ++i) left &= left - 1ull;
      const int sg = __ffsll(static_cast<long long>(left)) - 1;
      const size_t at = (rbase + g0 + sg) * kSegSubs;
      const int4 q = a.sub_step[at + lane];
      const int pse = a.sub_se[at + lane];
      part_rec[slot][lane] = q;
      part_se[slot][lane] = pse;
      const int next_se = static_cast<int>(__builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(pse), 0x130, 0xf, 0xf, false));  // wave_shl:1: the lane above
      unsigned long long want = __ballot(pse < 0 || (lane < 63 && next_se != pse));
      int pp[kWalkAhead];
      float val[kWalkAhead];
#pragma unroll
      for (int c = 0; c < kWalkAhead; ++c) {
        pp[c] = -1;
        val[c] = 0.0f;
        if (want != 0ull) {
          pp[c] = __ffsll(static_cast<long long>(want)) - 1;
          want &= want - 1ull;
          const int idx = (g0 + sg) * kSegElems + pp[c] * kPart + lane;
          if (idx < a.vocab) val[c] = erow[idx];
        }
      }
      uint2 run;
      int head;
      wave_prepare_runs(pse >= 0 ? Step{static_cast<uint32_t>(q.x), static_cast<uint32_t>(q.y)} : kStepLeaves, pse, &run, &head);
      part_run[slot][lane] = run;
      part_head[slot][lane] = static_cast<unsigned char>(head);
#pragma unroll
      for (int c = 0; c < kWalkAhead; ++c) {
        if (lane == 0) ahead_part[slot][c] = pp[c];
        if (pp[c] >= 0) ahead[slot][c][lane] = val[c];
      }
    }
    __syncthreads();
    if (wave != 0) continue;
    const uint2 s_run = seg_run[lane];
    const int s_head = seg_head[lane];
    int seg = 0;  // inside the group
    while (seg < g_n) {
      bool same_run;
      // the prepared run of whole segments, if one starts here in the binade the sum is in now
      const int ahead_seg = wave_apply_run(s, s_run, s_head, r.z, seg, g_n, &same_run);
      if (ahead_seg > seg) {
        seg = ahead_seg;
        continue;
      }
      const int z = wave_read_lane(r.z, seg);
      if (z != -2) {
        // a segment with a record of its own that the prepared runs did not take: the scan from here
        const int se = seq_decompose(s).se;
        const Step f = lane < seg ? kStepIdentity : (r.z == se ? Step{static_cast<uint32_t>(r.x), static_cast<uint32_t>(r.y)} : kStepLeaves);
        const int next = wave_apply_steps(s, f, seg, g_n);
        if (next > seg) {
          seg = next;
          continue;
        }
      }
      // segment `seg` part by part
      const int first = (g0 + seg) * kSegElems;
      const int n = a.vocab - first < kSegElems ? a.vocab - first : kSegElems;
      const int n_parts = (n + kPart - 1) / kPart;
      const int slot = __popcll(special & ((1ull << seg) - 1ull));
      const bool cached = z == -2 && slot < kWalkSpecials;
      int4 q = make_int4(0, 0, 0, 0);
      int pse = -1;
      uint2 p_run = make_uint2(0u, 0u);
      int p_head = -1;
      if (cached) {
        q = part_rec[slot][lane];
        pse = part_se[slot][lane];
        p_run = part_run[slot][lane];
        p_head = part_head[slot][lane];
      } else if (z == -2) {
        q = a.sub_step[(rbase + g0 + seg) * kSegSubs + lane];
        pse = a.sub_se[(rbase + g0 + seg) * kSegSubs + lane];
      }
      int part = 0;
      while (part < n_parts) {
        // the prepared run of parts, if one starts here in the binade the sum is in now; where it ends inside
        // its own run, the sum leaves the binade in that part
        const int ahead_part_n = wave_apply_run(s, p_run, p_head, pse, part, n_parts, &same_run);
        if (ahead_part_n > part) {
          part = ahead_part_n;
          if (part >= n_parts) break;
          if (!same_run) continue;
        } else {
          const int pe = seq_decompose(s).se;
          Step pf = kStepLeaves;
          if (lane < part) pf = kStepIdentity;
          else if (pse >= 0 && pse == pe) pf = Step{static_cast<uint32_t>(q.x), static_cast<uint32_t>(q.y)};
          else if (pse >= 0 && pse + 1 == pe) pf = Step{static_cast<uint32_t>(q.z), static_cast<uint32_t>(q.w)};
          part = wave_apply_steps(s, pf, part, n_parts);
          if (part >= n_parts) break;
        }
        // this part's elements one by one, from LDS where they were fetched ahead
        const int np = n - part * kPart < kPart ? n - part * kPart : kPart;
        const float* src = erow + first + part * kPart;
        int hit = -1;
        if (cached) {
#pragma unroll
          for (int c = 0; c < kWalkAhead; ++c)
            if (ahead_part[slot][c] == part) hit = c;
        }
        const float x = hit >= 0 ? ahead[slot][hit][lane] : (lane < np ? src[lane] : 0.0f);
        s = wave_read_lane(wave_serial_prefix(lane == 0 ? s + x : x, 64), 63);
        ++part;
      }
      ++seg;
    }
  }
  if (wave == 0 && lane == 0) {
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
        // x - max is never -0 where it shows (see softmax_kernel): the maximum here lost the sign of its zero
        const float d = x[i] - max_score;
        x[i] = (d == 0.0f ? 0.0f : d) * a.inv_temp - lse;
      } else {
        const float ex = erow[i];
        x[i] = sum > 0.0f ? ex * inv_sum : ex;
      }
    }
  }
}

}  // namespace ms

extern "C" hipError_t ms_launch_seqsum_max(const ms::SeqSumArgs* a, int dtype, hipStream_t stream) {
  const dim3 grid(a->segs, a->rows), block(ms::kSegBlock);
  if (dtype == MI355X_F16) hipLaunchKernelGGL(ms::seqsum_max_kernel<uint16_t>, grid, block, 0, stream, *a);
  else if (dtype == MI355X_BF16) hipLaunchKernelGGL(ms::seqsum_max_kernel<ms::bf16_t>, grid, block, 0, stream, *a);
  else hipLaunchKernelGGL(ms::seqsum_max_kernel<float>, grid, block, 0, stream, *a);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_seqsum_walk(const ms::SeqSumArgs* a, hipStream_t stream) {
  hipLaunchKernelGGL(ms::seqsum_walk_kernel, dim3(a->rows), dim3(64 * ms::kWalkWaves), 0, stream, *a);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_seqsum(const ms::SeqSumArgs* a, int dtype, hipStream_t stream) {
  const dim3 grid(a->segs, a->rows), block(ms::kSegBlock);
  hipError_t e = ms_launch_seqsum_max(a, dtype, stream);
  if (e != hipSuccess) return e;
  const ms::NothingBetween nothing;
  if (dtype == MI355X_F16)
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<uint16_t, ms::NothingBetween>), grid, block, 0, stream, *a, nothing);
  else if (dtype == MI355X_BF16)
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<ms::bf16_t, ms::NothingBetween>), grid, block, 0, stream, *a, nothing);
  else
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<float, ms::NothingBetween>), grid, block, 0, stream, *a, nothing);
  return ms_launch_seqsum_walk(a, stream);
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
