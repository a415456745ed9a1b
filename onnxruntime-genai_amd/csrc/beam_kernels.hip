// Beam search: per-row log-softmax + candidate selection, per-batch merge to the 2*beams best, the
// device-resident BeamSearchScorer and the beam-reordered sequence append.
#include "kernels.h"
#include "block_seq.h"
#include "wave_select.h"
#include "seg_io.h"
#include "seqsum_exp_step.h"

namespace ms {

constexpr int kBeamListCap = 1024;  // candidates a row may hold in LDS before the slow exact path

// Calls fn(index, value) for every element of a row, the block's threads taking 16-byte vectors in
// turn (four vectors in flight per thread); every thread makes the same number of calls per vector
// round, with index -1 past the end of the row, so fn may contain wave-wide operations.
template <typename InT, typename Fn>
__device__ __forceinline__ void row_for_each(const InT* x, int V, Fn fn) {
  constexpr int VEC = 16 / sizeof(InT);
  const int step = static_cast<int>(blockDim.x) * VEC;
  for (int base = 0; base < V; base += 4 * step) {
    float v[4][VEC];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i0 = base + r * step + static_cast<int>(threadIdx.x) * VEC;
      if (i0 + VEC <= V) {
        const v4u_any q = *reinterpret_cast<const v4u_any*>(x + i0);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        if constexpr (VEC == 4) {
#pragma unroll
          for (int c = 0; c < 4; ++c) v[r][c] = __uint_as_float(w[c]);
        } else if constexpr (__is_same(InT, uint16_t)) {
          v4u qq;
          qq.x = q.x, qq.y = q.y, qq.z = q.z, qq.w = q.w;
          widen_half8(qq, v[r]);
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            v[r][2 * c] = narrow_bits_to_float<InT>(w[c] & 0xffffu);
            v[r][2 * c + 1] = narrow_bits_to_float<InT>(w[c] >> 16);
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[r][c] = (i0 + c < V) ? load_one<InT>(x, i0 + c) : 0.0f;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i0 = base + r * step + static_cast<int>(threadIdx.x) * VEC;
      if (base + r * step < V) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) fn(i0 + c < V ? i0 + c : -1, v[r][c]);
      }
    }
  }
}

// One 1024-thread block per batch-beam row.  BeamSearch_Cpu::SelectTop (src/search.cpp:101-123):
// scores = ((x - max) * 1.0f - log(sum exp)) + beam_score, the sum accumulated in index order in
// fp32 (reproduced exactly by the scan of seq_scan.h).  The value is monotone in x, so the row's
// 2*beams best come from its largest logits: a pooled bound on per-thread maxima gives a cut whose
// final score decides membership; everything at or above it is sorted by (score desc, token asc).
template <typename InT>
__global__ __launch_bounds__(1024) void beam_row_kernel(const BeamArgs a) {
  __shared__ SeqShared sh;
  __shared__ __align__(16) float stage[1024 * 8];
  __shared__ u64 list[kBeamListCap];
  __shared__ uint32_t pool[64];
  __shared__ uint32_t red[16];
  __shared__ u64 red64[16];
  __shared__ uint32_t count;
  const int row = blockIdx.x, tid = threadIdx.x;
  const int V = a.vocab, m = 2 * a.beams;
  const InT* x = static_cast<const InT*>(a.logits) + static_cast<size_t>(row) * a.row_stride;
  float fm = -__builtin_inff();
  row_for_each<InT>(x, V, [&](int i, float val) {
    if (i >= 0) fm = fmaxf(fm, val);
  });
  constexpr int kVec = 16 / sizeof(InT);
  const uint32_t lkey = tid * kVec < V ? order_key(fm) : 0u;
  const float own_max = key_to_float(block_max<uint32_t>(lkey, red));
  const float max_score = a.row_max ? a.row_max[row] : own_max;
  const int n_lanes = (V + kVec - 1) / kVec < 1024 ? (V + kVec - 1) / kVec : 1024;
  const uint32_t tau = block_pool_bound(lkey, m, (n_lanes + 63) / 64, pool);
  auto e = [=](int i) { return em::expf_exact(load_one<InT>(x, i) - max_score); };
  int dummy;
  const float lse = em::logf_exact(a.row_sum ? a.row_sum[row] : block_seq_sum<8>(0.0f, V, e, NoStop{}, &dummy, sh, stage, 256));
  const float bs = a.beam_scores[row];
  auto final_score = [=](float v) { return ((v - max_score) - lse) + bs; };
  // tau == 0: fewer than m offers (tiny vocabulary): every element is a candidate
  const float cut = tau != 0u ? final_score(key_to_float(tau)) : -__builtin_inff();
  if (tid == 0) count = 0u;
  __syncthreads();
  row_for_each<InT>(x, V, [&](int i, float val) {
    const float f = final_score(val);
    const bool cand = i >= 0 && ((f >= cut) || (tau == 0u));
    const uint32_t pos = wave_slot(cand, &count);
    if (cand && pos < kBeamListCap) list[pos] = make_key64(order_key(f), static_cast<uint32_t>(i));
  });
  __syncthreads();
  const uint32_t n = count;
  float* out_s = a.row_scores + static_cast<size_t>(row) * kBeamMaxCand;
  int32_t* out_t = a.row_tokens + static_cast<size_t>(row) * kBeamMaxCand;
  if (n <= kBeamListCap) {
    int n2 = 64;
    while (n2 < static_cast<int>(n)) n2 <<= 1;
    for (int p = static_cast<int>(n) + tid; p < n2; p += blockDim.x) list[p] = 0;
    __syncthreads();
    block_sort_desc(list, n2);
    if (tid < m) {
      const u64 k = tid < static_cast<int>(n) ? list[tid] : 0;
      out_s[tid] = key_to_float(key64_okey(k));
      out_t[tid] = k ? static_cast<int32_t>(key64_index(k)) : -1;
    }
    return;
  }
  // Heavy ties (e.g. a constant row): extract the m best one at a time, each the largest
  // (score, lowest token) key strictly below the previous one.
  u64 last = ~0ull;
  for (int r = 0; r < m; ++r) {
    u64 best = 0;
    for (int i = tid; i < V; i += blockDim.x) {
      const u64 k = make_key64(order_key(final_score(load_one<InT>(x, i))), static_cast<uint32_t>(i));
      if (k < last && k > best) best = k;
    }
    best = block_max<u64>(best, red64);
    if (tid == 0) {
      out_s[r] = key_to_float(key64_okey(best));
      out_t[r] = best ? static_cast<int32_t>(key64_index(best)) : -1;
    }
    last = best ? best : 0;
  }
}

// One block per batch entry: the 2*beams best of the beams x 2*beams row candidates by
// (score desc, beam*vocab+token asc), as the flat partial_sort of src/search.cpp:148-163 orders them.
__global__ __launch_bounds__(256) void beam_merge_kernel(const BeamArgs a) {
  __shared__ u64 keys[512];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int m = 2 * a.beams, n = a.beams * m;
  int n2 = 64;
  while (n2 < n) n2 <<= 1;
  for (int p = tid; p < n2; p += blockDim.x) {
    u64 k = 0;
    if (p < n) {
      const int beam = p / m, j = p % m;
      const size_t src = static_cast<size_t>(b * a.beams + beam) * kBeamMaxCand + j;
      const int tok = a.row_tokens[src];
      if (tok >= 0)
        k = make_key64(order_key(a.row_scores[src]), static_cast<uint32_t>(beam) * static_cast<uint32_t>(a.vocab) +
                                                         static_cast<uint32_t>(tok));
    }
    keys[p] = k;
  }
  __syncthreads();
  block_sort_desc(keys, n2);
  if (tid < m) {
    const u64 k = keys[tid];
    const uint32_t flat = key64_index(k);
    a.out_scores[b * m + tid] = key_to_float(key64_okey(k));
    a.out_tokens[b * m + tid] = static_cast<int32_t>(flat % static_cast<uint32_t>(a.vocab));
    a.out_beams[b * m + tid] = static_cast<int32_t>(flat / static_cast<uint32_t>(a.vocab));
  }
}

// ---- BeamSearchScorer::Process (src/beam_search_scorer.cpp:84-171), one wave per batch entry ----------
// All lanes follow the same scalar control flow; the lanes only share the work of cloning sequences.
__device__ __forceinline__ bool scorer_is_eos(const ScorerState& s, int tok) {
  for (int i = 0; i < s.n_eos; ++i)
    if (s.eos[i] == tok) return true;
  return false;
}

// BeamHypotheses::Add (src/beam_search_scorer.cpp:19-39).  Hypotheses live in beams+1 token rows per
// batch entry; `slot` maps rank -> row, so inserting shifts ranks, not tokens.
// `used`: the entry's hypothesis count, which the caller holds (the same in all lanes) and this keeps up to date.
__device__ __forceinline__ void scorer_add(const ScorerState& s, int batch, const int32_t* seq, int length,
                                           float sum_logprobs, int& used) {
  const int nb = s.beams, lane = lane_id();
  float* hs = s.hyp_score + batch * nb;
  int* hl = s.hyp_len + batch * nb;
  int* slot = s.hyp_slot + batch * (nb + 1);
  const float score = sum_logprobs / s.pow_table[length];
  int index = used;
  int row;
  if (index == nb) {
    if (score <= hs[nb - 1]) return;
    index = nb - 1;
    row = slot[nb - 1];  // the evicted hypothesis' row is reused
  } else {
    row = slot[index];
    used = index + 1;
    if (lane == 0) s.hyp_used[batch] = index + 1;
  }
  int32_t* dst = s.hyp_tokens + (static_cast<size_t>(batch) * (nb + 1) + row) * s.max_length;
  for (int i = lane; i < length; i += 64) dst[i] = seq[i];
  __builtin_amdgcn_wave_barrier();
  if (lane == 0) {
    for (; index > 0 && score > hs[index - 1]; index--) {
      hs[index] = hs[index - 1];
      hl[index] = hl[index - 1];
      slot[index] = slot[index - 1];
    }
    hs[index] = score;
    hl[index] = length;
    slot[index] = row;
  }
  __threadfence_block();
  __builtin_amdgcn_wave_barrier();
}

// Reads through to memory that other workgroups of the same launch have written (after a fence on both sides).
__device__ __forceinline__ float load_agent(const float* p) {
  return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ int load_agent(const int* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The end of BeamSearchScorer::Process for an entry that holds `beams` hypotheses and does not stop early
// (src/beam_search_scorer.cpp:155-170): done unless the best candidate could still improve on the worst kept
// hypothesis.  The reference's window over the candidates starts at batch*beams rather than batch*2*beams (:161),
// so it looks at other entries' candidates; kept as is, which is why this runs once all entries' candidates exist.
__device__ __forceinline__ void scorer_check_done(const ScorerState& s, int batch, const float* all_scores,
                                                  int sequence_length) {
  const int nb = s.beams, top_k = 2 * nb;
  float best = load_agent(all_scores + batch * nb);
  for (int i = 1; i < top_k; ++i) best = fmaxf(best, load_agent(all_scores + batch * nb + i));
  const float current = best / s.pow_table[sequence_length];
  const bool can_improve = load_agent(s.hyp_score + batch * nb + nb - 1) < current;  // CanImprove
  if (!can_improve) {
    s.done[batch] = 1;
    atomicSub(s.not_done, 1);
  }
}

// What a scorer step reads of the entry's state before it looks at the candidates; asked for early, the loads
// are back by the time the candidates are.
struct ScorerEntryState {
  int done, used;   // the same in all lanes
  int tok, src;     // lane i < beams: token and source row that beam row i holds from the step before
};
__device__ __forceinline__ ScorerEntryState scorer_entry_state(const ScorerState& s, int batch) {
  const int lane = lane_id(), nb = s.beams;
  ScorerEntryState e;
  e.done = s.done[batch];
  e.used = s.hyp_used[batch];
  e.tok = lane < nb ? s.next_tokens[batch * nb + lane] : s.pad;
  e.src = lane < nb ? s.next_indices[batch * nb + lane] : 0;
  return e;
}

// BeamSearchScorer::Process for one batch entry (one wave); scorer_append follows it: lane i keeps the (token,
// source row) of beam row i in `next`, and the wave then copies those rows of the current sequences into the next
// buffer with the token appended.  A done entry's rows copy global row 0, as the reference does with its index 0;
// nothing read here is written by another entry's wave in the same launch.  cand_*: the entry's own 2*beams
// candidates.  Returns (the same in all lanes) whether scorer_check_done still has to run for the entry.
__device__ __forceinline__ bool scorer_entry(const ScorerState& s, int batch, const ScorerEntryState& st,
                                             const int32_t* sequences, int sequence_length, const float* cand_scores,
                                             const int32_t* cand_tokens, const int32_t* cand_indices,
                                             ScorerEntryState& next) {
  const int lane = lane_id();
  const int nb = s.beams, top_k = 2 * nb;
  int my_tok = s.pad, my_src = 0;  // what a done entry emits
  bool check = false;
  if (st.done) {
    if (lane < nb) {
      s.next_scores[batch * nb + lane] = 0.0f;
      s.next_tokens[batch * nb + lane] = s.pad;
      s.next_indices[batch * nb + lane] = 0;
    }
  } else {
    // a beam row that gets no candidate this step (more EOS candidates than the reference expects) keeps the
    // token and source row it had, as the reference's arrays do
    my_tok = st.tok;
    my_src = st.src;
    int used = st.used;
    int beam_idx = 0;
    for (int j = 0; j < top_k; ++j) {
      const int tok = cand_tokens[j];
      const float score = cand_scores[j];
      const int bbi = batch * nb + cand_indices[j];
      if (scorer_is_eos(s, tok)) {
        if (j >= nb) continue;
        scorer_add(s, batch, sequences + static_cast<size_t>(bbi) * s.max_length, sequence_length, score, used);
      } else {
        if (lane == beam_idx) {
          my_tok = tok;
          my_src = bbi;
          s.next_scores[batch * nb + beam_idx] = score;
          s.next_tokens[batch * nb + beam_idx] = tok;
          s.next_indices[batch * nb + beam_idx] = bbi;
        }
        ++beam_idx;
      }
      if (beam_idx == nb) break;
    }
    if (used >= nb) {
      if (s.early_stopping) {
        if (lane == 0) {
          s.done[batch] = 1;
          atomicSub(s.not_done, 1);
        }
      } else {
        check = true;
      }
    }
  }
  next.tok = my_tok;
  next.src = my_src;
  return check;
}

// BeamSearch_Cpu::AppendNextTokensToSequences for the entry's rows, from what scorer_entry left in `next`.
__device__ __forceinline__ void scorer_append(const ScorerState& s, int batch, const ScorerEntryState& next,
                                              const int32_t* sequences, int32_t* sequences_next, int sequence_length) {
  const int lane = lane_id(), nb = s.beams;
  const int my_tok = next.tok, my_src = next.src;
  // the rows four at a time: their loads are all under way before the first store waits for one
  for (int i0 = 0; i0 < nb; i0 += 4) {
    const int32_t* src[4];
    int32_t* dst[4];
    int tok[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u < nb ? i0 + u : nb - 1;  // (a row past the end repeats the last one)
      src[u] = sequences + static_cast<size_t>(wave_read_lane(my_src, i)) * s.max_length;
      dst[u] = sequences_next + static_cast<size_t>(batch * nb + i) * s.max_length;
      tok[u] = wave_read_lane(my_tok, i);
    }
    for (int t = lane; t < sequence_length; t += 64) {
      int32_t v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = src[u][t];
#pragma unroll
      for (int u = 0; u < 4; ++u) dst[u][t] = v[u];
    }
    if (lane == 0) {
#pragma unroll
      for (int u = 0; u < 4; ++u) dst[u][sequence_length] = tok[u];
    }
  }
}

__global__ __launch_bounds__(64) void beam_scorer_step_kernel(const ScorerState s, const int32_t* sequences,
                                                              int32_t* sequences_next, int sequence_length,
                                                              const float* cand_scores, const int32_t* cand_tokens,
                                                              const int32_t* cand_indices) {
  const int batch = blockIdx.x, top_k = 2 * s.beams;
  const ScorerEntryState st = scorer_entry_state(s, batch);
  ScorerEntryState next{};
  const bool check = scorer_entry(s, batch, st, sequences, sequence_length, cand_scores + batch * top_k,
                                  cand_tokens + batch * top_k, cand_indices + batch * top_k, next);
  scorer_append(s, batch, next, sequences, sequences_next, sequence_length);
  if (check && lane_id() == 0) scorer_check_done(s, batch, cand_scores, sequence_length);
}

__global__ __launch_bounds__(64) void beam_scorer_finalize_kernel(const ScorerState s, const int32_t* sequences,
                                                                  int sequence_length) {
  const int batch = blockIdx.x;
  if (s.done[batch]) return;
  int used = s.hyp_used[batch];
  for (int j = 0; j < s.beams; ++j) {
    const int bbi = batch * s.beams + j;
    scorer_add(s, batch, sequences + static_cast<size_t>(bbi) * s.max_length, sequence_length, s.next_scores[bbi], used);
  }
}


// ---- long rows: candidates per segment, scored once the exact sum is known --------------------------------
//
// The final score ((x - max) - log(sum)) + beam_score is a non-decreasing function of the logit x, so the
// 2*beams best final scores of a batch entry belong to elements that are among the 2*beams largest logits of
// their own segment.  SegmentLists lists those per segment (inside the exact sum's launch that holds the
// segment's logits in registers anyway); beam_fin_kernel scores the listed elements and keeps the best by
// (final score desc, beam * vocab + token asc), the order of the flat partial_sort of src/search.cpp:148-163.
// Rounding can give different logits the same final score, and then the lowest index wins, which the logit
// order does not know.  A segment whose list is full (it may hold more elements of the same final score as its
// last entry) and whose last entry reaches the final score of the entry's 2*beams-th best makes the finishing
// workgroup rescan the rows themselves; so do non-finite maxima and entries with fewer than 2*beams numbers.

constexpr int kSegCandCap = 512;        // candidates a segment may list before it reports an overflow
constexpr u64 kSegOverflow = ~0ull;     // first entry of a segment that listed more than kSegCandCap

// Runs inside the launch that writes the exponentials, while a segment's workgroup waits for the sums of the
// segments before it: v are the segment's logits as that launch loaded them (zeros past the end of the row).
template <typename InT>
struct SegmentLists {
  BeamArgs a;
  struct Shared {
    u64 list[kSegCandCap];
    uint32_t wave_bound[kSegBlock / 64];
    uint32_t count;
  };
  template <bool FULL>
  __device__ __forceinline__ void run(Shared& sh, const float (&v)[kSegPer], int seg, int row) const {
    u64* const list = sh.list;
    uint32_t* const wave_bound = sh.wave_bound;
    uint32_t& count = sh.count;
    const int tid = threadIdx.x;
    const int V = a.vocab, m = 2 * a.beams;
    float fm = -__builtin_inff();
#pragma unroll
    for (int e = 0; e < kSegPer; ++e)
      if (FULL || seg_index<InT>(seg, e) < V) fm = fmaxf(fm, v[e]);
    const uint32_t offer = (FULL || seg_index<InT>(seg, 0) < V) ? order_key(fm) : 0u;  // threads past the end of the row offer nothing
    // A wave's m-th best thread maximum (0 with fewer than m offers) has m of the wave's elements at or above it;
    // so has the largest of the four, and with it everything that can be among the segment's m best.
    const uint32_t mth = wave_read_lane(wave_sort_desc_fast<uint32_t>(offer), m - 1);
    if ((tid & 63) == 0) wave_bound[tid >> 6] = mth;
    if (tid == 0) count = 0u;
    __syncthreads();
    uint32_t tau = wave_bound[0];
#pragma unroll
    for (int w = 1; w < kSegBlock / 64; ++w) tau = wave_bound[w] > tau ? wave_bound[w] : tau;
    // a thread's candidates are counted first, so that a wave asks for its list positions once
    uint32_t mine = 0u;
#pragma unroll
    for (int e = 0; e < kSegPer; ++e) {
      const bool cand = (FULL || seg_index<InT>(seg, e) < V) && (tau == 0u || order_key(v[e]) >= tau);  // tau == 0: fewer than m offers, list everything
      mine |= cand ? 1u << e : 0u;
    }
    const uint32_t n_mine = static_cast<uint32_t>(__popc(mine));
    const uint32_t upto = wave_prefix_sum<uint32_t>(n_mine);
    const uint32_t n_wave = wave_read_lane(upto, 63);
    uint32_t pos = 0u;
    if (n_wave != 0u) {
      if ((tid & 63) == 0) pos = atomicAdd(&count, n_wave);
      pos = wave_read_lane(pos, 0) + upto - n_mine;
    }
#pragma unroll
    for (int e = 0; e < kSegPer; ++e) {
      if ((mine >> e) & 1u) {
        if (pos < kSegCandCap) list[pos] = make_key64(order_key(v[e]), static_cast<uint32_t>(seg_index<InT>(seg, e)));
        ++pos;
      }
    }
    __syncthreads();
    const int n = static_cast<int>(count);
    u64* out = a.seg_cand + (static_cast<size_t>(row) * a.segs + seg) * m;
    if (n > kSegCandCap) {
      if (tid < m) out[tid] = tid == 0 ? kSegOverflow : 0ull;
    } else if (n <= 64) {  // the usual case: one wave sorts the list in registers
      if (tid < 64) {
        const u64 k = wave_sort_desc_fast<u64>(tid < n ? list[tid] : 0ull);
        if (tid < m) out[tid] = k;
      }
    } else {
      int n2 = 128;
      while (n2 < n) n2 <<= 1;
      for (int p = n + tid; p < n2; p += kSegBlock) list[p] = 0ull;
      __syncthreads();
      block_sort_desc(list, n2);
      if (tid < m) out[tid] = list[tid];
    }
  }
};

// SCORER: the entry's workgroup goes on with the entry's scorer step (scorer_entry, by its first wave, from the
// candidates in LDS); the tests that need every entry's candidates are left to the workgroup that gets through last.
template <typename InT, bool SCORER>
__global__ __launch_bounds__(256) void beam_fin_kernel(const BeamArgs a, const ScorerStep sp) {
  constexpr int R = kBeamFinCap / 256;
  __shared__ u64 red64[4];
  __shared__ uint32_t red[4];
  __shared__ u64 best_list[kBeamMaxCand];
  __shared__ float s_max[kBeamMaxCand / 2], s_lse[kBeamMaxCand / 2], s_bs[kBeamMaxCand / 2];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int V = a.vocab, m = 2 * a.beams, per_row = a.segs * m, n = a.beams * per_row;
  // the listed candidates are requested before anything waits (they do not depend on the rows' sums)
  const u64* cand = a.seg_cand + static_cast<size_t>(b * a.beams) * per_row;
  const int nr = (n + 255) >> 8;  // key slots per thread in use
  u64 raw[R];
#pragma unroll
  for (int r = 0; r < R; ++r) raw[r] = (r < nr && tid + r * 256 < n) ? cand[tid + r * 256] : 0ull;
  ScorerEntryState entry_state{};
  if constexpr (SCORER) {
    if (tid < 64) entry_state = scorer_entry_state(sp.s, b);
  }
  bool odd = false;  // a row whose maximum is not a finite number: its scores need not follow the logit order
  if (tid < a.beams) {
    const int row = b * a.beams + tid;
    s_max[tid] = a.row_max[row];
    s_lse[tid] = em::logf_exact(a.row_sum[row]);
    s_bs[tid] = a.beam_scores[row];
    odd = !(fabsf(s_max[tid]) < __builtin_inff());
  }
  __syncthreads();
  u64 key[R];
  uint32_t full_reach = odd ? 0xffffffffu : 0u;  // best final score among the last entries of full lists
  // entry p = tid + 256 r of the batch entry's lists: beam p / per_row, position j = p % m inside its list
  int beam = tid / per_row, j = tid % m;
  int q = tid - beam * per_row;
  const int dj = 256 % m;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    key[r] = 0ull;
    if (r < nr && tid + r * 256 < n) {
      const u64 c = raw[r];
      if (c == kSegOverflow) {
        full_reach = 0xffffffffu;
      } else if (c != 0ull) {
        const float f = ((key_to_float(key64_okey(c)) - s_max[beam]) - s_lse[beam]) + s_bs[beam];
        const uint32_t fk = order_key(f);
        key[r] = make_key64(fk, static_cast<uint32_t>(beam) * static_cast<uint32_t>(V) + key64_index(c));
        if (j == m - 1 && fk > full_reach) full_reach = fk;
      }
    }
    q += 256;
    while (q >= per_row) q -= per_row, ++beam;
    j += dj;
    if (j >= m) j -= m;
  }
  // The m best keys, best first.  Every wave lists its keys that reach the m-th best of its 64 per-lane maxima (at
  // least m of its keys do, so the wave's m best are among them; with fewer than m lanes holding keys, all keys), the
  // four lists together usually hold fewer than 64 keys, and wave 0 sorts those.
  __shared__ u64 hit[4][64];
  __shared__ uint32_t hit_n[4];
  __shared__ u64 wave_best[4 * kBeamMaxCand];
  const int lane = tid & 63, wave = tid >> 6;
  {
    u64 lane_best = 0ull;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < nr && key[r] > lane_best) lane_best = key[r];
    const u64 tau = wave_read_lane(wave_sort_desc_fast<u64>(lane_best), m - 1);
    uint32_t woff = 0u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const bool cand = r < nr && key[r] != 0ull && key[r] >= tau;
      const u64 bal = __ballot(cand);
      if (bal == 0ull) continue;
      if (cand) {
        const uint32_t pos = woff + __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(bal >> 32),
                                                              __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(bal), 0u));
        if (pos < 64u) hit[wave][pos] = key[r];
      }
      woff += static_cast<uint32_t>(__popcll(bal));
    }
    if (lane == 0) hit_n[wave] = woff;
  }
  __syncthreads();
  const uint32_t n0 = hit_n[0], n1 = hit_n[1], n2 = hit_n[2], n3 = hit_n[3];
  u64 last = ~0ull;
  if (n0 + n1 + n2 + n3 <= 64u) {
    if (wave == 0) {
      const uint32_t p = static_cast<uint32_t>(lane);
      u64 k = 0ull;
      if (p < n0) k = hit[0][p];
      else if (p < n0 + n1) k = hit[1][p - n0];
      else if (p < n0 + n1 + n2) k = hit[2][p - n0 - n1];
      else if (p < n0 + n1 + n2 + n3) k = hit[3][p - n0 - n1 - n2];
      k = wave_sort_desc_fast<u64>(k);
      if (lane < m) best_list[lane] = k;
    }
  } else {
    // More than one wave's worth of listed keys (many beams, or ties at a bound): every wave extracts the m best of
    // its own keys, each the largest key below the previous one, then wave 0 extracts the m best of the four lists.
    for (int j = 0; j < m; ++j) {
      u64 best = 0ull;
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r < nr && key[r] < last && key[r] > best) best = key[r];
      best = wave_max(best);
      if (lane == 0) wave_best[wave * kBeamMaxCand + j] = best;
      last = best;  // 0 once nothing is left: later rounds find nothing either
    }
    __syncthreads();
    if (wave == 0) {
      // entries j < m of the four lists: two per lane (4 m <= 128)
      u64 mine[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e = lane + 64 * h;
        mine[h] = e < 4 * m ? wave_best[(e / m) * kBeamMaxCand + e % m] : 0ull;
      }
      last = ~0ull;
      for (int j = 0; j < m; ++j) {
        u64 best = 0ull;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          if (mine[h] < last && mine[h] > best) best = mine[h];
        best = wave_max(best);
        if (lane == 0) best_list[j] = best;
        last = best;
      }
    }
  }
  __syncthreads();
  last = best_list[m - 1];
  const uint32_t cut = key64_okey(last);
  const uint32_t reach = block_max<uint32_t>(full_reach, red);
  if (cut == 0u || reach >= cut) {
    // rescan the rows: the m best one at a time, each the largest key strictly below the previous one
    last = ~0ull;
    for (int j = 0; j < m; ++j) {
      u64 best = 0ull;
      for (int beam = 0; beam < a.beams; ++beam) {
        const InT* x = static_cast<const InT*>(a.logits) + static_cast<size_t>(b * a.beams + beam) * a.row_stride;
        const float mx = s_max[beam], lse = s_lse[beam], bs = s_bs[beam];
        for (int i = tid; i < V; i += 256) {
          const float f = ((load_one<InT>(x, i) - mx) - lse) + bs;
          const u64 k = make_key64(order_key(f), static_cast<uint32_t>(beam) * static_cast<uint32_t>(V) + static_cast<uint32_t>(i));
          if (k < last && k > best) best = k;
        }
      }
      best = block_max<u64>(best, red64);
      if (tid == 0) best_list[j] = best;
      last = best;
    }
  }
  __syncthreads();
  __shared__ float c_scores[kBeamMaxCand];
  __shared__ int32_t c_tokens[kBeamMaxCand], c_beams[kBeamMaxCand];
  if (tid < m) {
    const u64 k = best_list[tid];
    const uint32_t flat = key64_index(k);
    const float score = key_to_float(key64_okey(k));
    const int32_t tok = static_cast<int32_t>(flat % static_cast<uint32_t>(V));
    const int32_t beam = static_cast<int32_t>(flat / static_cast<uint32_t>(V));
    a.out_scores[b * m + tid] = score;
    a.out_tokens[b * m + tid] = tok;
    a.out_beams[b * m + tid] = beam;
    if constexpr (SCORER) c_scores[tid] = score, c_tokens[tid] = tok, c_beams[tid] = beam;
  }
  if constexpr (SCORER) {
    __syncthreads();
    if (wave != 0) return;
    const ScorerState& s = sp.s;
    ScorerEntryState next{};
    const bool check = scorer_entry(s, b, entry_state, sp.sequences, sp.sequence_length, c_scores, c_tokens, c_beams, next);
    if (lane == 0) s.pending[b] = check ? 1 : 0;
    // Everything the tests below read of this workgroup is out before it counts itself through, and the last one
    // through sees all of it; the sequences, which those tests do not read, are extended while the count travels.
    __threadfence();
    unsigned ticket = 0u;
    if (lane == 0) ticket = atomicAdd(s.arrive, 1u);
    scorer_append(s, b, next, sp.sequences, sp.sequences_next, sp.sequence_length);
    if (wave_read_lane(ticket, 0) != gridDim.x - 1u) return;
    __threadfence();
    if (lane == 0) *s.arrive = 0u;
    for (int e = lane; e < s.batch; e += 64) {
      if (load_agent(s.pending + e) != 0) scorer_check_done(s, e, a.out_scores, sp.sequence_length);
    }
  }
}

}  // namespace ms

// The exact sums' second launch (exponentials, step records) with the segments' candidate lists built in it.
extern "C" hipError_t ms_launch_beam_exp_step(const ms::SeqSumArgs* q, const ms::BeamArgs* a, int dtype, hipStream_t stream) {
  const dim3 grid(q->segs, q->rows), block(ms::kSegBlock);
  if (dtype == MI355X_F16)
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<uint16_t, ms::SegmentLists<uint16_t>>), grid, block, 0, stream, *q,
                       ms::SegmentLists<uint16_t>{*a});
  else if (dtype == MI355X_BF16)
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<ms::bf16_t, ms::SegmentLists<ms::bf16_t>>), grid, block, 0, stream, *q,
                       ms::SegmentLists<ms::bf16_t>{*a});
  else
    hipLaunchKernelGGL((ms::seqsum_exp_step_kernel<float, ms::SegmentLists<float>>), grid, block, 0, stream, *q,
                       ms::SegmentLists<float>{*a});
  return hipGetLastError();
}

namespace {
template <typename InT>
void launch_beam_finish(const ms::BeamArgs* a, const ms::ScorerStep* step, hipStream_t stream) {
  if (step)
    hipLaunchKernelGGL((ms::beam_fin_kernel<InT, true>), dim3(a->batch), dim3(256), 0, stream, *a, *step);
  else
    hipLaunchKernelGGL((ms::beam_fin_kernel<InT, false>), dim3(a->batch), dim3(256), 0, stream, *a, ms::ScorerStep{});
}
}  // namespace

extern "C" hipError_t ms_launch_beam_finish(const ms::BeamArgs* a, int dtype, const ms::ScorerStep* step,
                                            hipStream_t stream) {
  if (dtype == MI355X_F16) launch_beam_finish<uint16_t>(a, step, stream);
  else if (dtype == MI355X_BF16) launch_beam_finish<ms::bf16_t>(a, step, stream);
  else launch_beam_finish<float>(a, step, stream);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_beam_select(const ms::BeamArgs* a, int dtype, hipStream_t stream) {
  const int rows = a->batch * a->beams;
  if (dtype == MI355X_F16)
    hipLaunchKernelGGL(ms::beam_row_kernel<uint16_t>, dim3(rows), dim3(1024), 0, stream, *a);
  else if (dtype == MI355X_BF16)
    hipLaunchKernelGGL(ms::beam_row_kernel<ms::bf16_t>, dim3(rows), dim3(1024), 0, stream, *a);
  else
    hipLaunchKernelGGL(ms::beam_row_kernel<float>, dim3(rows), dim3(1024), 0, stream, *a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ms::beam_merge_kernel, dim3(a->batch), dim3(256), 0, stream, *a);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_scorer_step(const ms::ScorerState* s, const int32_t* sequences, int32_t* sequences_next,
                                            int sequence_length, const float* cs, const int32_t* ct, const int32_t* ci,
                                            hipStream_t stream) {
  hipLaunchKernelGGL(ms::beam_scorer_step_kernel, dim3(s->batch), dim3(64), 0, stream, *s, sequences, sequences_next,
                     sequence_length, cs, ct, ci);
  return hipGetLastError();
}
extern "C" hipError_t ms_launch_scorer_finalize(const ms::ScorerState* s, const int32_t* sequences, int sequence_length,
                                                hipStream_t stream) {
  hipLaunchKernelGGL(ms::beam_scorer_finalize_kernel, dim3(s->batch), dim3(64), 0, stream, *s, sequences, sequence_length);
  return hipGetLastError();
}

