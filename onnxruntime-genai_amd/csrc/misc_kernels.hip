// Softmax / log-softmax with the reference's sequential fp32 sum, the KV-cache beam gather, the
// speculative-decoding verifier, casts and the logits hand-off.
#include "kernels.h"
#include "block_seq.h"
#include "wave_select.h"

namespace ms {

// ---- Softmax / LogSoftMax (src/softmax.h:26-47) ------------------------------------------------------
// One 1024-thread block per row.  The sum of exponentials is accumulated in index order in fp32 --
// reproduced exactly by the scan of seq_scan.h -- so every output bit equals the reference's.
template <bool LOG>
__global__ __launch_bounds__(1024) void softmax_kernel(float* scores, int64_t row_stride, int vocab, float temperature) {
  __shared__ SeqShared sh;
  __shared__ uint32_t red[16];
  __shared__ __align__(16) float stage[1024 * 8];
  float* x = scores + static_cast<size_t>(blockIdx.x) * row_stride;
  float m = -__builtin_inff();
#pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) m = fmaxf(m, x[i]);
  const float max_score = key_to_float(block_max<uint32_t>(order_key(m), red));
  const float inv_temp = 1.0f / temperature;
  const float* xc = x;
  auto e = [=](int i) { return em::expf_exact((xc[i] - max_score) * inv_temp); };
  int dummy;
  const float sum = block_seq_sum<8>(0.0f, vocab, e, NoStop{}, &dummy, sh, stage, 256);
  if (LOG) {
    const float lse = em::logf_exact(sum);
#pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      // The maximum went through an order key, which holds +0 for either zero, while the reference subtracts the
      // row's own first maximal element.  The sign of a zero difference only shows when lse is 0, that is when the
      // maximum is a single element -- and that element minus itself is +0 -- so +0 is right wherever it matters.
      const float d = x[i] - max_score;
      const float s = (d == 0.0f ? 0.0f : d) * inv_temp;
      x[i] = s - lse;
    }
  } else {
    const float inv_sum = 1.0f / sum;
#pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      const float ex = em::expf_exact((x[i] - max_score) * inv_temp);
      x[i] = sum > 0.0f ? ex * inv_sum : ex;
    }
  }
}

// ---- categorical draws of a batch in the order one engine serves them --------------------------------------
// GreedySearch_Cpu draws row after row from one std::mt19937 (src/search.cpp:207-243, SampleCategoricalToken
// src/sampling_distribution.h:218-227): a row whose kept set holds one token consumes nothing
// (std::discrete_distribution over a single weight returns 0 without touching the engine), nor does a finished
// row.  The caller precomputes the next `rows` canonical doubles of its engine; row r takes the one whose index is
// the number of consuming rows before it.  One workgroup per row; row 0 also reports how many were consumed.
__global__ __launch_bounds__(256) void draw_in_order_kernel(const int32_t* kept_count, const int32_t* kept_ids,
                                                            const float* kept_probs, int cap, int rows, const int32_t* skip,
                                                            const double* pool, int32_t* out_tokens, int32_t* draws_used) {
  __shared__ SeqShared sh;
  __shared__ int red_before[4], red_total[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  // A row consumes a draw when the kept set it is given holds two tokens or more: the count as this kernel uses
  // it, cut to the capacity of the lists.  A count beyond the capacity breaks the caller's contract (the row
  // would draw from a truncated set): *draws_used then reports -1 instead of a number of draws.
  int before = 0, total = 0, broken = 0;
  for (int r = tid; r < rows; r += 256) {
    const int listed = kept_count[r] < cap ? kept_count[r] : cap;
    const int c = (!(skip && skip[r] != 0) && listed >= 2) ? 1 : 0;
    broken |= kept_count[r] > cap ? 1 : 0;
    total += c;
    before += r < row ? c : 0;
  }
  before = wave_sum<int>(before);
  total = wave_sum<int>(total);
  broken = wave_sum<int>(broken);
  if ((tid & 63) == 0) {
    red_before[tid >> 6] = before;
    red_total[tid >> 6] = broken != 0 ? -1 : total;
  }
  __syncthreads();
  before = (red_before[0] + red_before[1]) + (red_before[2] + red_before[3]);
  total = (red_total[0] < 0 || red_total[1] < 0 || red_total[2] < 0 || red_total[3] < 0)
              ? -1
              : (red_total[0] + red_total[1]) + (red_total[2] + red_total[3]);
  int n = kept_count[row];
  n = n < cap ? n : cap;
  const bool consumes = !(skip && skip[row] != 0) && n >= 2;
  int pos = 0;
  if (consumes) {
    const float* pr = kept_probs + static_cast<size_t>(row) * cap;
    pos = block_discrete_draw<4>(n, [=](int i) { return pr[i]; }, pool[before], sh);
  }
  if (tid == 0) {
    out_tokens[row] = kept_ids[static_cast<size_t>(row) * cap + pos];
    if (row == 0 && draws_used) *draws_used = total;
  }
}

// ---- no-repeat-n-gram bans (src/sampling_distribution.h:64-79, src/search.cpp:432-469) -------------------
// One workgroup per row.  Every earlier occurrence of the row's last ngram-1 history ids marks the id
// that followed it.  The row's bitmap is assembled in LDS, one window of kBanWindow ids at a time,
// and written out whole, so rows without any ban get an all-zero bitmap.
constexpr int kBanWindow = 1 << 18;

__global__ __launch_bounds__(256) void ngram_ban_kernel(const Xform xf, int vocab, int ngram, uint32_t* ban) {
  __shared__ uint32_t bits[kBanWindow / 32];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int words = (vocab - 1) / 32 + 1;
  uint32_t* brow = ban + static_cast<size_t>(row) * words;
  const int32_t* h = xf.history + static_cast<size_t>(row) * xf.history_stride;
  const int n = xf.hist_len(row);
  const int pl = ngram - 1;
  for (int base = 0; base < vocab; base += kBanWindow) {
    for (int i = tid; i < kBanWindow / 32; i += 256) bits[i] = 0u;
    __syncthreads();
    for (int start = tid; start + ngram <= n; start += 256) {
      bool match = true;
      for (int j = 0; j < pl && match; ++j) match = h[start + j] == h[n - pl + j];
      if (match) {
        const int tok = h[start + pl];
        if (tok >= base && tok < vocab && tok - base < kBanWindow) atomicOr(&bits[(tok - base) >> 5], 1u << ((tok - base) & 31));
      }
    }
    __syncthreads();
    for (int i = tid; i < kBanWindow / 32 && base / 32 + i < words; i += 256) brow[base / 32 + i] = bits[i];
    __syncthreads();
  }
}

// ---- KV-cache beam gather (src/models/kv_cache.cpp:710-740) -----------------------------------------
// past[t][j] = present[t][beam_indices[j]] for blocks of block_bytes bytes.  grid = (tiles, rows,
// tensors); every block moves kGatherTile bytes with 128-bit non-temporal loads and stores.
constexpr int kGatherTile = 16384;
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void kv_gather_kernel(const void* const* present, void* const* past,
                                                        const int32_t* beam_indices, size_t block_bytes) {
  const int row = blockIdx.y, t = blockIdx.z;
  const size_t tile0 = static_cast<size_t>(blockIdx.x) * kGatherTile;
  const char* src = static_cast<const char*>(present[t]) + static_cast<size_t>(beam_indices[row]) * block_bytes + tile0;
  char* dst = static_cast<char*>(past[t]) + static_cast<size_t>(row) * block_bytes + tile0;
  const size_t remain = block_bytes - tile0;
  const int n16 = static_cast<int>((remain < static_cast<size_t>(kGatherTile) ? remain : kGatherTile) / 16);
  // (The tensors' addresses come out of a table in memory, which tells the compiler nothing about where they point:
  // they are device memory, and the accesses say so -- plain global loads and stores instead of flat ones.)
  typedef __attribute__((address_space(1))) const v4u* DeviceVec;
  typedef __attribute__((address_space(1))) v4u* DeviceVecOut;
  v4u regs[kGatherTile / 16 / 256];
#pragma unroll
  for (int j = 0; j < kGatherTile / 16 / 256; ++j) {
    const int i = j * 256 + threadIdx.x;
    if (i < n16) regs[j] = __builtin_nontemporal_load((DeviceVec)src + i);
  }
#pragma unroll
  for (int j = 0; j < kGatherTile / 16 / 256; ++j) {
    const int i = j * 256 + threadIdx.x;
    if (i < n16) __builtin_nontemporal_store(regs[j], (DeviceVecOut)dst + i);
  }
}

// The same gather for blocks or tensors that are not 16-byte aligned (odd head sizes, sliced views): T is
// the widest unsigned type that divides the block size and every tensor address.  grid = (tiles, rows,
// tensors); a workgroup strides over its row's block.
template <typename T>
__global__ __launch_bounds__(256) void kv_gather_narrow_kernel(const void* const* present, void* const* past,
                                                               const int32_t* beam_indices, size_t block_bytes) {
  const int row = blockIdx.y, t = blockIdx.z;
  const T* src = reinterpret_cast<const T*>(static_cast<const char*>(present[t]) +
                                            static_cast<size_t>(beam_indices[row]) * block_bytes);
  T* dst = reinterpret_cast<T*>(static_cast<char*>(past[t]) + static_cast<size_t>(row) * block_bytes);
  const size_t n = block_bytes / sizeof(T);
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256)
    dst[i] = src[i];
}

// ---- speculative-decoding verification ---------------------------------------------------------------
// block_discrete_draw for at most WINDOWS windows of blockDim * ITEMS weights, read once: the weights stay in
// registers between the pass that sums them and the pass that scans them.  Reports weights that sum to
// exactly 0 through all_zero instead of drawing from them.  Same arithmetic and the same sequential
// replay near a boundary as block_discrete_draw.
struct NoVectorLoads {};  // block_discrete_draw_once without a loader of whole groups of weights

template <int ITEMS, int WINDOWS, typename GetW, typename GetGroup = NoVectorLoads>
__device__ __forceinline__ int block_discrete_draw_once(int n, GetW w, double u, SeqShared& sh, float* stage, bool* all_zero,
                                                        GetGroup group = GetGroup{}) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6, nw = blockDim.x >> 6;
  const int span = static_cast<int>(blockDim.x) * ITEMS;
  *all_zero = false;
  float wv[WINDOWS][ITEMS];
  if constexpr (!std::is_same<GetGroup, NoVectorLoads>::value) {
    // group(i, out) loads the ITEMS weights i .. i + ITEMS - 1 (i a multiple of ITEMS, all below n) with wide
    // loads: a thread reads its own consecutive weights directly, neighbouring lanes neighbouring groups, and no
    // transposition through LDS (two barriers per window) is needed.
#pragma unroll
    for (int c = 0; c < WINDOWS; ++c) {
      const int i0 = c * span + tid * ITEMS;
      if (i0 + ITEMS <= n) {
        group(i0, wv[c]);
      } else {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) wv[c][j] = i0 + j < n ? w(i0 + j) : 0.0f;
      }
    }
  } else {
    // Every weight is requested before the first barrier (a barrier waits for the loads in flight, so fetching
    // window by window would pay the memory latency once per window), consecutive lanes on consecutive indices;
    // then each window is transposed through LDS so that a thread holds ITEMS consecutive weights.
    const int bd = static_cast<int>(blockDim.x);
    float raw[WINDOWS][ITEMS];
#pragma unroll
    for (int c = 0; c < WINDOWS; ++c)
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) {
        const int idx = c * span + j * bd + tid;
        raw[c][j] = idx < n ? w(idx) : 0.0f;
      }
#pragma unroll
    for (int c = 0; c < WINDOWS; ++c) {
#pragma unroll
      for (int j = 0; j < ITEMS; ++j) wv[c][j] = 0.0f;
      if (c * span < n) {
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) stage[j * bd + tid] = raw[c][j];
        __syncthreads();
        static_assert(ITEMS % 4 == 0, "whole float4 reads");
#pragma unroll
        for (int j = 0; j < ITEMS; j += 4) {
          const float4 q = *reinterpret_cast<const float4*>(stage + tid * ITEMS + j);
          wv[c][j] = q.x, wv[c][j + 1] = q.y, wv[c][j + 2] = q.z, wv[c][j + 3] = q.w;
        }
        __syncthreads();  // the staging buffer is rewritten by the next window
      }
    }
  }
  // The windows' scans are independent until their totals chain up: all of them run before the one barrier, and
  // the total of the distribution comes out of them (any summation order will do: the guard band covers it).
  __shared__ double win_scan[WINDOWS][16];
  double pv[WINDOWS][ITEMS], loc[WINDOWS], inc[WINDOWS];
#pragma unroll
  for (int c = 0; c < WINDOWS; ++c) {
    loc[c] = 0.0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      pv[c][j] = static_cast<double>(wv[c][j]);
      loc[c] += pv[c][j];
    }
    inc[c] = wave_scan_add(loc[c]);
    if (lane == 63) win_scan[c][wave] = inc[c];
  }
  __syncthreads();
  // sums of the waves before this one and of every window, all windows in one scan: row c of sixteen lanes takes
  // window c's wave sums, and the lane shifts inside rows scan the four rows at once
  static_assert(WINDOWS <= 4, "one row of sixteen lanes per window");
  const int my_window = (lane >> 4) < WINDOWS ? (lane >> 4) : 0;
  double ws = ((lane >> 4) < WINDOWS && (lane & 15) < nw) ? win_scan[my_window][lane & 15] : 0.0;
  ws = row_scan_add(ws);
  double window_total[WINDOWS];
  double total = 0.0;
#pragma unroll
  for (int c = 0; c < WINDOWS; ++c) {
    window_total[c] = wave_read_lane(ws, c * 16 + 15);
    total += window_total[c];
  }
  if (total != total) return 0;  // NaN weights: see block_discrete_draw
  if (total == 0.0) {
    *all_zero = true;
    return 0;
  }
  if (n < 2) return 0;
  const double guard = 16.0 * static_cast<double>(n) * 1.1102230246251565e-16 * total;
  const double target = u * total;
  double carry = 0.0;
  int first = kIntMax;
  int risky = 0;
#pragma unroll
  for (int c = 0; c < WINDOWS; ++c) {
    const double wp = carry + (wave > 0 ? wave_read_lane(ws, c * 16 + wave - 1) : 0.0);
    draw_scan_thread<ITEMS>(pv[c], wp + (inc[c] - loc[c]), loc[c], c * span + tid * ITEMS, n, target, guard, first, risky);
    carry += window_total[c];
  }
  int a = first, b = risky ? 0 : 1;
  block_min2(a, b, sh);
  if (b != 0) return a;
  if (tid == 0) {  // sequential replay with the reference's own operations
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

// One 1024-thread block per batch entry.  Accept loop of SpeculativeDecodingStrategy::RunRound
// (src/speculative_decoding_strategy.cpp:718-762) on dense distributions, then the round's single
// categorical draw: the residual max(p-q,0) at the first rejected position (SampleCorrectionToken,
// src/speculative_sampling.h:39-57; the target row itself when the residual is all zero) or the
// bonus row K on full acceptance.
__global__ __launch_bounds__(1024) void spec_verify_kernel(const float* p_target, const float* p_draft,
                                                           const int32_t* draft_tokens, const float* accept_u,
                                                           const double* sample_u, int K, int vocab,
                                                           int32_t* accepted_len, int32_t* final_token) {
  __shared__ SeqShared sh;
  __shared__ __align__(16) float stage[1024 * 8];
  __shared__ int sh_n;
  const int b = blockIdx.x;
  const size_t base = static_cast<size_t>(b) * (K + 1) * vocab;
  if (threadIdx.x < 64) {
    // every position's accept test at once (their loads overlap); the loop of the reference stops at
    // the first failure, i.e. at the lowest failing lane
    int rejected_at = K;
    for (int n0 = 0; n0 < K && rejected_at == K; n0 += 64) {
      const int n = n0 + static_cast<int>(threadIdx.x);
      bool reject = false;
      if (n < K) {
        const int d = draft_tokens[b * K + n];
        const float pt = p_target[base + static_cast<size_t>(n) * vocab + d];
        const float pd = p_draft[base + static_cast<size_t>(n) * vocab + d];
        const float acc = pd <= 0.0f ? 1.0f : fminf(1.0f, pt / pd);  // ComputeAcceptProb, :140-146
        reject = !(accept_u[b * K + n] < acc);
      }
      const int f = first_lane(__ballot(reject));
      if (f >= 0) rejected_at = n0 + f;
    }
    if (threadIdx.x == 0) sh_n = rejected_at;
  }
  __syncthreads();
  const int n = sh_n;
  const float* pt = p_target + base + static_cast<size_t>(n) * vocab;
  const float* pd = p_draft + base + static_cast<size_t>(n) * vocab;
  // The residual max(p - q, 0) at the first rejected position is drawn from unless it is all zero
  // (the reference's fp32 "sum > 0" holds iff some residual is positive, and so does the double sum
  // the draw starts with): then, and on full acceptance, the target row itself is.  Vocabularies of up
  // to four windows are read once per draw.
  constexpr int kItems = 8, kWindows = 4;
  const bool once = vocab <= kWindows * kItems * 1024;
  // (the weights are read eight at a time, with 128-bit loads that take rows of any alignment)
  int pos = 0;
  bool from_target = n >= K;
  if (!from_target) {
    auto w = [=](int i) {
      const float d = pt[i] - pd[i];
      return d > 0.0f ? d : 0.0f;
    };
    auto w8 = [=](int i, float (&out)[kItems]) {
      const v4f_any t0 = *reinterpret_cast<const v4f_any*>(pt + i), t1 = *reinterpret_cast<const v4f_any*>(pt + i + 4);
      const v4f_any d0 = *reinterpret_cast<const v4f_any*>(pd + i), d1 = *reinterpret_cast<const v4f_any*>(pd + i + 4);
      const float t[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
      const float d[8] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float r = t[j] - d[j];
        out[j] = r > 0.0f ? r : 0.0f;
      }
    };
    if (once) {
      pos = block_discrete_draw_once<kItems, kWindows>(vocab, w, sample_u[b], sh, stage, &from_target, w8);
    } else {
      int any = 0;
#pragma unroll 8
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) any |= (pt[i] - pd[i] > 0.0f);
      from_target = __syncthreads_or(any) == 0;
      if (!from_target) pos = block_discrete_draw<kItems>(vocab, w, sample_u[b], sh, stage);
    }
    __syncthreads();
  }
  if (from_target) {
    auto w = [=](int i) { return pt[i]; };
    auto w8 = [=](int i, float (&out)[kItems]) {
      const v4f_any t0 = *reinterpret_cast<const v4f_any*>(pt + i), t1 = *reinterpret_cast<const v4f_any*>(pt + i + 4);
      out[0] = t0.x, out[1] = t0.y, out[2] = t0.z, out[3] = t0.w, out[4] = t1.x, out[5] = t1.y, out[6] = t1.z, out[7] = t1.w;
    };
    bool unused;
    if (once) pos = block_discrete_draw_once<kItems, kWindows>(vocab, w, sample_u[b], sh, stage, &unused, w8);
    else pos = block_discrete_draw<kItems>(vocab, w, sample_u[b], sh, stage);
  }
  if (threadIdx.x == 0) {
    accepted_len[b] = n;
    final_token[b] = pos;
  }
}

// ---- EOS bookkeeping and sequence append after token selection --------------------------------------
// CheckForEOSAndPad + AppendNextTokensToSequences (src/cuda/search_cuda.cu:33-48,80-117) in one launch of
// one workgroup.
struct TailEos {
  int n;
  int32_t ids[MI355X_MAX_EOS];
};

__global__ __launch_bounds__(256) void greedy_tail_kernel(int32_t* next_tokens, int32_t* eos_seen, int batch, TailEos eos,
                                                          int32_t pad, int32_t* sequences, int max_length,
                                                          int current_length, int32_t* done) {
  int live = 0;
  for (int b = threadIdx.x; b < batch; b += 256) {
    int32_t tok = next_tokens[b];
    int seen = eos_seen[b];
    if (seen) {
      tok = pad;
      next_tokens[b] = tok;
    } else {
      for (int e = 0; e < eos.n; ++e) seen |= (tok == eos.ids[e]);
      if (seen) eos_seen[b] = 1;
    }
    live |= !seen;
    if (current_length < max_length) sequences[static_cast<size_t>(b) * max_length + current_length] = tok;
  }
  if (__syncthreads_or(live) == 0 && threadIdx.x == 0) *done = 1;
}

// ---- speculative verification on sparse selections ----------------------------------------------------
// One 256-thread block per sequence.  Target rows 0..K (row i judges proposal token i, row K is the
// bonus row) and draft rows 0..K-1 are kept sets: count, ids, probabilities, padded to a capacity.
//   mode 0  the accept loop of SpeculativeDecodingStrategy::RunRound
//           (src/speculative_decoding_strategy.cpp:718-762): GetSparseTokenProbability,
//           ComputeAcceptProb, then SampleCorrectionToken at the first reject (residual over the target
//           row's ids; the target row itself when the residual sums to zero) or SampleSparseToken on
//           the bonus row (src/speculative_sampling.h:22-57,140-146).  sample_u[e] is the categorical
//           draw available after e accept draws.
//   mode 1  VerifyDeterministicProposal (src/speculative_sampling.h:96-127): sample every target row in
//           turn until the sample differs from the proposal; sample_u holds the draws in the order rows
//           with at least two entries consume them.
//   mode 2  greedy targets: entry 0 of every target row is the row's greedy token.
// A row whose count exceeds its capacity (truncated by the producer) or is below 1: the sequence reports -1.
constexpr int kSpecMaxK = 64;

__device__ __forceinline__ float wave_sparse_prob(const int32_t* ids, const float* probs, int n, int32_t token) {
  const int lane = lane_id();
  for (int j0 = 0; j0 < n; j0 += 64) {
    const int j = j0 + lane;
    const int f = first_lane(__ballot(j < n && ids[j] == token));
    if (f >= 0) return probs[j0 + f];
  }
  return 0.0f;
}

__global__ __launch_bounds__(256) void spec_verify_sparse_kernel(const SpecSparseArgs a) {
  __shared__ SeqShared sh;
  __shared__ float s_pt[kSpecMaxK], s_pd[kSpecMaxK];
  __shared__ int s_n, s_bad;
  const int b = blockIdx.x, tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  const int K = a.K;
  const int32_t* tc = a.t_count + static_cast<size_t>(b) * (K + 1);
  const int32_t* prop = a.proposal + static_cast<size_t>(b) * K;
  auto t_ids = [&](int r) { return a.t_ids + (static_cast<size_t>(b) * (K + 1) + r) * a.t_cap; };
  auto t_probs = [&](int r) { return a.t_probs + (static_cast<size_t>(b) * (K + 1) + r) * a.t_cap; };
  if (tid == 0) s_bad = 0;
  __syncthreads();
  for (int r = tid; r <= K; r += 256) {
    bool bad = tc[r] > a.t_cap || tc[r] < 1;
    if (a.mode == 0 && r < K) bad = bad || a.d_count[static_cast<size_t>(b) * K + r] > a.d_cap;
    if (bad) s_bad = 1;
  }
  __syncthreads();
  if (s_bad) {
    if (tid == 0) {
      a.accepted_len[b] = -1;
      a.final_token[b] = -1;
      a.engine_draws[b] = 0;
    }
    return;
  }
  if (a.mode == 2) {
    if (tid == 0) {
      int n = 0;
      while (n < K && t_ids(n)[0] == prop[n]) ++n;
      a.accepted_len[b] = n;
      a.final_token[b] = t_ids(n)[0];
      a.engine_draws[b] = 0;
    }
    return;
  }
  if (a.mode == 1) {
    int used = 0, accepted = 0;
    int32_t tok = -1;
    for (int i = 0; i <= K; ++i) {
      const int n = tc[i];
      const float* pr = t_probs(i);
      const int pos = block_discrete_draw<4>(n, [=](int j) { return pr[j]; },
                                             n >= 2 ? a.sample_u[static_cast<size_t>(b) * (K + 1) + used] : 0.0, sh);
      if (n >= 2) ++used;
      tok = t_ids(i)[pos];
      if (i == K || tok != prop[i]) break;
      ++accepted;
    }
    if (tid == 0) {
      a.accepted_len[b] = accepted;
      a.final_token[b] = tok;
      a.engine_draws[b] = 2 * used;
    }
    return;
  }
  // mode 0: every position's two look-ups at once, a wave per position
  const int32_t* dc = a.d_count + static_cast<size_t>(b) * K;
  for (int i = wave; i < K; i += 4) {
    const float pt = wave_sparse_prob(t_ids(i), t_probs(i), tc[i], prop[i]);
    const float pd = wave_sparse_prob(a.d_ids + (static_cast<size_t>(b) * K + i) * a.d_cap,
                                      a.d_probs + (static_cast<size_t>(b) * K + i) * a.d_cap, dc[i], prop[i]);
    if (lane == 0) {
      s_pt[i] = pt;
      s_pd[i] = pd;
    }
  }
  __syncthreads();
  if (tid == 0) {
    int n = 0;
    for (; n < K; ++n) {
      const float acc = s_pd[n] <= 0.0f ? 1.0f : fminf(1.0f, s_pt[n] / s_pd[n]);  // ComputeAcceptProb
      if (!(a.accept_u[static_cast<size_t>(b) * K + n] < acc)) break;
    }
    s_n = n;
  }
  __syncthreads();
  const int n = s_n;
  const int evaluated = n < K ? n + 1 : K;
  const int nt = tc[n];
  const int32_t* ids = t_ids(n);
  const float* pr = t_probs(n);
  bool use_residual = false;
  float* res = a.residual + static_cast<size_t>(b) * a.residual_stride;
  if (n < K) {
    const int32_t* di = a.d_ids + (static_cast<size_t>(b) * K + n) * a.d_cap;
    const float* dp = a.d_probs + (static_cast<size_t>(b) * K + n) * a.d_cap;
    const int nd = dc[n];
    int any = 0;
    for (int j = tid; j < nt; j += 256) {
      const int32_t id = ids[j];
      float q = 0.0f;
      for (int m = 0; m < nd; ++m)
        if (di[m] == id) {
          q = dp[m];
          break;
        }
      const float d = pr[j] - q;
      const float r = d > 0.0f ? d : 0.0f;
      res[j] = r;
      any |= r > 0.0f;
    }
    // the reference's sequential fp32 sum of non-negative terms is positive iff one of them is
    use_residual = __syncthreads_or(any) != 0;
  }
  const double u = a.sample_u[static_cast<size_t>(b) * (K + 1) + evaluated];
  int pos;
  if (use_residual) {
    const float* rr = res;
    pos = block_discrete_draw<4>(nt, [=](int j) { return rr[j]; }, u, sh);
  } else {
    pos = block_discrete_draw<4>(nt, [=](int j) { return pr[j]; }, u, sh);
  }
  if (tid == 0) {
    a.accepted_len[b] = n;
    a.final_token[b] = ids[pos];
    a.engine_draws[b] = evaluated + (nt >= 2 ? 2 : 0);
  }
}

// ---- DeviceInterface::Cast (src/cpu/interface.cpp:74-106) -----------------------------------------
// kind: 0 fp16->fp32, 1 bf16->fp32, 2 fp32->fp16, 3 fp32->bf16 (upper 16 bits), 4 int32->int64.
__global__ __launch_bounds__(256) void cast_kernel(const void* in, void* out, size_t count, int kind) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
    switch (kind) {
      case 0: static_cast<float*>(out)[i] = half_bits_to_float(static_cast<const uint16_t*>(in)[i]); break;
      case 1: static_cast<float*>(out)[i] = bf16_bits_to_float(static_cast<const uint16_t*>(in)[i]); break;
      case 2: static_cast<uint16_t*>(out)[i] = static_cast<uint16_t>(float_to_half_bits(static_cast<const float*>(in)[i])); break;
      case 3: static_cast<uint16_t*>(out)[i] = static_cast<uint16_t>(__float_as_uint(static_cast<const float*>(in)[i]) >> 16); break;
      default: static_cast<int64_t*>(out)[i] = static_cast<const int32_t*>(in)[i]; break;
    }
  }
}

// ---- logits hand-off: last-token slice + widening in one pass (Logits::Get, src/models/logits.cpp:33-82)
// raw is [rows, seq_len, vocab] of fp32 / fp16 / bf16; row r's source is token token_index[r] (the
// last token when token_index is null).  out: [rows] rows of `vocab` floats at out_stride.
template <int KIND>  // 0 fp16, 1 bf16, 2 fp32
__global__ __launch_bounds__(256) void logits_handoff_kernel(const void* raw, int seq_len, int vocab,
                                                             const int32_t* token_index, float* out, int64_t out_stride) {
  const int row = blockIdx.y;
  const int tok = token_index ? token_index[row] : seq_len - 1;
  const size_t src0 = (static_cast<size_t>(row) * seq_len + tok) * vocab;
  float* dst = out + static_cast<size_t>(row) * out_stride;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < vocab; i += gridDim.x * blockDim.x) {
    if (KIND == 0) dst[i] = half_bits_to_float(static_cast<const uint16_t*>(raw)[src0 + i]);
    else if (KIND == 1) dst[i] = bf16_bits_to_float(static_cast<const uint16_t*>(raw)[src0 + i]);
    else dst[i] = static_cast<const float*>(raw)[src0 + i];
  }
}

}  // namespace ms

extern "C" hipError_t ms_launch_cast(const void* in, void* out, size_t count, int kind, hipStream_t stream) {
  size_t blocks = (count + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(ms::cast_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, in, out, count, kind);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_logits_handoff(const void* raw, int kind, int rows, int seq_len, int vocab,
                                               const int32_t* token_index, float* out, int64_t out_stride,
                                               hipStream_t stream) {
  int gx = (vocab + 255) / 256;
  if (gx > 256) gx = 256;
  const dim3 grid(gx, rows), block(256);
  if (kind == 0)
    hipLaunchKernelGGL(ms::logits_handoff_kernel<0>, grid, block, 0, stream, raw, seq_len, vocab, token_index, out, out_stride);
  else if (kind == 1)
    hipLaunchKernelGGL(ms::logits_handoff_kernel<1>, grid, block, 0, stream, raw, seq_len, vocab, token_index, out, out_stride);
  else
    hipLaunchKernelGGL(ms::logits_handoff_kernel<2>, grid, block, 0, stream, raw, seq_len, vocab, token_index, out, out_stride);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_softmax(float* scores, int64_t row_stride, int rows, int vocab, float temperature,
                                        int log_softmax, hipStream_t stream) {
  if (log_softmax)
    hipLaunchKernelGGL(ms::softmax_kernel<true>, dim3(rows), dim3(1024), 0, stream, scores, row_stride, vocab, temperature);
  else
    hipLaunchKernelGGL(ms::softmax_kernel<false>, dim3(rows), dim3(1024), 0, stream, scores, row_stride, vocab, temperature);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_draw_in_order(const int32_t* kept_count, const int32_t* kept_ids, const float* kept_probs,
                                               int cap, int rows, const int32_t* skip, const double* pool,
                                               int32_t* out_tokens, int32_t* draws_used, hipStream_t stream) {
  hipLaunchKernelGGL(ms::draw_in_order_kernel, dim3(rows), dim3(256), 0, stream, kept_count, kept_ids, kept_probs, cap, rows,
                     skip, pool, out_tokens, draws_used);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_ngram_ban(const ms::Xform* xf, int rows, int vocab, int ngram, uint32_t* ban,
                                          hipStream_t stream) {
  hipLaunchKernelGGL(ms::ngram_ban_kernel, dim3(rows), dim3(256), 0, stream, *xf, vocab, ngram, ban);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_kv_gather(const void* const* present_dev, void* const* past_dev, int n_tensors,
                                          const int32_t* beam_indices, int rows, size_t block_bytes, int width,
                                          hipStream_t stream) {
  if (width == 16) {
    const unsigned tiles = static_cast<unsigned>((block_bytes + ms::kGatherTile - 1) / ms::kGatherTile);
    hipLaunchKernelGGL(ms::kv_gather_kernel, dim3(tiles, rows, n_tensors), dim3(256), 0, stream, present_dev, past_dev,
                       beam_indices, block_bytes);
    return hipGetLastError();
  }
  const size_t per_wg = static_cast<size_t>(256) * 8 * width;  // eight elements per thread
  size_t tiles = (block_bytes + per_wg - 1) / per_wg;
  if (tiles > 4096) tiles = 4096;
  const dim3 grid(static_cast<unsigned>(tiles), rows, n_tensors);
  switch (width) {
    case 8:
      hipLaunchKernelGGL(ms::kv_gather_narrow_kernel<uint64_t>, grid, dim3(256), 0, stream, present_dev, past_dev,
                         beam_indices, block_bytes);
      break;
    case 4:
      hipLaunchKernelGGL(ms::kv_gather_narrow_kernel<uint32_t>, grid, dim3(256), 0, stream, present_dev, past_dev,
                         beam_indices, block_bytes);
      break;
    case 2:
      hipLaunchKernelGGL(ms::kv_gather_narrow_kernel<uint16_t>, grid, dim3(256), 0, stream, present_dev, past_dev,
                         beam_indices, block_bytes);
      break;
    case 1:
      hipLaunchKernelGGL(ms::kv_gather_narrow_kernel<uint8_t>, grid, dim3(256), 0, stream, present_dev, past_dev,
                         beam_indices, block_bytes);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_spec_verify(const float* p_target, const float* p_draft, const int32_t* draft_tokens,
                                            const float* accept_u, const double* sample_u, int batch, int K, int vocab,
                                            int32_t* accepted_len, int32_t* final_token, hipStream_t stream) {
  hipLaunchKernelGGL(ms::spec_verify_kernel, dim3(batch), dim3(1024), 0, stream, p_target, p_draft, draft_tokens,
                     accept_u, sample_u, K, vocab, accepted_len, final_token);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_greedy_tail(int32_t* next_tokens, int32_t* eos_seen, int batch, const int32_t* eos_ids,
                                            int n_eos, int32_t pad, int32_t* sequences, int max_length,
                                            int current_length, int32_t* done, hipStream_t stream) {
  ms::TailEos eos{};
  eos.n = n_eos;
  for (int i = 0; i < n_eos; ++i) eos.ids[i] = eos_ids[i];
  hipLaunchKernelGGL(ms::greedy_tail_kernel, dim3(1), dim3(256), 0, stream, next_tokens, eos_seen, batch, eos, pad,
                     sequences, max_length, current_length, done);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_spec_verify_sparse(const ms::SpecSparseArgs* a, int batch, hipStream_t stream) {
  hipLaunchKernelGGL(ms::spec_verify_sparse_kernel, dim3(batch), dim3(256), 0, stream, *a);
  return hipGetLastError();
}

