// Streaming kernels of the sampling path (templates; a source file per element type instantiates them).
//
// sample_fused_kernel (top-k rows, k <= 64; one launch per step): every workgroup (512 threads x 64
// logits) streams one 32K-logit chunk of one row with 128-bit non-temporal loads, logits processing
// fused, keeps the chunk's best 64 candidates and publishes them sorted; the workgroup of a row's last
// chunk polls for the other chunks' lists, merges them four at a time (bitonic merges in registers)
// and runs the reference's scalar epilogue (softmax over the k, nucleus cut, categorical draw) in rank
// order.  nucleus_stream_kernel (rows with k <= 1; 1024 threads x 32 logits per workgroup) compacts
// every chunk's candidates into the row's key buffer; nucleus_finish_kernel sorts them and finishes.
// Anything the fast paths decline (k > 64, heavy ties, tiny vocabularies, more history ids in a chunk
// than its list holds) goes through general_row, an exact full sort.  Each streaming kernel exists
// with and without the code of the logits processing (_xf) and with the per-row parameters in a
// device table or inside the kernel arguments (_rows).
#pragma once
#include "kernels.h"
#include "block_seq.h"
#include "wave_select.h"

namespace ms {

typedef float v4f __attribute__((ext_vector_type(4)));

// (k, p, T) of a row.  INLINE kernels carry a table as their second argument and read it through the
// kernel-argument segment itself (constant address space, scalar loads): indexing the by-value
// argument object with a run-time row would make the compiler copy the whole object to private memory.
static_assert(sizeof(SampleArgs) % alignof(InlineParams) == 0, "the table follows the first argument without padding");
template <bool INLINE>
__device__ __forceinline__ mi355x_sample_params row_params(const SampleArgs& a, int row, mi355x_sample_params uniform) {
  if constexpr (INLINE) {
    typedef __attribute__((address_space(4))) const char* KernargPtr;
    const KernargPtr base = (KernargPtr)__builtin_amdgcn_kernarg_segment_ptr();
    typedef __attribute__((address_space(4))) const mi355x_sample_params* TablePtr;
    const TablePtr table = (TablePtr)(base + sizeof(SampleArgs));
    mi355x_sample_params q;
    q.k = __builtin_amdgcn_readfirstlane(table[row].k);
    q.p = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(table[row].p)));
    q.temperature = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(table[row].temperature)));
    return q;
  } else {
    // The device table is read-only during the launch: read through the constant address space, its
    // entries come by scalar loads like the uniform parameters from the kernel arguments, the row's mode
    // is a scalar, and nothing here waits for a vector load before the logits are requested.
    mi355x_sample_params q = uniform;
    if (a.per_row) {
      typedef __attribute__((address_space(4))) const mi355x_sample_params* TablePtr;
      const TablePtr table = (TablePtr)a.per_row;
      q.k = table[row].k;
      q.p = table[row].p;
      q.temperature = table[row].temperature;
    }
    return q;
  }
}
template <bool INLINE>
__device__ __forceinline__ mi355x_sample_params row_params(const SampleArgs& a, int row) {
  return row_params<INLINE>(a, row, a.uniform);
}

__device__ __forceinline__ int next_pow2(int v) {
  int p = 64;
  while (p < v) p <<= 1;
  return p;
}

__device__ __forceinline__ RowOutputs row_outputs(const SampleArgs& a, int row) {
  return RowOutputs{a.out_tokens + row, a.kept_count ? a.kept_count + row : nullptr,
                    a.kept_ids ? a.kept_ids + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                    a.kept_probs ? a.kept_probs + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                    a.kept_capacity};
}

// A row of the logits as fp32 values, whatever it is stored as: InT float, uint16_t (fp16 bits) or bf16_t,
// widened with the conversions of the reference's CPU path; AnyDtype decides per access from
// SampleArgs::dtype (code that revisits single elements of a row outside the streaming kernels).
struct AnyDtype {};
template <typename InT>
struct RowPtr {
  const InT* p;
  __device__ __forceinline__ RowPtr(const void* row0, int) : p(static_cast<const InT*>(row0)) {}
  __device__ __forceinline__ float operator[](int i) const { return load_one<InT>(p, i); }
};
template <>
struct RowPtr<AnyDtype> {
  const void* p;
  int dtype;
  __device__ __forceinline__ RowPtr(const void* row0, int dtype_code) : p(row0), dtype(dtype_code) {}
  __device__ __forceinline__ float operator[](int i) const {
    if (dtype == MI355X_F16) return half_bits_to_float(static_cast<const uint16_t*>(p)[i]);
    if (dtype == MI355X_BF16) return bf16_bits_to_float(static_cast<const uint16_t*>(p)[i]);
    return static_cast<const float*>(p)[i];
  }
};

// First element of row `row`.  Rows normally lie row_stride elements apart; the kernels that carry a table in
// their arguments (INLINE) also take rows scattered over memory, one pointer per row in that table (null: not used).
template <bool INLINE>
__device__ __forceinline__ const void* row_start(const SampleArgs& a, int row, size_t elem_bytes) {
  if constexpr (INLINE) {
    typedef __attribute__((address_space(4))) const char* KernargPtr;
    const KernargPtr base = (KernargPtr)__builtin_amdgcn_kernarg_segment_ptr();
    typedef __attribute__((address_space(4))) const unsigned long long* TablePtr;
    const TablePtr table = (TablePtr)(base + sizeof(SampleArgs) + offsetof(InlineParams, row_ptr));
    const unsigned long long ptr = table[row];
    if (ptr != 0ull) {
      const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ptr));
      const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ptr >> 32));
      return reinterpret_cast<const void*>((static_cast<unsigned long long>(hi) << 32) | lo);
    }
  }
  return static_cast<const char*>(a.logits) + static_cast<size_t>(row) * a.row_stride * elem_bytes;
}
__device__ __forceinline__ size_t dtype_bytes(int dtype) { return (dtype == MI355X_F16 || dtype == MI355X_BF16) ? 2 : 4; }

// Exact general path for one row, any (k, p, T), any vocabulary size: rebuilds the processed row as
// key64s in global scratch, sorts all of it, then runs the reference algorithm on the sorted row.
// Run by one whole block.  scratch holds next_pow2(vocab) entries.
struct SortInGlobalMemory {
  __device__ void operator()(u64* keys, int n2, int) const { block_sort_desc(keys, n2); }
};

// LDS for select_topk_desc: a list of kSelectCap keys, one word per thread, a few counters.
constexpr int kSelectCap = 2048;
struct TopkSelectLds {
  u64* list;
  uint32_t* maxima;  // blockDim.x words
  uint32_t* words;   // 4 + blockDim.x / 64 words
};

// The kk (1 .. 64) largest of the n distinct keys of a row, key i belonging to id i (so that, among keys of one score,
// a lower index is a larger key), sorted descending into s.list[0 .. kk): what a row that asks for its k best
// needs of the full sort, at the cost of four passes over the keys.  The kk-th largest of the threads' best scores
// is a score that at least kk keys reach; the keys above it are listed as they are found (fewer than kk of them,
// unless threads hold several), and of the keys that tie with it -- all the masked ids of a row, for one -- the
// first ones in index order fill up the kk, found by counting ties wave by wave over contiguous runs of indices.
// Returns false, with nothing decided, when more than kSelectCap keys lie above that score.  Run by a whole block
// (a power of two of threads, at least 64); contains barriers.
__device__ __forceinline__ bool select_topk_desc(const u64* keys, int n, int kk, const TopkSelectLds& s) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6, nw = static_cast<int>(blockDim.x) >> 6;
  uint32_t best = 0u;
  for (int i = tid; i < n; i += blockDim.x) {
    const uint32_t score = key64_okey(keys[i]);
    best = score > best ? score : best;
  }
  s.maxima[tid] = best;
  if (tid == 0) s.words[0] = 0u;
  __syncthreads();
  block_sort_desc(s.maxima, static_cast<int>(blockDim.x));
  const uint32_t tau = s.maxima[kk - 1];
  const int seg = ((n + nw - 1) / nw + 63) & ~63;  // wave w owns the indices w * seg .. (w + 1) * seg - 1
  const int lo = wave * seg, hi = lo + seg < n ? lo + seg : n;
  uint32_t ties = 0u;
  for (int i0 = lo; i0 < hi; i0 += 64) {
    const int i = i0 + lane;
    const u64 k = i < hi ? keys[i] : 0;
    const bool above = i < hi && key64_okey(k) > tau;
    const u64 ab = __ballot(above);
    if (ab != 0ull) {
      uint32_t base = 0u;
      if (lane == 0) base = atomicAdd(&s.words[0], static_cast<uint32_t>(__popcll(ab)));
      base = __builtin_amdgcn_readfirstlane(base);
      const uint32_t pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(ab >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(ab), base));
      if (above && pos < static_cast<uint32_t>(kSelectCap)) s.list[pos] = k;
    }
    ties += static_cast<uint32_t>(__popcll(__ballot(i < hi && key64_okey(k) == tau)));
  }
  if (lane == 0) s.words[4 + wave] = ties;
  __syncthreads();
  const uint32_t n_above = s.words[0];
  if (n_above > static_cast<uint32_t>(kSelectCap)) return false;
  uint32_t n_list = n_above;
  if (n_above < static_cast<uint32_t>(kk)) {
    const uint32_t want = static_cast<uint32_t>(kk) - n_above;  // at least that many keys tie
    uint32_t run = 0u;
    for (int w = 0; w < wave; ++w) run += s.words[4 + w];
    for (int i0 = lo; i0 < hi && run < want; i0 += 64) {
      const int i = i0 + lane;
      const u64 k = i < hi ? keys[i] : 0;
      const bool tie = i < hi && key64_okey(k) == tau;
      const u64 tb = __ballot(tie);
      const uint32_t rank = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(tb >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(tb), run));
      if (tie && rank < want) s.list[n_above + rank] = k;
      run += static_cast<uint32_t>(__popcll(tb));
    }
    n_list = static_cast<uint32_t>(kk);
  }
  const int n2 = next_pow2(static_cast<int>(n_list));  // (at least 64)
  for (int i = static_cast<int>(n_list) + tid; i < n2; i += blockDim.x) s.list[i] = 0;
  __syncthreads();
  block_sort_desc(s.list, n2);
  return true;
}

template <typename InT, typename SortFn = SortInGlobalMemory, int EPI_ITEMS = 4>
__device__ __forceinline__ void general_row(const SampleArgs& a, int row, const void* row0, const mi355x_sample_params prm,
                                            u64* scratch, SeqShared& sh, SortFn sort_desc = SortFn{},
                                            const TopkSelectLds* select = nullptr) {
  const int V = a.vocab;
  const RowPtr<InT> lrow(row0, a.dtype);
  const int n2 = next_pow2(V);
  const bool has_mask = a.xf.mask != nullptr;
  const uint32_t* mrow = has_mask ? a.xf.mask + static_cast<size_t>(row) * ((V - 1) / 32 + 1) : nullptr;
  const int n_eos = a.xf.eos_count(row);
  const uint32_t* ban_row = a.xf.ban_row(row, V);
  constexpr int kLoads = 4;  // loads a thread has in flight
  for (int i0 = threadIdx.x; i0 < n2; i0 += kLoads * blockDim.x) {
    float raw[kLoads];
    uint32_t mw[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      const int i = i0 + u * blockDim.x;
      raw[u] = i < V ? lrow[i] : 0.0f;
      mw[u] = (has_mask && i < V) ? mrow[i >> 5] : 0u;
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i >= n2) continue;
      u64 k = 0;
      if (i < V) {
        const float x = xform_value(raw[u], a.xf.penalty, a.xf.eos, i, mw[u], has_mask, false, n_eos, ban_row);
        k = make_key64(order_key(x), static_cast<uint32_t>(i));
        if (i == 0 && x != x && a.emit_topk == kEmitArgmax) k = ~0ull;  // ArgMax starts from id 0 and nothing compares above a NaN
      }
      scratch[i] = k;
    }
  }
  __syncthreads();
  if (a.xf.use_penalty()) {
    const int32_t* h = a.xf.history + static_cast<size_t>(row) * a.xf.history_stride;
    const int hlen = a.xf.hist_len(row);
    for (int j = threadIdx.x; j < hlen; j += blockDim.x) {
      const int tok = h[j];
      if (tok < 0 || tok >= V) continue;
      bool dup = false;
      for (int jj = 0; jj < j && !dup; ++jj) dup = (h[jj] == tok);
      if (dup) continue;
      const float x = xform_value(lrow[tok], a.xf.penalty, a.xf.eos, tok, has_mask ? mrow[tok >> 5] : 0u, has_mask, true, n_eos, ban_row);
      scratch[tok] = (tok == 0 && x != x && a.emit_topk == kEmitArgmax) ? ~0ull : make_key64(order_key(x), static_cast<uint32_t>(tok));
    }
    __syncthreads();
  }
  // A row that asks for its k best (k <= 64) has them selected where the kernel provides the LDS for it; every other
  // row is sorted whole.  `sc`: the row's keys in descending order, as many as the row's parameters ask for.
  const u64* sc = scratch;
  int n_sorted = V;
  {
    const int kk = prm.k < V ? prm.k : V;
    if (select != nullptr && (a.emit_topk != 0 || prm.k > 1) && kk >= 1 && kk <= 64 && select_topk_desc(scratch, V, kk, *select)) {
      sc = select->list;
      n_sorted = kk;
    } else {
      sort_desc(scratch, n2, V);  // descending; entries from V on are 0
    }
  }
  if (a.emit_topk) {
    const int kk = prm.k < V ? prm.k : V;
    for (int j = threadIdx.x; j < kk; j += blockDim.x) {
      const uint32_t id = key64_index(sc[j]);
      a.out_tokens[static_cast<size_t>(row) * prm.k + j] = static_cast<int32_t>(id);
      if (a.out_scores) a.out_scores[static_cast<size_t>(row) * prm.k + j] = lrow[id];  // the value itself: keys do not tell -0 from +0
    }
    if (threadIdx.x == 0) atomicAdd(a.fallback_rows, 1u);
    return;
  }
  const float max_score = key_to_float(key64_okey(sc[0]));
  const float inv_temp = 1.0f / prm.temperature;
  const RowOutputs out = row_outputs(a, row);
  auto sorted = [=](int i) { return sc[i]; };
  auto exps = [=](int i) { return em::expf_exact((key_to_float(key64_okey(sc[i])) - max_score) * inv_temp); };
  block_sample_epilogue<EPI_ITEMS>(sorted, exps, n_sorted, V, prm, a.uniforms[row], out, sh);
  if (threadIdx.x == 0) atomicAdd(a.fallback_rows, 1u);
}

__device__ __forceinline__ int row_mode(mi355x_sample_params prm, int vocab, int chunks, int emit_topk = 0) {
  if (vocab <= 64 || chunks * kSmallCap > kAllCap) return kModeGeneral;
  if (emit_topk == kEmitArgmax) return kModeTopkSmall;
  if (prm.k > 1 || emit_topk) {
    const int kk = prm.k < vocab ? prm.k : vocab;
    return kk <= 64 ? kModeTopkSmall : (kk <= kLargeKMax ? kModeTopkLarge : kModeGeneral);
  }
  if (!(prm.p < 1.0f)) return kModeGeneral;  // sampling from the whole vocabulary: every element is a candidate
  return kModeNucleus;
}

// Depth below the row maximum (in score units) past which no element can lie strictly inside the
// nucleus: once exp((s-max)/T) <= (1-p)/(p*V) -- with a margin of e^2 for fp32 rounding -- the stop
// test prefix >= p*(prefix + (V-i-1)*e) of FindNucleus is certainly true, because prefix >= 1.
__device__ __forceinline__ float nucleus_depth(mi355x_sample_params prm, int vocab) {
  float d = 105.0f;  // exp underflows to exactly 0 below -103.98
  if (prm.p <= 0.0f) d = 0.0f;
  else if (prm.p < 0.999f) d = fminf(105.0f, logf(prm.p * static_cast<float>(vocab) / (1.0f - prm.p)) + 2.0f);
  return d * prm.temperature;
}

// The same depth when more is known about the prefix than that it holds the maximum: `mass` is (a lower bound of) the
// sum of exp((s - max)/T) over the elements within kDepthMassReach exponent units of the maximum.  An element deeper
// than those follows all of them in rank order, so its prefix is at least `mass` and the stop test holds once
// exp((s-max)/T) <= mass * (1-p)/(p*V), with a margin of e^0.5 for the roundings on both sides (of the reference's
// fp32 prefix, of this sum).  The depth never ends above the reach, or the sum would count elements that follow.
constexpr float kDepthWaveReach = 6.0f, kDepthBlockSlack = 3.0f;  // below a wave's maximum; of that below the chunk's
constexpr float kDepthMassReach = kDepthWaveReach + kDepthBlockSlack;
__device__ __forceinline__ float nucleus_depth(mi355x_sample_params prm, int vocab, float mass) {
  float d = 105.0f;
  if (prm.p <= 0.0f) d = 0.0f;
  else if (prm.p < 0.999f)
    d = fminf(105.0f, fmaxf(kDepthMassReach, logf(prm.p * static_cast<float>(vocab) / (1.0f - prm.p)) - logf(fmaxf(mass, 1.0f))) + 0.5f);
  return d * prm.temperature;
}

// Values of a published candidate slot that are not keys (a key's low half is ~id, far above these).
constexpr u64 kSlotEmpty = 1, kSlotOverflow = 2;
constexpr int kWaveListCap = 128;  // hits one wave can list per chunk
constexpr int kExtraCap = 2048;    // distinct history ids one chunk can hold; beyond, the row takes the exact path
constexpr uint32_t kChunkCntOverflow = 0xffffffffu;  // chunk_cnt of a nucleus chunk that gave up

// LDS of the fused kernel.
struct FusedShared {
  uint32_t hist_bits[kSChunk / 32];
  uint32_t mask_bits[kSChunk / 32];
  u64 wave_list[kSMaxWaves * kWaveListCap];  // each wave's hits of this chunk, before the sort
  u64 list_hi[64];          // second half of a long list, sorted ascending
  u64 own[64];              // the finishing workgroup's own list
  u64 lists[kAllCap / 4];   // first-level results of the finishing workgroup's merge (rows of > 4 chunks)
  uint32_t pool[64];
  uint32_t poisoned;              // the workgroup's copy of the flag that sends every row to the exact path
  uint32_t n_hits;                // hits of the chunk on the ranking route of the top-k rows
  uint32_t rank_failed;           // a wave or the chunk holds more hits than the ranking route provides for
  uint32_t wave_val[kSMaxWaves];
  u64 wave_val64[kSMaxWaves];
  uint32_t count, flag;
  uint32_t nan0;  // the processed logit of id 0 is a NaN (set in chunk 0; used by the argmax output)
  uint32_t n_extra;
  float extra_val[kExtraCap];     // processed logits of the history ids of this chunk ...
  uint32_t extra_idx[kExtraCap];  // ... and their ids
  SeqShared seq;
};

// Register element e of a thread (e = 0 .. elements per thread - 1) relative to the thread's first id: a thread
// owns VEC consecutive ids per 16-byte load (4 fp32 or 8 sixteen-bit values), its loads lie BLOCK * VEC ids apart.
template <int BLOCK, int VEC>
__device__ __forceinline__ constexpr int elem_offset(int e) {
  return (e / VEC) * BLOCK * VEC + e % VEC;
}
// Vocabulary id of element c of the thread's quad q (registers 4q .. 4q+3).
template <int BLOCK, int VEC>
__device__ __forceinline__ int elem_index(int chunk, int q, int c) {
  return chunk * kSChunk + static_cast<int>(threadIdx.x) * VEC + elem_offset<BLOCK, VEC>(q * 4 + c);
}

// The 32-entry table of expf_core, one entry per lane (lane & 31), fetched by lane shuffle.
struct LaneExp2Tab {
  uint32_t lo, hi;
  __device__ uint64_t operator()(uint32_t i) const {
    const uint32_t l = __shfl(lo, static_cast<int>(i), 64);
    const uint32_t h = __shfl(hi, static_cast<int>(i), 64);
    return (static_cast<uint64_t>(h) << 32) | l;
  }
};

__device__ __forceinline__ float read_lane(float x, int l) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), l));
}
__device__ __forceinline__ u64 read_lane(u64 x, int l) {
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(x), l);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(x >> 32), l);
  return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ double read_lane(double x, int l) {
  const u64 b = static_cast<u64>(__double_as_longlong(x));
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(b), l);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(b >> 32), l);
  return __longlong_as_double(static_cast<long long>((static_cast<u64>(hi) << 32) | lo));
}

// Epilogue for k <= 64 run by one wave: lane j holds the j-th best (key64), j < m.
// Follows ComputeSampledCategorical's top-k branch (src/sampling_distribution.h:243-281) and
// std::discrete_distribution literally: every fp32 sum is accumulated in rank order.  The fp64
// cumulative distribution is first evaluated in tree order on the raw weights; only if the draw lies
// within rounding distance of one of its values is it rebuilt with the reference's own sequence of
// operations (division by the sum, sequential partial sums), so the chosen position is always the
// sequential one.
__device__ __forceinline__ void wave_topk_epilogue(u64 key, int m, mi355x_sample_params prm, double u,
                                                   LaneExp2Tab tab, const RowOutputs& out) {
  const int lane = lane_id();
  m = __builtin_amdgcn_readfirstlane(m);
  const float score = key_to_float(key64_okey(key));
  const float max_score = read_lane(score, 0);
  const float inv_temp = 1.0f / prm.temperature;
  const float e_all = em::expf_core((score - max_score) * inv_temp, tab);
  const float e = lane < m ? e_all : 0.0f;
  const float sum = read_lane(wave_serial_prefix(e, m), m - 1);
  const float pr = sum > 0.0f ? e / sum : e;
  // cumulative probabilities, eight chain steps at a time; with a top-p cut the chain stops at the
  // first group that contains the cut (lanes below the number of steps done hold final values)
  const bool cut = prm.p > 0.0f && prm.p < 1.0f;
  float cum = 0.0f;
  int keep = m;
  for (int t = 0; t < m; t += 8) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float prev = __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(cum), 0x138, 0xf, 0xf, false));
      cum = prev + pr;
    }
    if (cut) {
      const int f = first_lane(__ballot(lane < t + 8 && lane < m && cum >= prm.p));
      if (f >= 0) {
        keep = f + 1;
        break;
      }
    }
  }
  keep = __builtin_amdgcn_readfirstlane(keep);
  const float keep_sum = read_lane(cum, keep - 1);
  const float inv = keep_sum > 0.0f ? 1.0f / keep_sum : 0.0f;
  const float q = pr * inv;
  int pos = 0;
  if (keep >= 2) {
    const double qd = lane < keep ? static_cast<double>(q) : 0.0;
    const double w = wave_scan_add(qd);
    const double total = read_lane(w, keep - 1);
    const double target = u * total;
    const double guard = 16.0 * static_cast<double>(keep) * 1.1102230246251565e-16 * total;
    const bool risky = __ballot(lane < keep - 1 && fabs(w - target) <= guard) != 0ull;
    if (!risky) {
      pos = first_lane(__ballot(lane < keep && (lane == keep - 1 || w >= target)));
    } else {
      const double dsum = read_lane(wave_serial_prefix(qd, keep), keep - 1);
      const double pn = qd / dsum;
      double cp = wave_serial_prefix(pn, keep);
      if (lane == keep - 1) cp = 1.0;
      pos = first_lane(__ballot(lane < keep && cp >= u));
    }
    if (pos < 0) pos = keep - 1;
    if (total != total) pos = 0;  // NaN weights: std::lower_bound over NaN quotients ends on 0
  }
  const uint32_t idx = key64_index(key);
  const int32_t tok = static_cast<int32_t>(__builtin_amdgcn_readlane(idx, pos));
  if (lane == 0) {
    *out.token = tok;
    if (out.kept_count) *out.kept_count = keep;
  }
  if (out.kept_ids && lane < keep && lane < out.kept_capacity) {
    out.kept_ids[lane] = static_cast<int32_t>(idx);
    if (out.kept_probs) out.kept_probs[lane] = q;
  }
}

// The token alone, for calls that ask for nothing else: k <= 64, lane j holds the j-th best, j < m.
// Every decision of wave_topk_epilogue -- where the top-p cut falls, which position the draw selects -- compares
// a sequentially rounded fp32 or fp64 sum with a fixed number.  Here both are taken from ONE fp64 prefix sum of
// the exponentials in tree order: S_j / S_{m-1} differs from the reference's cumulative probability by less than
// 2 * 63 * 2^-24 + 2^-23 < 8e-6 (two sequential fp32 sums of at most 64 positive terms and one division), and
// S_j / S_{keep-1} from its fp64 cumulative distribution by less than 3e-7 (the common factors cancel; two fp32
// roundings per weight remain).  A comparison that falls inside those bands decides nothing: the function then
// returns false and the caller runs wave_topk_epilogue, so the token is always the sequential one.
__device__ __forceinline__ bool wave_topk_token_fast(u64 key, int m, mi355x_sample_params prm, float inv_temp, double u,
                                                     LaneExp2Tab tab, int32_t* token) {
  const int lane = lane_id();
  m = __builtin_amdgcn_readfirstlane(m);
  const float score = key_to_float(key64_okey(key));
  const float max_score = read_lane(score, 0);
  const float e_all = em::expf_core((score - max_score) * inv_temp, tab);
  const double ed = lane < m ? static_cast<double>(e_all) : 0.0;
  const double S = wave_scan_add(ed);
  const double total = read_lane(S, m - 1);
  bool decided = total >= 1.0 && total <= 128.0;  // the best element weighs exp(0) = 1; false for NaN weights
  int keep = m;
  if (prm.p > 0.0f && prm.p < 1.0f) {
    const double mass = static_cast<double>(prm.p) * total;
    const bool in_band = lane < m && fabs(S - mass) <= 1e-5 * total;
    decided = decided && __ballot(in_band) == 0ull;
    const int f = first_lane(__ballot(lane < m && S >= mass));
    if (f >= 0) keep = f + 1;
  }
  int pos = 0;
  if (keep >= 2) {
    const double kept_total = read_lane(S, keep - 1);
    const double target = u * kept_total;
    const bool in_band = lane < keep - 1 && fabs(S - target) <= 1e-6 * kept_total;
    decided = decided && __ballot(in_band) == 0ull;
    pos = first_lane(__ballot(lane == keep - 1 || S >= target));
  }
  if (!decided) return false;
  const uint32_t idx = key64_index(key);
  const int32_t tok = static_cast<int32_t>(__builtin_amdgcn_readlane(idx, pos));
  if (lane == 0) *token = tok;
  return true;
}

static __device__ const uint64_t g_exp2_tab[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL,
};

// Workgroup barrier that orders LDS accesses only: unlike __syncthreads() it does not wait for the
// global loads still in flight.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// block_max with barriers that do not wait for global memory.
template <int kSWaves, typename T>
__device__ __forceinline__ T block_max_lds(T v, T* scratch) {
  v = wave_max(v);
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  if (lane == 0) scratch[wave] = v;
  lds_barrier();
  static_assert(kSWaves <= 16, "a lane per wave inside one row of lanes");
  const T r = row16_max<T>(lane < kSWaves ? scratch[lane] : T(0));  // lane w looks at wave w's
  lds_barrier();
  return r;
}

// The kk-th largest of the values the block's threads offer (N per thread; 1 <= kk <= N * blockDim.x), every thread
// gets it: a radix selection from the top byte down.  A round counts the offers that still match the bytes found so
// far into 256 bins with LDS atomics (eight copies of every bin, chosen by the lane, so that offers sharing a byte --
// all of them share the first -- do not queue on one word), 256 threads sum the copies of one bin each, scan the
// sums from the top digit down and the thread whose bin holds the wanted rank publishes digit and rank.  No sort,
// three barriers a round.  bins: kKthBinWords words of LDS that no thread uses for anything else until the function
// returns; blockDim.x >= 256.
constexpr int kKthBinCopies = 8, kKthBinWords = 256 * kKthBinCopies + 16;
template <int N>
__device__ __forceinline__ uint32_t block_kth_largest(const uint32_t (&offer)[N], int kk, uint32_t* bins) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  uint32_t* const wave_sum_of = bins + 256 * kKthBinCopies;  // [4], then the published digit and rank
  uint32_t* const pick = wave_sum_of + 4;
  for (int i = tid; i < 256 * kKthBinCopies; i += blockDim.x) bins[i] = 0u;
  lds_barrier();
  uint32_t prefix = 0u, need = static_cast<uint32_t>(kk);
#pragma unroll
  for (int round = 0; round < 4; ++round) {
    const int shift = 24 - 8 * round;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const bool match = round == 0 || (offer[j] >> (shift + 8)) == (prefix >> (shift + 8));
      if (match) atomicAdd(&bins[((offer[j] >> shift) & 255u) * kKthBinCopies + (lane & (kKthBinCopies - 1))], 1u);
    }
    lds_barrier();
    uint32_t count = 0u, upto = 0u;
    const uint32_t digit = 255u - static_cast<uint32_t>(tid);  // thread t owns digit 255 - t: a prefix sum counts the digits above
    if (tid < 256) {
#pragma unroll
      for (int i = 0; i < kKthBinCopies; ++i) count += bins[digit * kKthBinCopies + i];
      upto = wave_prefix_sum<uint32_t>(count);
      if (lane == 63) wave_sum_of[wave] = upto;
    }
    lds_barrier();
    if (tid < 256) {
      uint32_t above = upto - count;
      for (int w = 0; w < wave; ++w) above += wave_sum_of[w];
      if (above < need && need <= above + count) {
        pick[0] = digit;
        pick[1] = need - above;
      }
    }
    if (round < 3)
      for (int i = tid; i < 256 * kKthBinCopies; i += blockDim.x) bins[i] = 0u;  // (every read of this round's bins lies before the last barrier)
    lds_barrier();
    prefix |= pick[0] << shift;
    need = pick[1];
  }
  lds_barrier();  // (the words are free again)
  return prefix;
}

// Applies the two LDS bitmaps of a chunk to the registers of a thread: an id whose bit in `allowed` is
// clear becomes kLowest, an id whose bit in `history` is set becomes NaN (its processed value lives in
// the extras list).  Branch-free: the bit, spread over a word, selects between the two bit patterns.
template <int kSBlock, int VEC, bool ALLOWED, bool HISTORY>
__device__ __forceinline__ void mask_registers(float (&v)[kSChunk / kSBlock], const uint32_t* allowed,
                                               const uint32_t* history, int tid) {
  constexpr int kSVec = kSChunk / (kSBlock * 4);
#pragma unroll
  for (int j = 0; j < kSVec; ++j) {
    const int rel0 = tid * VEC + elem_offset<kSBlock, VEC>(j * 4);
    const uint32_t anib = ALLOWED ? allowed[rel0 >> 5] >> (rel0 & 31) : 0u;
    const uint32_t hnib = HISTORY ? history[rel0 >> 5] >> (rel0 & 31) : 0u;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint32_t x = __float_as_uint(v[j * 4 + c]);
      if (ALLOWED) {
        uint32_t keep = static_cast<uint32_t>(static_cast<int32_t>(anib << (31 - c)) >> 31);
        asm volatile("" : "+v"(keep));  // stays a bitwise select (one instruction) instead of compare + select
        x = (x & keep) | (0xff7fffffu & ~keep);  // bits of kLowest
      }
      if (HISTORY) {
        const uint32_t drop = static_cast<uint32_t>(static_cast<int32_t>(hnib << (31 - c)) >> 31);
        x |= drop;  // all ones is a NaN
      }
      v[j * 4 + c] = __uint_as_float(x);
    }
    if ((j & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // at most eight bitmap words in registers at a time
  }
}

// Streaming pass of one (row, chunk) of a top-k<=64 or nucleus row.  Returns true when this workgroup
// must run the general path for the row (it was the last to arrive and the fast path declined).
template <typename InT, bool NUCLEUS, bool XFORM, bool LARGEK = false, bool ARGMAX = false>
__device__ __forceinline__ bool stream_row(const SampleArgs& a, int row, const void* row0, int chunk,
                                           mi355x_sample_params prm, FusedShared& sm) {
  constexpr int kSBlock = NUCLEUS ? kNucleusBlock : kTopkBlock;  // threads of this workgroup
  constexpr int kSWaves = kSBlock / 64;
  constexpr int kSVec = kSChunk / (kSBlock * 4);  // quads of logits per thread (fp32 rows: its 128-bit loads)
  constexpr int kSElems = kSVec * 4;              // logits held in registers per thread
  constexpr int VEC = 16 / static_cast<int>(sizeof(InT));  // logits per 128-bit load
  constexpr int kSLoads = kSElems / VEC;                   // 128-bit loads per thread
  const int V = a.vocab;
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  u64* big_row = a.big + static_cast<size_t>(row) * a.big_stride;
  const InT* lrow = static_cast<const InT*>(row0);
  constexpr bool kOneRun = XFORM && sizeof(InT) == 4;  // the loads of a chunk are one straight run, see there
  // (The loads below are 128-bit loads that assume no more than their elements' alignment, v4f_any / v4u_any: rows
  // that do not start on a 16-byte boundary used to be read element by element, 64 loads per thread where 16 do,
  // 3.5 us more per step at 64 x 50257.)
  const float kNaN = __uint_as_float(0x7fc00000u);  // marks ids >= vocab: never a maximum, never >= a bound
  // The bitmap words and the first history ids of this thread are requested before the logits: loads come back in
  // the order they were asked for, and the history has a chain of its own to start (mark the ids, read their logits
  // again, penalise them) that should run while the logits arrive, not after them.
  constexpr int kWordsPerThread = kSChunk / 32 / kSBlock;  // bitmap words a thread stages
  static_assert(kWordsPerThread >= 1 && kSChunk / 32 == kWordsPerThread * kSBlock, "whole bitmap words per thread");
  const bool active = XFORM && a.xf.active();  // kernels without logits processing carry none of its code
  const bool pen = active && a.xf.use_penalty();
  const bool has_mask = active && a.xf.mask != nullptr;
  const int words = (V - 1) / 32 + 1;
  const uint32_t* mrow = has_mask ? a.xf.mask + static_cast<size_t>(row) * words : nullptr;
  const int32_t* hist = pen ? a.xf.history + static_cast<size_t>(row) * a.xf.history_stride : nullptr;
  // The first two history ids of every thread are requested before the logits: as many as the common length says,
  // or, where rows have lengths of their own, as many as a row of the history holds (what lies beyond the row's
  // length is fetched and not looked at).  A history shared by all rows (stride 0) has no such bound: its ids are
  // fetched once the length is there.
  const bool hist_ahead = pen && (a.xf.history_lens == nullptr || a.xf.history_stride > 0);
  const int hist_ahead_ids = a.xf.history_lens == nullptr ? a.xf.history_len : a.xf.history_stride;
  int hist_pre[2] = {-1, -1};
  uint32_t mask_pre[kWordsPerThread];
  // Kernels with logits processing also request the row's history length (where rows have lengths of their own) and
  // the flag that sends every row to the exact path before the logits: whatever is requested before them arrives
  // before them, so the processing's preparations run while the logits are in flight.  (Both used to be loaded where
  // they were first needed, behind the logits, each a round trip of its own.)
  int row_hlen = 0;
  uint32_t flag_pre = 0u;
  if constexpr (XFORM) {
    const int uniform_hlen = arg_now(a.xf.history_len);
    row_hlen = uniform_hlen;
    // (indexed through a lane's register, so that the length stays in one: as a value common to the wave it would be
    // moved to a scalar register at once, which waits for it)
    if (active && a.xf.history_lens != nullptr) row_hlen = a.xf.history_lens[row + (lane >> 6)];
    if (tid == 0) flag_pre = a.fallback_rows[1];
  }
#pragma unroll
  for (int q = 0; q < 2; ++q)
    if (hist_ahead && tid + q * kSBlock < hist_ahead_ids) hist_pre[q] = hist[tid + q * kSBlock];
#pragma unroll
  for (int q = 0; q < kWordsPerThread; ++q) {
    mask_pre[q] = ~0u;
    if (has_mask) {
      const int w = chunk * (kSChunk / 32) + tid + q * kSBlock;
      mask_pre[q] = w < words ? mrow[w] : 0u;
    }
  }
  float v[kSElems];
  // ---- logits processing ----------------------------------------------------------------------
  // Grammar mask and min-length masking reach the registers as one LDS bitmap of allowed ids (a clear
  // bit -> kLowest; ids past the vocabulary count as allowed and keep their NaN).  The ids of the row's
  // history are few and their processing (a correctly rounded division, the n-gram ban) is long, so
  // they leave the register arrays altogether: a second bitmap turns them into NaN there, and the
  // threads that marked them compute their processed values into a short list in LDS, `extras`, which
  // every later phase visits next to the registers.
  // All of this but the application to the registers needs only what was requested before the logits, and it is
  // called inside every path of the loads below, right behind that path's requests: there the number of requests
  // behind the earlier ones is known exactly and a wait for those leaves the logits in flight.  (Where the paths
  // join again the compiler has to assume the fewest requests any path may have made, none, and waits for the
  // logits themselves at the first use of an earlier value: the preparations then start when the logits are there.)
  uint32_t n_extra = 0u;
  bool extra_overflow = false;
  int n_eos_row = 0;
  auto xform_prep = [&]() {
    // One thread reads the flag that sends every row to the exact path, and the workgroup looks at that copy behind
    // its first barrier: read by every wave for itself, at its own time, a flag raised in between would send some
    // waves of a workgroup one way and the rest the other, with barriers waiting on both sides.
    if (tid == 0) sm.poisoned = flag_pre;
    if (!active) return;
    // Xform::eos_count with the length that was requested before the logits
    const int n_eos = (a.xf.history_lens && a.xf.min_length > 0 && row_hlen >= a.xf.min_length) ? 0 : a.xf.n_eos;
    n_eos_row = n_eos;
    if (tid == 0) {
      sm.n_extra = 0u;
      sm.nan0 = 0u;
    }
#pragma unroll
    for (int q = 0; q < kWordsPerThread; ++q) {
      const int i = tid + q * kSBlock;
      const int w = chunk * (kSChunk / 32) + i;
      uint32_t word = mask_pre[q];
      for (int e = 0; e < n_eos; ++e)
        if ((a.xf.eos[e] >> 5) == w) word &= ~(1u << (a.xf.eos[e] & 31));
      const int n_real = V - w * 32;  // ids of this word inside the vocabulary
      if (n_real < 32) word |= n_real <= 0 ? ~0u : (~0u << n_real);
      sm.mask_bits[i] = word;
      sm.hist_bits[i] = 0u;
    }
    lds_barrier();
    if (pen) {
      const int hlen = row_hlen;
      const float penalty = a.xf.penalty;
      const uint32_t* ban_row = a.xf.ban_row(row, V);
      // the thread that is first to mark an id computes its processed value
      auto visit = [&](int id) {
        const int rel = id - chunk * kSChunk;
        if (rel >= 0 && rel < kSChunk && id < V) {
          const uint32_t bit = 1u << (rel & 31);
          if (!(atomicOr(&sm.hist_bits[rel >> 5], bit) & bit)) {
            const uint32_t slot = atomicAdd(&sm.n_extra, 1u);
            if (slot < static_cast<uint32_t>(kExtraCap)) {
              const uint32_t mw = has_mask ? mrow[id >> 5] : 0u;
              const float val = xform_value(load_one<InT>(lrow, id), penalty, a.xf.eos, id, mw, has_mask, true, n_eos, ban_row);
              sm.extra_val[slot] = val;
              sm.extra_idx[slot] = static_cast<uint32_t>(id);
              if (id == 0 && val != val) sm.nan0 = 1u;
            }
          }
        }
      };
      int first = tid;
      if (hist_ahead) {
        if (tid < hlen) visit(hist_pre[0]);
        if (tid + kSBlock < hlen) visit(hist_pre[1]);
        first = tid + 2 * kSBlock;
      }
      for (int i = first; i < hlen; i += kSBlock) visit(hist[i]);
      lds_barrier();
      n_extra = sm.n_extra;
      extra_overflow = n_extra > static_cast<uint32_t>(kExtraCap);  // the row takes the exact path
      if (extra_overflow) n_extra = 0u;
    }
  };
  // a chunk that lies inside its row requests its loads without a test between them
  const bool whole_chunk = (chunk + 1) * kSChunk <= V;
  if constexpr (kOneRun) {
    // Kernels with logits processing request the loads of a chunk in one straight run, whatever the row's end and
    // wherever the row starts: 128-bit loads that only need their elements' alignment (the hardware reads from any
    // address; rows that do not start on a 16-byte boundary cost it more cache lines), a load that would cross the
    // row's end reads the row's last four elements instead, one beyond it the row's first, and the registers are put
    // right further down, after the processing's preparations.  The number of requests behind the earlier ones
    // (history ids, mask words, the flag) is then known where those are first used, and the wait for them leaves the
    // logits in flight.  With a branch per kind of chunk or row the compiler has to assume, where the branches join,
    // the fewest requests any of them may have made -- and ahead of any joint continuation of two such paths it
    // waits for everything -- so that the preparations would start when the logits are there.
#pragma unroll
    for (int j = 0; j < kSLoads; ++j) {
      const int i0 = elem_index<kSBlock, VEC>(chunk, j, 0);
      const int from = i0 + 4 <= V ? i0 : (i0 < V ? V - 4 : 0);
      const v4f_any q = __builtin_nontemporal_load(reinterpret_cast<const v4f_any*>(lrow + from));
      v[j * 4 + 0] = q.x;
      v[j * 4 + 1] = q.y;
      v[j * 4 + 2] = q.z;
      v[j * 4 + 3] = q.w;
    }
    xform_prep();
  } else if constexpr (VEC == 4) {
    if (whole_chunk) {
      const v4f_any* src = reinterpret_cast<const v4f_any*>(lrow + static_cast<size_t>(chunk) * kSChunk) + tid;
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        const v4f_any q = __builtin_nontemporal_load(src + j * kSBlock);
        v[j * 4 + 0] = q.x;
        v[j * 4 + 1] = q.y;
        v[j * 4 + 2] = q.z;
        v[j * 4 + 3] = q.w;
      }
    } else {
      // The row's last chunk.  Every register is set to NaN before the first load is requested and the loads that
      // lie inside the row are requested back to back: a register written after a load into it was requested
      // (even by other lanes) makes the compiler wait for that load first, which strings the sixteen loads of a
      // thread out one memory round trip after the other.  The one load that straddles the row's end follows.
#pragma unroll
      for (int e = 0; e < kSElems; ++e) asm volatile("v_mov_b32 %0, 0x7fc00000" : "=v"(v[e]));
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        const int i0 = elem_index<kSBlock, VEC>(chunk, j, 0);
        if (i0 + 4 <= V) {
          const v4f_any q = __builtin_nontemporal_load(reinterpret_cast<const v4f_any*>(lrow + i0));
          v[j * 4 + 0] = q.x;
          v[j * 4 + 1] = q.y;
          v[j * 4 + 2] = q.z;
          v[j * 4 + 3] = q.w;
        }
      }
      if ((V & 3) != 0) {
#pragma unroll
        for (int j = 0; j < kSLoads; ++j) {
          const int i0 = elem_index<kSBlock, VEC>(chunk, j, 0);
          if (i0 < V && i0 + 4 > V) {
#pragma unroll
            for (int c = 0; c < 3; ++c)
              if (i0 + c < V) v[j * 4 + c] = load_one<InT>(lrow, i0 + c);
          }
        }
      }
    }
  } else {
    v4u raw[kSLoads];
    if constexpr (XFORM) {
      // Sixteen-bit rows of the kernels with logits processing: eight 128-bit loads per thread in one straight run,
      // like the fp32 rows' sixteen, and the processing's preparations right behind them.  A load that would cross
      // the row's end reads from the row's start instead; the (at most seven) elements of the one group of eight
      // that straddles the end are fetched once more, one by one and by every thread alike, and the registers past
      // the end are put right after the widening.
      float row_end[VEC - 1];
      if (!whole_chunk) {  // (ahead of the run, which so is the same number of requests for every chunk)
#pragma unroll
        for (int c = 0; c < VEC - 1; ++c) {
          const int i = (V & ~(VEC - 1)) + c;
          row_end[c] = load_one<InT>(lrow, i < V ? i : 0);
        }
      }
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        const int i0 = elem_index<kSBlock, VEC>(chunk, 2 * j, 0);
        raw[j] = __builtin_nontemporal_load(reinterpret_cast<const v4u_any*>(lrow + (i0 + VEC <= V ? i0 : 0)));
      }
      xform_prep();
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        if constexpr (sizeof(InT) == 2 && !__is_same(InT, bf16_t)) widen_half8(raw[j], &v[j * VEC]);
        else widen_bf16x8(raw[j], &v[j * VEC]);
      }
      if (!whole_chunk) {
        const int r = V & (VEC - 1);  // elements of the straddling group that lie inside the row
#pragma unroll
        for (int j = 0; j < kSLoads; ++j) {
          const int i0 = elem_index<kSBlock, VEC>(chunk, 2 * j, 0);
          if (i0 + VEC > V) {
            const bool straddles = i0 < V;
#pragma unroll
            for (int c = 0; c < VEC; ++c) v[j * VEC + c] = (straddles && c < r) ? row_end[c < VEC - 1 ? c : 0] : kNaN;
          }
        }
      }
    } else {
      // sixteen-bit rows: all loads are requested before the first is widened
      uint32_t whole = 0u;  // bit j: load j lies inside the row
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        const int i0 = elem_index<kSBlock, VEC>(chunk, 2 * j, 0);
        if (i0 + VEC <= V) {
          raw[j] = __builtin_nontemporal_load(reinterpret_cast<const v4u_any*>(lrow + i0));
          whole |= 1u << j;
        }
      }
#pragma unroll
      for (int j = 0; j < kSLoads; ++j) {
        const int i0 = elem_index<kSBlock, VEC>(chunk, 2 * j, 0);
        if ((whole >> j) & 1u) {
          if constexpr (sizeof(InT) == 2 && !__is_same(InT, bf16_t)) widen_half8(raw[j], &v[j * VEC]);
          else widen_bf16x8(raw[j], &v[j * VEC]);
        } else {
#pragma unroll
          for (int c = 0; c < VEC; ++c) v[j * VEC + c] = (i0 + c < V) ? load_one<InT>(lrow, i0 + c) : kNaN;
        }
      }
    }
  }
  if constexpr (!XFORM) {
    if (tid == 0) sm.poisoned = a.fallback_rows[1];
  }
  // The arguments the phases after the streaming pass need are fetched now, while the logits are in
  // flight, instead of one by one where they are first used.
  const int n_chunks = arg_now(a.chunks);
  u64* const cand_small = arg_now(a.cand_small);
  const double* const uniforms = arg_now(a.uniforms);
  const int emit_topk = arg_now(a.emit_topk);
  const int poll_limit = arg_now(a.poll_limit);
  const RowOutputs outputs = {arg_now(a.out_tokens) + row,
                              arg_now(a.kept_count),
                              arg_now(a.kept_ids),
                              arg_now(a.kept_probs),
                              arg_now(a.kept_capacity)};
  if constexpr (XFORM) {
    // fp32 rows: the registers past the row's end, see the loads above
    if constexpr (kOneRun) {
      if (!whole_chunk) {
#pragma unroll
        for (int j = 0; j < kSLoads; ++j) {
          const int i0 = elem_index<kSBlock, VEC>(chunk, j, 0);
          if (i0 + 4 > V) {  // elements V-4 .. V-1 in the registers where i0 .. V-1 belong, or nothing of the row
            const int r = i0 < V ? V - i0 : 0;  // elements of the quad that lie inside the row
            const float q1 = v[j * 4 + 1], q2 = v[j * 4 + 2], q3 = v[j * 4 + 3];
            v[j * 4 + 0] = r == 0 ? kNaN : (r == 1 ? q3 : (r == 2 ? q2 : q1));
            v[j * 4 + 1] = r < 2 ? kNaN : (r == 2 ? q3 : q2);
            v[j * 4 + 2] = r < 3 ? kNaN : q3;
            v[j * 4 + 3] = kNaN;
          }
        }
      }
    }
    if (active) {
      // without a grammar mask and without EOS masking every id is allowed (ids past the vocabulary are NaN already)
      if (has_mask || n_eos_row > 0) mask_registers<kSBlock, VEC, true, true>(v, sm.mask_bits, sm.hist_bits, tid);
      else mask_registers<kSBlock, VEC, false, true>(v, sm.mask_bits, sm.hist_bits, tid);
    }
  }
  // per-thread maximum in the float domain (fmaxf skips NaN), keeping the maximum of every float4
  float qm[kSVec];
  float fm = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < kSVec; ++j) {
    qm[j] = fmaxf(fmaxf(v[j * 4], v[j * 4 + 1]), fmaxf(v[j * 4 + 2], v[j * 4 + 3]));
    fm = fmaxf(fm, qm[j]);
  }
  for (uint32_t i = tid; i < n_extra; i += kSBlock) fm = fmaxf(fm, sm.extra_val[i]);
  // 0: the thread holds no element
  const uint32_t lmax = (elem_index<kSBlock, VEC>(chunk, 0, 0) < V || static_cast<uint32_t>(tid) < n_extra) ? order_key(fm) : 0u;
  if (tid == 0) {
    sm.count = 0u;
    if constexpr (!NUCLEUS) {
      // id 0's processed value is v[0] unless id 0 is in the history (then its owner has set the flag)
      const bool in_history = XFORM && pen && (sm.hist_bits[0] & 1u) != 0u;
      const bool is_nan = chunk == 0 && !in_history && v[0] != v[0];
      if (!(XFORM && active)) sm.nan0 = is_nan ? 1u : 0u;
      else if (is_nan) sm.nan0 = 1u;
    }
  }

  if constexpr (NUCLEUS) {
    // Everything within nucleus_depth of the chunk maximum goes to the row's key buffer, in no
    // particular order (the finish kernel sorts).  A wave counts its candidates, reserves a range of
    // the chunk's list with one LDS atomic and fills it; the slot of a candidate is the wave's running
    // count plus the number of candidate lanes below.
    // Rows with 64 < k <= kLargeKMax come here too: their candidates are the elements that reach the
    // k-th best of the chunk's per-thread maxima (or, for larger k, of the maxima of the quarters of every thread's
    // elements: at least k elements do; with fewer than k numbers, all), which contain the chunk's k best.
    static_assert(kLargeKOneOffer <= kSBlock && 4 * kLargeKOneOffer <= 4 * kSBlock && kLargeKMax <= kSChunk && kSElems % 4 == 0,
                  "one offer per thread, four, or every element");
    static_assert(sizeof(sm.wave_list) >= kKthBinWords * sizeof(uint32_t) && kSBlock >= 256, "the selection's bins lie in the hit lists' LDS");
    constexpr bool large_k = LARGEK;
    uint32_t cmax = 0u;
    float thr = -__builtin_inff();
    if constexpr (!LARGEK) {
      // The chunk's maximum and, with it, the mass of the chunk's elements near that maximum, which bounds the prefix
      // of everything deeper (any element of the row that lies deeper than this chunk's threshold follows them in
      // rank order) and so moves the threshold up.  One exchange between the waves serves both: a wave sums
      // exp((s - its own maximum)/T) over its elements within kDepthWaveReach of that maximum (whole-wave tests
      // skip the exponentials where no lane has such an element: hardly any has), and the waves whose maximum lies
      // within kDepthBlockSlack of the chunk's contribute, rescaled.
      const uint32_t wkey = wave_max<uint32_t>(lmax);
      const float fw = key_to_float(wkey), inv_t = 1.0f / prm.temperature;  // (no number in the wave: NaN, every test fails)
      const float lim = fw - kDepthWaveReach * prm.temperature;
      float near = 0.0f;
#pragma unroll
      for (int e = 0; e < kSElems; ++e) {
        const bool in = v[e] >= lim;
        if (__ballot(in) != 0ull) near += in ? __expf((v[e] - fw) * inv_t) : 0.0f;
      }
      for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
        const float ev = i0 + tid < n_extra ? sm.extra_val[i0 + tid] : kNaN;
        near += ev >= lim ? __expf((ev - fw) * inv_t) : 0.0f;
      }
      near = wave_sum<float>(near);
      if (lane == 0) sm.wave_val64[wave] = (static_cast<u64>(wkey) << 32) | __float_as_uint(near);
      lds_barrier();
      const u64 of_wave = lane < kSWaves ? sm.wave_val64[lane] : 0;
      cmax = wave_max<uint32_t>(static_cast<uint32_t>(of_wave >> 32));
      const float fcmax = key_to_float(cmax);
      const float below = (key_to_float(static_cast<uint32_t>(of_wave >> 32)) - fcmax) * inv_t;
      const float mass =
          wave_sum<float>(below >= -kDepthBlockSlack ? __uint_as_float(static_cast<uint32_t>(of_wave)) * __expf(below) : 0.0f);
      lds_barrier();
      if (cmax != 0u) thr = fcmax - nucleus_depth(prm, V, mass);
    } else {
      cmax = block_max<uint32_t>(lmax, sm.wave_val);
    }
    if (large_k) {
      const int kk = prm.k < V ? prm.k : V;
      uint32_t* const bins = reinterpret_cast<uint32_t*>(sm.wave_list);
      uint32_t kth;
      if (kk <= kLargeKOneOffer) {
        const uint32_t offer[1] = {lmax};
        kth = block_kth_largest<1>(offer, kk, bins);
      } else {
        // the best element of each quarter of the thread's registers (up to k = 2048) or every element (a k that
        // close to the number of offers would make a bound from maxima useless), as order keys; the thread's share
        // of the history ids' list counts for the first.  At least k elements reach the k-th best of those offers,
        // or fewer than k exist and all are kept
        auto group_maxima = [&](auto groups) {
          constexpr int G = decltype(groups)::value;
          uint32_t best[G];
#pragma unroll
          for (int q = 0; q < G; ++q) best[q] = 0u;
#pragma unroll
          for (int e = 0; e < kSElems; ++e) {
            const uint32_t key = order_key(v[e]);  // 0 for NaN: no element
            best[e / (kSElems / G)] = key > best[e / (kSElems / G)] ? key : best[e / (kSElems / G)];
          }
          for (uint32_t i = tid; i < n_extra; i += kSBlock) {
            const uint32_t key = order_key(sm.extra_val[i]);
            best[0] = key > best[0] ? key : best[0];
          }
          return block_kth_largest<G>(best, kk, bins);
        };
        kth = kk <= 4 * kLargeKOneOffer ? group_maxima(std::integral_constant<int, 4>{}) : group_maxima(std::integral_constant<int, kSElems>{});
      }
      if (kth != 0u) thr = key_to_float(kth);
    }
    // First pass: the wave's number of candidates, and (nucleus rows) the thread's best element below the threshold,
    // from the same compare.
    uint32_t wcnt = 0u;
    float fb = -__builtin_inff();
#pragma unroll
    for (int e = 0; e < kSElems; ++e) {
      const bool cand = v[e] >= thr;  // false for NaN
      wcnt += static_cast<uint32_t>(__popcll(__ballot(cand)));
      if constexpr (!LARGEK) fb = fmaxf(fb, cand ? -__builtin_inff() : v[e]);  // (fmaxf passes a NaN by)
    }
    for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
      const uint32_t i = i0 + tid;
      wcnt += static_cast<uint32_t>(__popcll(__ballot(i < n_extra && sm.extra_val[i] >= thr)));
    }
    uint32_t woff = 0u;
    if (lane == 0) woff = atomicAdd(&sm.count, wcnt);
    woff = __builtin_amdgcn_readfirstlane(woff);
    // Second pass: the stores.  The list holds (raw float bits, ~id): the finish kernel turns the bits
    // into order keys.  The compares are made afresh against a copy of the threshold the compiler
    // cannot identify with the first one, so that the 64 lane masks of the first pass need not stay
    // alive.  Nothing below waits for the stores.
    char* const dst = reinterpret_cast<char*>(big_row + static_cast<size_t>(chunk) * kSChunk);
    float thr2 = thr;
    asm volatile("" : "+v"(thr2));
    const uint32_t nid0 = ~static_cast<uint32_t>(elem_index<kSBlock, VEC>(chunk, 0, 0));  // ~(id0 + d) = ~id0 - d
#pragma unroll
    for (int e = 0; e < kSElems; ++e) {
      const bool cand = v[e] >= thr2;
      const u64 b = __ballot(cand);
      if (cand) {
        const uint32_t pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(b >> 32),
                                                       __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(b), woff));
        const uint32_t nid = nid0 - static_cast<uint32_t>(elem_offset<kSBlock, VEC>(e));
        *reinterpret_cast<u64*>(dst + pos * 8u) = make_key64(__float_as_uint(v[e]), ~nid);
      }
      woff += static_cast<uint32_t>(__popcll(b));
      __builtin_amdgcn_sched_barrier(0);  // keeps the keys of later elements from being built early
    }
    u64 extra_below = 0;  // the best of this thread's extras below the threshold, as a whole key
    for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
      const uint32_t i = i0 + tid;
      const float ev = i < n_extra ? sm.extra_val[i] : kNaN;
      const uint32_t ei = i < n_extra ? sm.extra_idx[i] : 0u;
      const bool cand = ev >= thr2;
      const u64 b = __ballot(cand);
      if (cand) {
        const uint32_t pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(b >> 32),
                                                       __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(b), woff));
        *reinterpret_cast<u64*>(dst + pos * 8u) = make_key64(__float_as_uint(ev), ei);
      }
      woff += static_cast<uint32_t>(__popcll(b));
      const u64 key = make_key64(order_key(ev), ei);
      if (ev < thr2 && key > extra_below) extra_below = key;
    }
    u64 best_below = 0;
    if constexpr (!LARGEK) {  // (a top-k row's kept set ends with its k-th element: nothing below the list is ever needed)
      // The best element below the threshold, first of equals: the block agrees on the best score, then
      // the few threads that hold it look up its lowest id.
      float thr3 = thr;
      asm volatile("" : "+v"(thr3));
      uint32_t fbk = 0u;  // 0: the thread has no element below the threshold
      if (fb > -__builtin_inff()) {
        fbk = order_key(fb);
      } else if (thr3 > -__builtin_inff()) {  // an element equal to -inf is one, too
        bool any = false;
#pragma unroll
        for (int e = 0; e < kSElems; ++e) any = any || v[e] == -__builtin_inff();
        if (any) fbk = order_key(-__builtin_inff());
      }
      const uint32_t ebk = key64_okey(extra_below);
      const uint32_t own = fbk > ebk ? fbk : ebk;
      const uint32_t wbk = wave_max<uint32_t>(own);  // (the wave first: one exchange between the waves, of whole keys)
      if (wbk != 0u && own == wbk) {
        best_below = ebk == wbk ? extra_below : 0;
        if (fbk == wbk) {
          const float bbf = key_to_float(wbk);
          int fe = 0;
#pragma unroll
          for (int e = kSElems - 1; e >= 0; --e)
            if (v[e] == bbf) fe = e;
          const u64 key = make_key64(wbk, static_cast<uint32_t>(elem_index<kSBlock, VEC>(chunk, fe >> 2, fe & 3)));
          best_below = key > best_below ? key : best_below;
        }
      }
    }
    if constexpr (!LARGEK) {
      best_below = wave_max<u64>(best_below);
      if (lane == 0) sm.wave_val64[wave] = best_below;
    }
    lds_barrier();  // (also orders the atomics on sm.count)
    if constexpr (!LARGEK) best_below = wave_max<u64>(lane < kSWaves ? sm.wave_val64[lane] : 0);
    if (tid == 0) {
      const size_t ci = static_cast<size_t>(row) * a.chunks + chunk;
      a.chunk_cnt[ci] = extra_overflow ? kChunkCntOverflow : sm.count;
      a.chunk_max[ci] = cmax;
      a.chunk_thr[ci] = order_key(thr);
      a.chunk_next[ci] = best_below;
    }
    return false;
  }

  // A finishing workgroup that once gave up waiting may have left published lists behind; from then on
  // (the flag word next to the fallback counter, copied to sm.poisoned) every row takes the exact path, which
  // reads no such state.
  if constexpr (ARGMAX) {
    // ---- argmax ---------------------------------------------------------------------------------
    // ArgMax (src/search.h:9-29) keeps id 0 unless a later value compares greater: the largest value, the
    // lowest id among equals, NaNs never win, and a NaN at id 0 wins outright.  A thread's candidate is
    // the first of its elements that equals its maximum; the key (order key, ~id) orders candidates the
    // same way, so the row's answer is the largest key: no bound, no lists, no sort.  Every chunk
    // publishes its best key in the first entry of its candidate slots; the workgroup of the row's last
    // chunk polls for them, as the top-k rows do for their lists.
    // Two rounds: the workgroup agrees on the chunk's largest value first (a 32-bit reduction), then only the
    // lanes that hold it look for its place -- with scalar tests of whole-wave compare masks, since hardly any
    // lane does -- and the lowest id wins a second reduction.  (Every thread finding the place of its own
    // maximum, as a single reduction over (value, id) keys needs, costs each wave some 150 instructions.)
    const uint32_t cmax = block_max_lds<kSWaves, uint32_t>(lmax, sm.wave_val);
    const bool finisher = chunk == n_chunks - 1;
    if (sm.poisoned != 0u) return finisher;
    uint32_t widx = 0xffffffffu;  // lowest id of the wave's elements that equal the chunk's maximum
    if (cmax != 0u) {
      const float cf = key_to_float(cmax);
      if (__ballot(fm == cf) != 0ull) {
        const uint32_t wave_id0 = static_cast<uint32_t>(chunk) * kSChunk +
                                  static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(wave)) * 64u * VEC;
        u64 qe[kSVec];
#pragma unroll
        for (int j = 0; j < kSVec; ++j) {
          qe[j] = __ballot(qm[j] == cf);
          asm volatile("" : "+s"(qe[j]));
        }
#pragma unroll
        for (int j = 0; j < kSVec; ++j) {
          if (qe[j] != 0ull) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              const u64 m = __ballot(v[j * 4 + c] == cf);
              if (m != 0ull) {
                const uint32_t id = wave_id0 + static_cast<uint32_t>(elem_offset<kSBlock, VEC>(j * 4 + c)) +
                                    static_cast<uint32_t>(__builtin_ctzll(m)) * VEC;
                widx = id < widx ? id : widx;
              }
            }
          }
        }
        for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
          const uint32_t i = i0 + tid;
          const bool hit = i < n_extra && sm.extra_val[i] == cf;
          const uint32_t id = wave_max<uint32_t>(hit ? ~sm.extra_idx[i] : 0u);
          if (id != 0u && ~id < widx) widx = ~id;
        }
      }
    }
    if (lane == 0) sm.wave_val[wave] = ~widx;  // (the reduction above ended with a barrier: the slots are free)
    lds_barrier();
    if (wave != 0 && !finisher) return false;
    if (wave == 0) {
      const uint32_t best = row16_max<uint32_t>(lane < kSWaves ? sm.wave_val[lane] : 0u);  // ~id of the lowest id
      u64 key = best != 0u ? (static_cast<u64>(cmax) << 32) | best : 0;
      if (chunk == 0 && sm.nan0 != 0u) key = ~0ull;
      if (n_chunks == 1) {  // the row is this chunk: nothing to hand over
        const bool found = !extra_overflow && key != 0;
        if (lane == 0) {
          sm.flag = found ? 1u : 0u;
          if (found) outputs.token[0] = static_cast<int32_t>(key64_index(key));
        }
      } else {
      const size_t ci = static_cast<size_t>(row) * n_chunks + chunk;
      const u64 slot = extra_overflow ? kSlotOverflow : (key != 0 ? key : kSlotEmpty);
      if (!finisher) {
        if (lane == 0) store_coherent(&cand_small[ci * kSmallCap], slot);
        return false;
      }
      u64* seg = cand_small + static_cast<size_t>(row) * n_chunks * kSmallCap;
      u64 got = lane < n_chunks - 1 ? 0 : (lane == n_chunks - 1 ? slot : kSlotEmpty);
      int spins = 0;
      while (true) {
        if (got == 0) got = load_coherent(&seg[lane * kSmallCap]);
        if (__ballot(got == 0) == 0ull) break;
        if (spins++ >= poll_limit) {
          if (lane == 0) atomicOr(a.fallback_rows + 1, 1u);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (lane < n_chunks - 1 && got != 0) store_coherent(&seg[lane * kSmallCap], 0);  // for the next launch
      const bool bad = __ballot(got == 0 || got == kSlotOverflow) != 0ull;
      const u64 best = wave_max(got <= kSlotOverflow ? 0 : got);
      const bool found = !bad && best != 0;  // otherwise the exact path decides (an overflowing history, a wait that gave up)
      if (lane == 0) {
        sm.flag = found ? 1u : 0u;
        if (found) outputs.token[0] = static_cast<int32_t>(key64_index(best));
      }
      }
    }
    __syncthreads();
    return sm.flag == 0u;
  }
  // ---- top-k, k <= 64 ---------------------------------------------------------------------------
  const int kk = prm.k < V ? prm.k : V;
  int n_valid = V - chunk * kSChunk;
  if (n_valid > kSChunk) n_valid = kSChunk;
  int n_lanes = n_valid >= VEC * kSBlock ? kSBlock : (n_valid + VEC - 1) / VEC;  // threads that hold elements
  if (static_cast<uint32_t>(n_lanes) < n_extra) n_lanes = n_extra < static_cast<uint32_t>(kSBlock) ? static_cast<int>(n_extra) : kSBlock;
  const size_t ci = static_cast<size_t>(row) * n_chunks + chunk;
  u64* dst = cand_small + ci * kSmallCap;
  if (tid == 64) {  // ordered before the ranking route's atomics by the barrier of the bound
    sm.n_hits = 0u;
    sm.rank_failed = 0u;
  }
  uint32_t tau = block_pool_bound(lmax, kk, (n_lanes + 63) / 64, sm.pool);
  if (sm.poisoned != 0u) return chunk == n_chunks - 1;
  // The pooled bound is exact unless one wave holds more than its share of the best k; with k close to
  // 64 it can sit low enough for the hits to overflow their lists, and in a short tail chunk it may
  // find fewer than k offers (0).  Either way the exact k-th best of the per-thread maxima takes its
  // place: about k + k*k/1024 elements reach that one.
  static_assert(kSWaves * kWaveListCap >= kSBlock, "the hit lists double as the sort buffer of the exact bound");
  uint32_t n_c = 0u, cnt[kSWaves];
  bool overflow = false;
  // exact k-th best of the per-thread maxima
  auto exact_bound = [&]() {
    u64* scratch = sm.wave_list;  // free until the hits are listed
    scratch[tid] = static_cast<u64>(lmax);
    __syncthreads();
    block_sort_desc(scratch, kSBlock);
    const uint32_t t = static_cast<uint32_t>(scratch[kk - 1]);
    __syncthreads();
    return t;
  };
  // Hits are rare (about k per chunk).  Every wave lists its own hits in a private LDS segment: the
  // slot of a hit is the wave's running count (a scalar) plus the number of hitting lanes below, so
  // no atomics, no second pass and no block-wide prefix are needed.  Ends with the per-wave counts.
  auto list_hits = [&](uint32_t bound) {
    // bound == 0: the chunk has fewer than k elements -- keep them all
    const float tau_f = bound != 0u ? key_to_float(bound) : -__builtin_inff();
    uint32_t woff = 0u;
#pragma unroll
    for (int j = 0; j < kSVec; ++j) {
      if (__ballot(qm[j] >= tau_f) != 0ull) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const bool hit = v[j * 4 + c] >= tau_f;
          const u64 b = __ballot(hit);
          if (b == 0ull) continue;
          if (hit) {
            const uint32_t pos = woff + __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(b >> 32),
                                                                  __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(b), 0u));
            // key64 of a real element is never 0 (its index half is ~idx != 0), so 0 marks an empty slot
            // listed with the raw float bits; the few entries that survive get their order keys later
            if (pos < kWaveListCap)
              sm.wave_list[wave * kWaveListCap + pos] =
                  make_key64(__float_as_uint(v[j * 4 + c]), static_cast<uint32_t>(elem_index<kSBlock, VEC>(chunk, j, c)));
          }
          woff += static_cast<uint32_t>(__popcll(b));
        }
      }
    }
    for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
      const uint32_t i = i0 + tid;
      const float ev = i < n_extra ? sm.extra_val[i] : kNaN;
      const bool hit = ev >= tau_f;
      const u64 b = __ballot(hit);
      if (hit) {
        const uint32_t pos = woff + __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(b >> 32),
                                                              __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(b), 0u));
        if (pos < kWaveListCap) sm.wave_list[wave * kWaveListCap + pos] = make_key64(__float_as_uint(ev), sm.extra_idx[i]);
      }
      woff += static_cast<uint32_t>(__popcll(b));
    }
    if (lane == 0) sm.wave_val[wave] = woff;
    __syncthreads();
    n_c = 0u;
    overflow = false;
#pragma unroll
    for (int w = 0; w < kSWaves; ++w) {
      cnt[w] = sm.wave_val[w];
      n_c += cnt[w];
      overflow = overflow || cnt[w] > static_cast<uint32_t>(kWaveListCap);
    }
    overflow = overflow || n_c > static_cast<uint32_t>(kListCap);
  };
  const bool pooled = tau != 0u;
  const bool finisher = chunk == n_chunks - 1;
  // ---- the ranking route ------------------------------------------------------------------------------
  // A hit's place in the chunk's sorted list is the number of hits with a larger key, and with about sixty hits
  // that is cheaper to count than to sort for.  Each wave walks its hits with scalar code (the lane's value is
  // read into a scalar register, value and id are collected in lanes), reserves room in the chunk's list with
  // one LDS atomic and appends its keys.  After a barrier every wave holds the whole list, a key per lane, and
  // ranks an eighth of it: one 64-bit compare over the wave and a population count per hit -- exact whatever the
  // ties, because the keys are distinct.  After a second barrier wave 0 publishes the ranked list.  More than 64
  // hits in a wave or more than kListCap in the chunk: the listing and sorting route below does the chunk instead.
  bool placed = false;
  if (__builtin_expect(pooled && emit_topk != kEmitArgmax && !extra_overflow, 1)) {
    const float tau_f = key_to_float(tau);
    u64 qb[kSVec];
#pragma unroll
    for (int j = 0; j < kSVec; ++j) {
      qb[j] = __ballot(qm[j] >= tau_f);
      asm volatile("" : "+s"(qb[j]));  // all compares are issued before the first mask is looked at
    }
    uint32_t hx = 0u, hid = 0u;  // lane h: value bits and id of the wave's h-th hit
    int n = 0;
    // The hits of one register, whose lanes hold consecutive runs of ids (lane 0: id_lane0), or of one round over
    // the history ids' list (LISTED: the ids come in `ids`).  Per hit: its lane, the lane's value into a scalar
    // register, value and id into lane n of hx / hid (a lane number beyond 63 wraps; n > 64 is noticed below).
    auto take = [&](u64 b, float val, uint32_t id_lane0, auto listed, uint32_t ids) {
      while (b != 0ull) {
        int l;
        uint32_t xb, id;
        if constexpr (decltype(listed)::value) {
          asm volatile(
              "s_ff1_i32_b64 %[l], %[b]\n\t"
              "s_bitset0_b64 %[b], %[l]\n\t"
              "v_readlane_b32 %[x], %[val], %[l]\n\t"
              "v_readlane_b32 %[id], %[ids], %[l]\n\t"
              "s_mov_b32 m0, %[n]\n\t"
              "s_add_i32 %[n], %[n], 1\n\t"
              "v_writelane_b32 %[hx], %[x], m0\n\t"
              "v_writelane_b32 %[hid], %[id], m0"
              : [b] "+s"(b), [n] "+s"(n), [hx] "+v"(hx), [hid] "+v"(hid), [l] "=&s"(l), [x] "=&s"(xb), [id] "=&s"(id)
              : [val] "v"(val), [ids] "v"(ids)
              : "m0", "scc");
        } else if constexpr (VEC == 4) {
          asm volatile(
              "s_ff1_i32_b64 %[l], %[b]\n\t"
              "s_bitset0_b64 %[b], %[l]\n\t"
              "v_readlane_b32 %[x], %[val], %[l]\n\t"
              "s_lshl2_add_u32 %[id], %[l], %[id0]\n\t"
              "s_mov_b32 m0, %[n]\n\t"
              "s_add_i32 %[n], %[n], 1\n\t"
              "v_writelane_b32 %[hx], %[x], m0\n\t"
              "v_writelane_b32 %[hid], %[id], m0"
              : [b] "+s"(b), [n] "+s"(n), [hx] "+v"(hx), [hid] "+v"(hid), [l] "=&s"(l), [x] "=&s"(xb), [id] "=&s"(id)
              : [val] "v"(val), [id0] "s"(id_lane0)
              : "m0", "scc");
        } else {
          asm volatile(
              "s_ff1_i32_b64 %[l], %[b]\n\t"
              "s_bitset0_b64 %[b], %[l]\n\t"
              "v_readlane_b32 %[x], %[val], %[l]\n\t"
              "s_lshl3_add_u32 %[id], %[l], %[id0]\n\t"
              "s_mov_b32 m0, %[n]\n\t"
              "s_add_i32 %[n], %[n], 1\n\t"
              "v_writelane_b32 %[hx], %[x], m0\n\t"
              "v_writelane_b32 %[hid], %[id], m0"
              : [b] "+s"(b), [n] "+s"(n), [hx] "+v"(hx), [hid] "+v"(hid), [l] "=&s"(l), [x] "=&s"(xb), [id] "=&s"(id)
              : [val] "v"(val), [id0] "s"(id_lane0)
              : "m0", "scc");
        }
      }
    };
    static_assert(VEC == 4 || VEC == 8, "a lane's run of ids is a shift of its number");
    const uint32_t wave_id0 = static_cast<uint32_t>(chunk) * kSChunk +
                              static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(wave)) * 64u * VEC;
#pragma unroll
    for (int j = 0; j < kSVec; ++j) {
      if (qb[j] != 0ull) {
        u64 eb[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) eb[c] = __ballot(v[j * 4 + c] >= tau_f);
#pragma unroll
        for (int c = 0; c < 4; ++c)
          take(eb[c], v[j * 4 + c], wave_id0 + static_cast<uint32_t>(elem_offset<kSBlock, VEC>(j * 4 + c)), std::false_type{}, 0u);
      }
    }
    for (uint32_t i0 = 0; i0 < n_extra; i0 += kSBlock) {
      const uint32_t i = i0 + tid;
      const float ev = i < n_extra ? sm.extra_val[i] : kNaN;
      const uint32_t ei = i < n_extra ? sm.extra_idx[i] : 0u;
      take(__ballot(ev >= tau_f), ev, 0u, std::true_type{}, ei);
    }
    u64* const hits = sm.wave_list;  // the chunk's hits as keys, in no order
    uint32_t base = 0u;
    if (lane == 0) base = atomicAdd(&sm.n_hits, static_cast<uint32_t>(n));
    base = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(base)));
    if (n > 64 || base + static_cast<uint32_t>(n) > static_cast<uint32_t>(kListCap)) {
      if (lane == 0) sm.rank_failed = 1u;
    } else if (lane < n) {
      hits[base + lane] = make_key64(order_key(__uint_as_float(hx)), hid);
    }
    __syncthreads();
    const uint32_t total = sm.n_hits;
    placed = sm.rank_failed == 0u;
    if (placed) {
      // lane l holds hit l (and hit 64 + l of a long list); wave w ranks hits 8w .. 8w+7 (16w .. 16w+15), lane i the i-th
      const bool wide = total > 64u;
      const int per = wide ? 16 : 8;
      const uint32_t first = static_cast<uint32_t>(wave * per);
      const u64 mine0 = static_cast<uint32_t>(lane) < total ? hits[lane] : 0;
      const u64 mykey = (lane < per && first + lane < total) ? hits[first + lane] : 0;
      uint32_t myrank = 0u;
      if (!wide) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const u64 key = read_lane(mine0, wave * 8 + i);
          const int r = __popcll(__ballot(mine0 > key));
          asm volatile("v_writelane_b32 %0, %1, %2" : "+v"(myrank) : "s"(r), "n"(i));
        }
      } else {
        const u64 mine1 = static_cast<uint32_t>(lane) + 64u < total ? hits[lane + 64] : 0;
        const u64 src = wave < 4 ? mine0 : mine1;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const u64 key = read_lane(src, (wave * 16 + i) & 63);
          const int r = __popcll(__ballot(mine0 > key)) + __popcll(__ballot(mine1 > key));
          asm volatile("v_writelane_b32 %0, %1, %2" : "+v"(myrank) : "s"(r), "n"(i));
        }
      }
      if (mykey != 0 && myrank < static_cast<uint32_t>(kSmallCap)) sm.own[myrank] = mykey;
      __syncthreads();
      if (wave == 0) {
        const u64 slot = static_cast<uint32_t>(lane) < total ? sm.own[lane] : kSlotEmpty;
        if (finisher) sm.own[lane] = slot;
        else store_coherent(&dst[lane], slot);
      }
      if (!finisher) return false;
    }
  }
  if (!placed) {
  if (__builtin_expect(!pooled, 0)) tau = exact_bound();
  list_hits(tau);
  if (__builtin_expect(overflow && pooled, 0)) {  // rare: a second, separate copy of the listing code, with the exact bound
    tau = exact_bound();
    list_hits(tau);
  }
  overflow = overflow || extra_overflow;
  // The chunk's best 64 candidates, sorted (best first): nothing ranked lower inside its own chunk can
  // be among the row's k <= 64 best.  Waves 0 and 1 sort one half of the list each, wave 0 merges.
  // The workgroup of the row's LAST chunk finishes the row; every other workgroup publishes its list
  // and is done.  A published slot is never 0: kSlotEmpty pads a short list, kSlotOverflow replaces a
  // list that did not fit.  The finishing workgroup polls the slots until all of them are non-zero and
  // clears them again for the next launch; no counter, no wait for the stores and no second round
  // trip lie between a chunk's sort and the row's merge.  Workgroups are dispatched in index order
  // and a publishing workgroup never waits, so the lists a finishing workgroup polls for belong to
  // workgroups that are running or done.
  const bool two_halves = n_c > 64u;
  u64 mykey = 0;
  if (wave < 2 && !overflow) {
    // entry p of the concatenated wave lists: list w covers [start_w, start_w + count_w)
    const uint32_t p = static_cast<uint32_t>(wave) * 64u + static_cast<uint32_t>(lane);
    if (p < n_c) {
      uint32_t start = 0u, w = 0u, off = 0u;
#pragma unroll
      for (int i = 0; i < kSWaves - 1; ++i) {
        start += cnt[i];
        if (p >= start) {
          w = static_cast<uint32_t>(i) + 1u;
          off = start;
        }
      }
      const u64 raw = sm.wave_list[w * kWaveListCap + (p - off)];
      mykey = (static_cast<u64>(order_key(__uint_as_float(static_cast<uint32_t>(raw >> 32)))) << 32) |
              (raw & 0xffffffffull);
    }
    if (wave == 0 || two_halves) mykey = wave_sort_desc_fast<u64>(mykey);
    if (wave == 1 && two_halves) sm.list_hi[63 - lane] = mykey;
  }
  if (two_halves && !overflow) __syncthreads();
  if (wave == 0) {
    if (!overflow && two_halves) {
      const u64 other = sm.list_hi[lane];  // ascending against descending: a bitonic pair
      mykey = other > mykey ? other : mykey;
      sort_merge<64, 32, u64>(mykey, lane);
    }
    // ArgMax starts from id 0 and nothing compares above a NaN (src/search.h:9-29): such a row's answer is 0
    if (emit_topk == kEmitArgmax && chunk == 0 && lane == 0 && sm.nan0 != 0u) mykey = ~0ull;
    const u64 slot = overflow ? kSlotOverflow : (mykey != 0 ? mykey : kSlotEmpty);
    if (finisher) sm.own[lane] = slot;
    else store_coherent(&dst[lane], slot);
  }
  }  // !placed
  if (!finisher) return false;

  // ---- the row's finishing workgroup ---------------------------------------------------------------
  LaneExp2Tab tab;
  {
    const uint64_t t = g_exp2_tab[lane & 31];  // issued now, consumed by the epilogue
    tab.lo = static_cast<uint32_t>(t);
    tab.hi = static_cast<uint32_t>(t >> 32);
  }
  const double u = emit_topk ? 0.0 : uniforms[row];
  const float inv_temp = 1.0f / prm.temperature;
  // sm.own is written by wave 0; with at most four chunks wave 0 alone reads it (a wave's LDS accesses execute in order)
  if (n_chunks > 4) __syncthreads();
  u64* seg = cand_small + static_cast<size_t>(row) * n_chunks * kSmallCap;
  // Wave w merges the sorted lists of chunks 4w .. 4w+3 in registers, straight from global memory;
  // rows of more than four chunks need a second level through LDS.  Wave 0 ends with the row's 64
  // best, checks that there are k of them, and runs the epilogue while the other waves wait at the
  // barrier that tells the workgroup whether the exact path is needed after all.
  const int chunks = n_chunks;
  const int groups = (chunks + 3) >> 2;
  u64 final_key = 0;
  bool bad = false;  // a list is missing (overflow, or the wait below gave up)
  if (wave < groups) {
    const int c0 = wave * 4;
    // lane's four slots, in the orientation wave_merge4 wants them
    const int cc[4] = {c0, c0 + 1, c0 + 2, c0 + 3};
    const int ii[4] = {lane, 63 - lane, 63 - lane, lane};
    u64 got[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (cc[q] >= chunks) got[q] = kSlotEmpty;
      else if (cc[q] == chunks - 1) got[q] = sm.own[ii[q]];
      else got[q] = 0;
    }
    int spins = 0;
    while (true) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (got[q] == 0) got[q] = load_coherent(&seg[cc[q] * kSmallCap + ii[q]]);
      if (__ballot(got[0] == 0 || got[1] == 0 || got[2] == 0 || got[3] == 0) == 0ull) break;
      if (spins++ >= poll_limit) {
        if (lane == 0) atomicOr(a.fallback_rows + 1, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (cc[q] < chunks - 1 && got[q] != 0) store_coherent(&seg[cc[q] * kSmallCap + ii[q]], 0);  // for the next launch
      bad = bad || got[q] == 0 || got[q] == kSlotOverflow;
      if (got[q] <= kSlotOverflow) got[q] = 0;
    }
    bad = __ballot(bad) != 0ull;
    const u64* g4 = got;
    final_key = wave_merge4([&](int c, int) -> u64 { return g4[c]; }, lane);
    if (groups > 1) sm.lists[wave * kSmallCap + lane] = final_key;
    if (bad && lane == 0) sm.count = 1u;  // zeroed by thread 0 before the barriers of the bound
  }
  if (groups > 1) {
    __syncthreads();
    if (wave == 0) {
      const u64* l = sm.lists;
      final_key = wave_merge4([&](int c, int i) -> u64 { return c < groups ? l[c * kSmallCap + i] : 0; }, lane);
      bad = sm.count != 0u;
    }
  }
  if (wave == 0) {
    const u64 kth = read_lane(final_key, kk - 1);
    const bool enough = !bad && kth != 0;  // otherwise NaNs are needed to fill k: the exact path decides
    if (lane == 0) sm.flag = enough ? 1u : 0u;
    if (enough) {
      if (lane >= kk) final_key = 0;
      if (emit_topk) {
        if (lane < kk) {
          const uint32_t id = key64_index(final_key);
          a.out_tokens[static_cast<size_t>(row) * prm.k + lane] = static_cast<int32_t>(id);
          if (emit_topk == 1)
            a.out_scores[static_cast<size_t>(row) * prm.k + lane] = RowPtr<InT>(row0, 0)[id];  // keys do not tell -0 from +0
        }
      } else {
        {
          RowOutputs out = outputs;  // pointers to this row's slots
          const bool token_only = !out.kept_count && !out.kept_ids && !out.kept_probs;
          if (!(token_only && wave_topk_token_fast(final_key, kk, prm, inv_temp, u, tab, out.token))) {
            out.kept_count = out.kept_count ? out.kept_count + row : nullptr;
            out.kept_ids = out.kept_ids ? out.kept_ids + static_cast<size_t>(row) * out.kept_capacity : nullptr;
            out.kept_probs = out.kept_probs ? out.kept_probs + static_cast<size_t>(row) * out.kept_capacity : nullptr;
            wave_topk_epilogue(final_key, kk, prm, u, tab, out);
          }
        }
      }
    }
  }
  __syncthreads();
  return sm.flag == 0u;
}

// Rows in nucleus mode and all other rows are streamed by kernels of their own (a launch may need
// both): each kernel holds the code of its mode only, and a change to one path leaves the machine
// code of the other as it was.
// The arguments a streaming kernel reads before it requests its logits, fetched together.  Kernel arguments come by
// scalar loads that return out of order, so every wait for one of them waits for all that are under way, and a
// value first needed behind a branch is requested behind that branch: left alone, five such round trips (per-row
// table? shape, mode, row pointer, flag word) stood in front of the first logits request of every wave.
// Returns the uniform (k, p, T) as values that exist before the first branch.
template <bool XFORM>
__device__ __forceinline__ mi355x_sample_params args_up_front(const SampleArgs& a) {
  if constexpr (XFORM) {  // what the logits processing reads before the logits are requested, in the same round trip
    const uint32_t* mask = a.xf.mask;
    const int32_t* history = a.xf.history;
    const int32_t* history_lens = a.xf.history_lens;
    const uint32_t* ban = a.xf.ban;
    int history_stride = a.xf.history_stride, history_len = a.xf.history_len, n_eos = a.xf.n_eos;
    float penalty = a.xf.penalty;
    asm volatile("" : "+s"(mask), "+s"(history), "+s"(history_lens), "+s"(ban), "+s"(history_stride), "+s"(history_len),
                 "+s"(n_eos), "+s"(penalty));
  }
  const void* logits = a.logits;
  int64_t row_stride = a.row_stride;
  int vocab = a.vocab, chunks = a.chunks, k = a.uniform.k, emit_topk = a.emit_topk, exact_kernel = a.exact_kernel;
  float p = a.uniform.p, temperature = a.uniform.temperature;
  const mi355x_sample_params* per_row = a.per_row;
  uint32_t* fallback_rows = a.fallback_rows;
  uint32_t* row_done = a.row_done;
  asm volatile(""
               : "+s"(logits), "+s"(row_stride), "+s"(vocab), "+s"(chunks), "+s"(k), "+s"(p), "+s"(temperature), "+s"(per_row),
                 "+s"(emit_topk), "+s"(exact_kernel), "+s"(fallback_rows), "+s"(row_done));
  mi355x_sample_params q;
  q.k = k;
  q.p = p;
  q.temperature = temperature;
  return q;
}

template <typename InT, bool INLINE, bool NUCLEUS, bool XFORM, bool LARGEK = false, bool ARGMAX = false>
__device__ __forceinline__ void sample_fused_body(const SampleArgs& a) {
  const mi355x_sample_params uniform_prm = args_up_front<XFORM>(a);
  const int row = blockIdx.y, chunk = blockIdx.x;
  __shared__ FusedShared sm;
  const mi355x_sample_params prm = row_params<INLINE>(a, row, uniform_prm);
  const void* const row0 = row_start<INLINE>(a, row, sizeof(InT));
  const int mode = row_mode(prm, a.vocab, a.chunks, a.emit_topk);
  if constexpr (NUCLEUS) {
    if (mode == (LARGEK ? kModeTopkLarge : kModeNucleus)) {
      if constexpr (XFORM && !LARGEK) {
        if (a.xf.mask && a.row_done && a.row_done[row] != 0u) return;  // finished by the sparse-mask kernel
      }
      stream_row<InT, true, XFORM, LARGEK>(a, row, row0, chunk, prm, sm);
    }
  } else {
    if (mode == kModeNucleus || mode == kModeTopkLarge) return;
    if (mode == kModeGeneral) {
      if (chunk != 0 || a.exact_kernel) return;  // exact_kernel: the exact-rows kernel sorts such rows much faster
    } else if (!stream_row<InT, false, XFORM, false, ARGMAX>(a, row, row0, chunk, prm, sm)) {
      return;
    }
    // Rows the fast paths decline end here, in the exact general path (a single inlined call site keeps
    // the argument block in scalar registers instead of a scratch copy).
    __syncthreads();
    static_assert(sizeof(sm.wave_list) >= kSelectCap * sizeof(u64) && sizeof(sm.lists) >= kTopkBlock * sizeof(uint32_t) &&
                      sizeof(sm.pool) >= (4 + kTopkBlock / 64) * sizeof(uint32_t), "the selection's LDS");
    const TopkSelectLds select{sm.wave_list, reinterpret_cast<uint32_t*>(sm.lists), sm.pool};
    general_row<InT>(a, row, row0, prm, a.big + static_cast<size_t>(row) * a.big_stride, sm.seq, SortInGlobalMemory{}, &select);
  }
}

// Kernel variants: per-row parameter table in the arguments or not (_rows); nucleus rows, top-k rows with
// 64 < k <= kLargeKMax (largek) or all other rows; with or without the code of the logits processing (_xf);
// one set per element type of the logits (SUFFIX: none for fp32, _f16, _bf16), each in a source file of its own.
#define MS_STREAM_KERNEL(NAME, SUFFIX, InT, NUCLEUS, XFORM, LARGEK)                                                      \
  __global__ __launch_bounds__(NUCLEUS ? kNucleusBlock : kTopkBlock) void NAME##SUFFIX##_kernel(const SampleArgs a) {   \
    sample_fused_body<InT, false, NUCLEUS, XFORM, LARGEK>(a);                                                            \
  }                                                                                                                      \
  __global__ __launch_bounds__(NUCLEUS ? kNucleusBlock : kTopkBlock) void NAME##SUFFIX##_rows_kernel(                    \
      const SampleArgs a, const InlineParams) {                                                                          \
    sample_fused_body<InT, true, NUCLEUS, XFORM, LARGEK>(a);                                                             \
  }

// Defines the streaming kernels of one element type (twelve for sampling, two for argmax) and
// ms_launch_stream##SUFFIX, which launches the one a call needs: which = 0 rows of every other mode (argmax
// calls: the argmax kernels), 1 nucleus rows, 2 rows with 64 < k <= kLargeKMax.
#define MS_STREAM_KERNELS(SUFFIX, InT)                                                                                   \
  namespace ms {                                                                                                         \
  MS_STREAM_KERNEL(sample_fused, SUFFIX, InT, false, false, false)                                                       \
  MS_STREAM_KERNEL(sample_fused_xf, SUFFIX, InT, false, true, false)                                                     \
  MS_STREAM_KERNEL(nucleus_stream, SUFFIX, InT, true, false, false)                                                      \
  MS_STREAM_KERNEL(nucleus_stream_xf, SUFFIX, InT, true, true, false)                                                    \
  MS_STREAM_KERNEL(largek_stream, SUFFIX, InT, true, false, true)                                                        \
  MS_STREAM_KERNEL(largek_stream_xf, SUFFIX, InT, true, true, true)                                                      \
  __global__ __launch_bounds__(kTopkBlock) void argmax_stream##SUFFIX##_kernel(const SampleArgs a) {                     \
    sample_fused_body<InT, false, false, false, false, true>(a);                                                         \
  }                                                                                                                      \
  __global__ __launch_bounds__(kTopkBlock) void argmax_stream_xf##SUFFIX##_kernel(const SampleArgs a) {                  \
    sample_fused_body<InT, false, false, true, false, true>(a);                                                          \
  }                                                                                                                      \
  }                                                                                                                      \
  extern "C" hipError_t ms_launch_stream##SUFFIX(const ms::SampleArgs* a, const ms::InlineParams* table, int which,      \
                                                 hipStream_t stream) {                                                   \
    const dim3 grid(a->chunks, a->rows), block(which == 0 ? ms::kTopkBlock : ms::kNucleusBlock);                         \
    const bool xf = a->xf.active();                                                                                      \
    if (which == 0 && a->emit_topk == ms::kEmitArgmax && !table) {                                                       \
      hipLaunchKernelGGL(xf ? ms::argmax_stream_xf##SUFFIX##_kernel : ms::argmax_stream##SUFFIX##_kernel, grid, block, 0, \
                         stream, *a);                                                                                    \
    } else if (table) {                                                                                                         \
      auto* f = which == 0   ? (xf ? ms::sample_fused_xf##SUFFIX##_rows_kernel : ms::sample_fused##SUFFIX##_rows_kernel) \
                : which == 1 ? (xf ? ms::nucleus_stream_xf##SUFFIX##_rows_kernel : ms::nucleus_stream##SUFFIX##_rows_kernel) \
                             : (xf ? ms::largek_stream_xf##SUFFIX##_rows_kernel : ms::largek_stream##SUFFIX##_rows_kernel); \
      hipLaunchKernelGGL(f, grid, block, 0, stream, *a, *table);                                                         \
    } else {                                                                                                             \
      auto* f = which == 0   ? (xf ? ms::sample_fused_xf##SUFFIX##_kernel : ms::sample_fused##SUFFIX##_kernel)           \
                : which == 1 ? (xf ? ms::nucleus_stream_xf##SUFFIX##_kernel : ms::nucleus_stream##SUFFIX##_kernel)       \
                             : (xf ? ms::largek_stream_xf##SUFFIX##_kernel : ms::largek_stream##SUFFIX##_kernel);        \
      hipLaunchKernelGGL(f, grid, block, 0, stream, *a);                                                                 \
    }                                                                                                                    \
    return hipGetLastError();                                                                                            \
  }

}  // namespace ms
