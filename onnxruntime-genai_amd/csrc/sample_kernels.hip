// Sampling kernels: one streaming pass over the logits (fused logits processing + candidate
// selection), finished per row by the last workgroup to arrive (top-k <= 64) or by a second per-row
// kernel (nucleus), with an exact general path for everything the fast paths decline.
#include "kernels.h"
#include "block_seq.h"

namespace ms {

// ------------------------------------------------------------------------------------------------
// Serial prefix over lanes: out[l] = ((x[0] + x[1]) + ...) + x[l], additions in lane order, as the
// reference's scalar loops do.  One DPP-shifted add per element.
__device__ __forceinline__ float wave_serial_prefix(float x, int count) {
  float s = 0.0f;
  for (int t = 0; t < count; ++t) {
    // wave_shr:1 -- lane l reads lane l-1; lane 0 keeps `old` (0.0f).
    const float prev = __uint_as_float(
        __builtin_amdgcn_update_dpp(0u, __float_as_uint(s), 0x138, 0xf, 0xf, false));
    s = prev + x;
  }
  return s;
}

__device__ __forceinline__ double wave_serial_prefix(double x, int count) {
  double s = 0.0;
  for (int t = 0; t < count; ++t) {
    const u64 b = static_cast<u64>(__double_as_longlong(s));
    const uint32_t lo = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b), 0x138, 0xf, 0xf, false);
    const uint32_t hi = __builtin_amdgcn_update_dpp(0u, static_cast<uint32_t>(b >> 32), 0x138, 0xf, 0xf, false);
    const double prev = __longlong_as_double(static_cast<long long>((static_cast<u64>(hi) << 32) | lo));
    s = prev + x;
  }
  return s;
}

// Slot allocation from a shared counter with one atomic per wave.  Must be reached by every lane of
// the wave; lanes with pred == false get an unspecified value.
__device__ __forceinline__ uint32_t wave_slot(bool pred, uint32_t* counter) {
  const u64 b = __ballot(pred);
  if (b == 0) return 0u;
  const int lane = lane_id();
  const int leader = __ffsll(static_cast<long long>(b)) - 1;
  uint32_t base = 0u;
  if (lane == leader) base = atomicAdd(counter, static_cast<uint32_t>(__popcll(b)));
  base = __shfl(base, leader, 64);
  return base + static_cast<uint32_t>(__popcll(b & ((1ull << lane) - 1ull)));
}

__device__ __forceinline__ int first_lane(u64 ballot) { return ballot ? __ffsll(static_cast<long long>(ballot)) - 1 : -1; }

// Epilogue for k <= 64 run by one wave: lane j holds the j-th best (key64), j < m.
// Follows ComputeSampledCategorical's top-k branch (src/sampling_distribution.h:243-281) and
// std::discrete_distribution literally: every sum is accumulated in rank order.
__device__ __forceinline__ void wave_topk_epilogue(u64 key, int m, mi355x_sample_params prm, double u, const RowOutputs& out) {
  const int lane = lane_id();
  const float score = key_to_float(key64_okey(key));
  const float max_score = shfl_t<float>(score, 0);
  const float inv_temp = 1.0f / prm.temperature;
  const float e = lane < m ? em::expf_exact((score - max_score) * inv_temp) : 0.0f;
  const float sum = shfl_t<float>(wave_serial_prefix(e, m), m - 1);
  const float pr = sum > 0.0f ? e / sum : e;
  const float cum = wave_serial_prefix(pr, m);
  int keep = m;
  if (prm.p > 0.0f && prm.p < 1.0f) {
    const int f = first_lane(__ballot(lane < m && cum >= prm.p));
    if (f >= 0) keep = f + 1;
  }
  const float keep_sum = shfl_t<float>(cum, keep - 1);
  const float inv = keep_sum > 0.0f ? 1.0f / keep_sum : 0.0f;
  const float q = pr * inv;
  int pos = 0;
  if (keep >= 2) {
    const double qd = lane < keep ? static_cast<double>(q) : 0.0;
    const double dsum = shfl_t<double>(wave_serial_prefix(qd, keep), keep - 1);
    const double pn = qd / dsum;
    double cp = wave_serial_prefix(pn, keep);
    if (lane == keep - 1) cp = 1.0;
    pos = first_lane(__ballot(lane < keep && cp >= u));
    if (pos < 0) pos = keep - 1;
  }
  const uint32_t idx = key64_index(key);
  const int32_t tok = static_cast<int32_t>(shfl_t<uint32_t>(idx, pos));
  if (lane == 0) {
    *out.token = tok;
    if (out.kept_count) *out.kept_count = keep;
  }
  if (out.kept_ids && lane < keep && lane < out.kept_capacity) {
    out.kept_ids[lane] = static_cast<int32_t>(idx);
    if (out.kept_probs) out.kept_probs[lane] = q;
  }
}

__device__ __forceinline__ int next_pow2(int v) {
  int p = 64;
  while (p < v) p <<= 1;
  return p;
}

// Exact general path for one row, any (k, p, T), any vocabulary size: rebuilds the processed row as
// key64s in global scratch, sorts all of it, then runs the reference algorithm on the sorted row.
// Run by one whole block.  scratch holds next_pow2(vocab) entries.
__device__ __forceinline__ void general_row(const SampleArgs& a, int row, u64* scratch, SeqShared& sh) {
  const int V = a.vocab;
  const float* lrow = a.logits + static_cast<size_t>(row) * a.row_stride;
  const int n2 = next_pow2(V);
  const bool has_mask = a.xf.mask != nullptr;
  const uint32_t* mrow = has_mask ? a.xf.mask + static_cast<size_t>(row) * ((V - 1) / 32 + 1) : nullptr;
  for (int i = threadIdx.x; i < n2; i += blockDim.x) {
    u64 k = 0;
    if (i < V) {
      const float x = xform_value(lrow[i], a.xf, i, has_mask ? mrow[i >> 5] : 0u, has_mask, false);
      k = make_key64(order_key(x), static_cast<uint32_t>(i));
    }
    scratch[i] = k;
  }
  __syncthreads();
  if (a.xf.use_penalty()) {
    const int32_t* h = a.xf.history + static_cast<size_t>(row) * a.xf.history_stride;
    for (int j = threadIdx.x; j < a.xf.history_len; j += blockDim.x) {
      const int tok = h[j];
      if (tok < 0 || tok >= V) continue;
      bool dup = false;
      for (int jj = 0; jj < j && !dup; ++jj) dup = (h[jj] == tok);
      if (dup) continue;
      const float x = xform_value(lrow[tok], a.xf, tok, has_mask ? mrow[tok >> 5] : 0u, has_mask, true);
      scratch[tok] = make_key64(order_key(x), static_cast<uint32_t>(tok));
    }
    __syncthreads();
  }
  block_sort_desc(scratch, n2);
  const mi355x_sample_params prm = a.per_row ? a.per_row[row] : a.uniform;
  const float max_score = key_to_float(key64_okey(scratch[0]));
  const float inv_temp = 1.0f / prm.temperature;
  RowOutputs out{a.out_tokens + row, a.kept_count ? a.kept_count + row : nullptr,
                 a.kept_ids ? a.kept_ids + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                 a.kept_probs ? a.kept_probs + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                 a.kept_capacity};
  const u64* sc = scratch;
  auto sorted = [=](int i) { return sc[i]; };
  auto exps = [=](int i) { return em::expf_exact((key_to_float(key64_okey(sc[i])) - max_score) * inv_temp); };
  block_sample_epilogue<4>(sorted, exps, V, V, prm, a.uniforms[row], out, sh);
  if (threadIdx.x == 0) atomicAdd(a.fallback_rows, 1u);
}

__device__ __forceinline__ int row_mode(mi355x_sample_params prm, int vocab) {
  if (vocab <= 64) return kModeGeneral;
  if (prm.k > 1) return (prm.k < vocab ? prm.k : vocab) <= 64 ? kModeTopkSmall : kModeGeneral;
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

// LDS of the streaming kernel.
struct StreamShared {
  uint32_t hist_bits[kChunk / 32];
  uint32_t pool[64];
  u64 stage[kSmallCap];
  u64 fin[kFinCap];
  uint32_t count, flag, count2;
  u64 red64[4];
  uint32_t red32[4];
  SeqShared seq;
};

// Streaming pass of one (row, chunk) of a top-k<=64 or nucleus row.  Returns true when this workgroup
// must run the general path for the row (it was the last to arrive and the candidate slots overflowed).
__device__ __forceinline__ bool stream_row(const SampleArgs& a, int row, int chunk, mi355x_sample_params prm,
                                           int mode, StreamShared& sm) {
  const int V = a.vocab;
  const int tid = threadIdx.x;
  u64* big_row = a.big + static_cast<size_t>(row) * a.big_stride;
  const float* lrow = a.logits + static_cast<size_t>(row) * a.row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(lrow) & 15u) == 0);
  float v[kElems];
  Loader<float>::load(lrow, aligned, V, chunk, v);
  if (a.xf.active()) {
    if (a.xf.use_penalty()) build_history_bitmap(a.xf, row, chunk * kChunk, sm.hist_bits);
    xform_chunk<float>(a.xf, row, V, chunk, sm.hist_bits, v);
  }
  uint32_t keys[kElems];
  uint32_t lmax = 0u;
#pragma unroll
  for (int e = 0; e < kElems; ++e) {
    const int idx = Loader<float>::index_of(chunk, e / 4, e % 4);
    keys[e] = idx < V ? order_key(v[e]) : 0u;
    lmax = keys[e] > lmax ? keys[e] : lmax;
  }
  if (tid == 0) sm.count = 0u;

  if (mode == kModeNucleus) {
    const uint32_t cmax = block_max<uint32_t>(lmax, sm.red32);  // barriers inside publish count = 0
    uint32_t thr = 0u;
    if (cmax != 0u) thr = order_key(key_to_float(cmax) - nucleus_depth(prm, V));
    u64 best_below = 0;
    u64* dst = big_row + static_cast<size_t>(chunk) * kChunk;
#pragma unroll
    for (int e = 0; e < kElems; ++e) {
      const int idx = Loader<float>::index_of(chunk, e / 4, e % 4);
      const u64 k64 = make_key64(keys[e], static_cast<uint32_t>(idx));
      const bool cand = idx < V && keys[e] >= thr && keys[e] != 0u;
      const uint32_t pos = wave_slot(cand, &sm.count);
      if (cand) dst[pos] = k64;
      else if (idx < V) best_below = k64 > best_below ? k64 : best_below;
    }
    best_below = block_max<u64>(best_below, sm.red64);
    if (tid == 0) {
      const size_t ci = static_cast<size_t>(row) * a.chunks + chunk;
      a.chunk_cnt[ci] = sm.count;
      a.chunk_max[ci] = cmax;
      a.chunk_next[ci] = best_below;
    }
    return false;
  }

  // ---- top-k, k <= 64 ----
  const int kk = prm.k < V ? prm.k : V;
  uint32_t tau = block_kth_bound(lmax, kk, sm.pool);
  if (tau == 0u) {
    // The pooled bound degenerated (a short tail chunk keeps its elements in one or two waves):
    // take the exact kk-th best of the 256 per-thread maxima instead.
    sm.fin[tid] = static_cast<u64>(lmax);
    __syncthreads();
    block_sort_desc(sm.fin, kBlock);
    tau = static_cast<uint32_t>(sm.fin[kk - 1]);
    __syncthreads();
  }
#pragma unroll
  for (int e = 0; e < kElems; ++e) {
    const int idx = Loader<float>::index_of(chunk, e / 4, e % 4);
    const bool cand = idx < V && keys[e] >= tau;
    const uint32_t pos = wave_slot(cand, &sm.count);
    if (cand && pos < kSmallCap) sm.stage[pos] = make_key64(keys[e], static_cast<uint32_t>(idx));
  }
  __syncthreads();
  const uint32_t n_c = sm.count;
  const size_t ci = static_cast<size_t>(row) * a.chunks + chunk;
  {
    u64* dst = a.cand_small + ci * kSmallCap;
    if (tid < kSmallCap && static_cast<uint32_t>(tid) < n_c) dst[tid] = sm.stage[tid];
    if (tid == 0) a.chunk_cnt[ci] = n_c;
  }
  __threadfence();
  __syncthreads();
  if (tid == 0) {
    const uint32_t old = atomicAdd(&a.row_arrive[row], 1u);
    sm.flag = (old == static_cast<uint32_t>(a.chunks) - 1u) ? 1u : 0u;
  }
  __syncthreads();
  if (!sm.flag) return false;
  __threadfence();

  // ---- last workgroup of the row: merge the chunks' candidates ----
  __syncthreads();
  if (tid == 0) {
    a.row_arrive[row] = 0u;  // ready for the next launch
    sm.count = 0u;
    sm.count2 = 0u;
    sm.flag = 0u;
  }
  __syncthreads();
  const int slots = a.chunks * kSmallCap;
  for (int p = tid; p < slots; p += kBlock) {
    const int ch = p / kSmallCap, sl = p % kSmallCap;
    const uint32_t cnt = load_coherent(&a.chunk_cnt[static_cast<size_t>(row) * a.chunks + ch]);
    if (cnt > kSmallCap) sm.flag = 1u;  // a chunk overflowed its slots
    if (static_cast<uint32_t>(sl) < cnt) {
      const u64 k64 = load_coherent(&a.cand_small[(static_cast<size_t>(row) * a.chunks + ch) * kSmallCap + sl]);
      const uint32_t pos = atomicAdd(&sm.count, 1u);
      if (pos < kFinCap) sm.fin[pos] = k64;
    }
  }
  __syncthreads();
  const uint32_t total = sm.count;
  if (sm.flag || total > kFinCap) return true;
  RowOutputs out{a.out_tokens + row, a.kept_count ? a.kept_count + row : nullptr,
                 a.kept_ids ? a.kept_ids + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                 a.kept_probs ? a.kept_probs + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                 a.kept_capacity};
  // second-level bound over the merged candidates
  uint32_t lm2 = 0u;
  for (uint32_t p = tid; p < total; p += kBlock) {
    const uint32_t ok = key64_okey(sm.fin[p]);
    lm2 = ok > lm2 ? ok : lm2;
  }
  const uint32_t tau2 = block_kth_bound(lm2, kk, sm.pool);
  u64* sel = sm.stage;  // reuse: up to 64 survivors
  for (uint32_t p = tid; p < total; p += kBlock) {
    const u64 k64 = sm.fin[p];
    if (key64_okey(k64) >= tau2) {
      const uint32_t pos = atomicAdd(&sm.count2, 1u);
      if (pos < 64u) sel[pos] = k64;
    }
  }
  __syncthreads();
  const uint32_t n_sel = sm.count2;
  if (n_sel > 64u) {
    // too many survivors (ties at the bound): sort all merged candidates in LDS instead
    const int n2 = next_pow2(static_cast<int>(total));
    for (int p = static_cast<int>(total) + tid; p < n2; p += kBlock) sm.fin[p] = 0;
    __syncthreads();
    block_sort_desc(sm.fin, n2);
    if (tid < 64) wave_topk_epilogue(tid < kk ? sm.fin[tid] : 0, kk, prm, a.uniforms[row], out);
    return false;
  }
  if (tid < 64) {
    u64 k64 = static_cast<uint32_t>(tid) < n_sel ? sel[tid] : 0;
    k64 = wave_sort_desc<u64>(k64);
    wave_topk_epilogue(k64, kk, prm, a.uniforms[row], out);
  }
  return false;
}

__global__ __launch_bounds__(kBlock) void sample_stream_kernel(const SampleArgs a) {
  const int row = blockIdx.y, chunk = blockIdx.x;
  __shared__ StreamShared sm;
  const mi355x_sample_params prm = a.per_row ? a.per_row[row] : a.uniform;
  const int mode = row_mode(prm, a.vocab);
  if (mode == kModeGeneral) {
    if (chunk != 0) return;
  } else if (!stream_row(a, row, chunk, prm, mode, sm)) {
    return;
  }
  // Rows the fast paths decline end here, in the exact general path (a single inlined call site keeps
  // the argument block in scalar registers instead of a scratch copy).
  __syncthreads();
  general_row(a, row, a.big + static_cast<size_t>(row) * a.big_stride, sm.seq);
}

// Per-row finish of the nucleus path: gathers the candidates the streaming pass left in `big`,
// sorts them in LDS and runs the exact epilogue.  One block of kFinishBlock threads per row;
// dynamic LDS: kNucleusCap key64s.
__global__ __launch_bounds__(kFinishBlock) void nucleus_finish_kernel(const SampleArgs a) {
  extern __shared__ u64 lds_keys[];
  __shared__ SeqShared seqsh;
  __shared__ uint32_t sh_count;
  __shared__ uint32_t red32[16];
  __shared__ u64 red64[16];
  const int row = blockIdx.x;
  const int V = a.vocab;
  const int tid = threadIdx.x;
  const mi355x_sample_params prm = a.per_row ? a.per_row[row] : a.uniform;
  if (row_mode(prm, V) != kModeNucleus) return;
  u64* big_row = a.big + static_cast<size_t>(row) * a.big_stride;
  const size_t cbase = static_cast<size_t>(row) * a.chunks;
  uint32_t m = 0u;
  for (int c = tid; c < a.chunks; c += blockDim.x) m = a.chunk_max[cbase + c] > m ? a.chunk_max[cbase + c] : m;
  if (tid == 0) sh_count = 0u;
  const uint32_t rmax = block_max<uint32_t>(m, red32);
  uint32_t thr = 0u;
  if (rmax != 0u) thr = order_key(key_to_float(rmax) - nucleus_depth(prm, V));
  u64 best_below = 0;
  for (int c = tid; c < a.chunks; c += blockDim.x) best_below = a.chunk_next[cbase + c] > best_below ? a.chunk_next[cbase + c] : best_below;
  for (int c = 0; c < a.chunks; ++c) {
    const uint32_t cnt = a.chunk_cnt[cbase + c];
    const u64* src = big_row + static_cast<size_t>(c) * kChunk;
    for (uint32_t i0 = 0; i0 < cnt; i0 += blockDim.x) {
      const uint32_t i = i0 + tid;
      const u64 k64 = i < cnt ? src[i] : 0;
      const bool cand = i < cnt && key64_okey(k64) >= thr;
      const uint32_t pos = wave_slot(cand, &sh_count);
      if (cand) {
        if (pos < kNucleusCap) lds_keys[pos] = k64;
      } else {
        best_below = k64 > best_below ? k64 : best_below;
      }
    }
  }
  best_below = block_max<u64>(best_below, red64);  // barriers inside also publish sh_count
  uint32_t n_c = sh_count;
  bool ok = n_c < kNucleusCap;  // room for the next-best element too
  if (ok) {
    if (best_below != 0 && tid == 0) lds_keys[n_c] = best_below;
    if (best_below != 0) n_c += 1;
    const int n2 = next_pow2(static_cast<int>(n_c));
    for (int p = static_cast<int>(n_c) + tid; p < n2; p += blockDim.x) lds_keys[p] = 0;
    __syncthreads();
    block_sort_desc(lds_keys, n2);
    // cache exp((s - max)/T) in the score half of every entry
    const float max_score = key_to_float(key64_okey(lds_keys[0]));
    __syncthreads();
    const float inv_temp = 1.0f / prm.temperature;
    for (uint32_t i = tid; i < n_c; i += blockDim.x) {
      const u64 k64 = lds_keys[i];
      const float e = em::expf_exact((key_to_float(key64_okey(k64)) - max_score) * inv_temp);
      lds_keys[i] = (static_cast<u64>(__float_as_uint(e)) << 32) | (k64 & 0xffffffffull);
    }
    __syncthreads();
    RowOutputs out{a.out_tokens + row, a.kept_count ? a.kept_count + row : nullptr,
                   a.kept_ids ? a.kept_ids + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                   a.kept_probs ? a.kept_probs + static_cast<size_t>(row) * a.kept_capacity : nullptr,
                   a.kept_capacity};
    const u64* lk = lds_keys;
    auto sorted = [=](int i) { return lk[i]; };
    auto exps = [=](int i) { return __uint_as_float(static_cast<uint32_t>(lk[i] >> 32)); };
    ok = block_sample_epilogue<4>(sorted, exps, static_cast<int>(n_c), V, prm, a.uniforms[row], out, seqsh);
  }
  if (!ok) {
    __syncthreads();
    general_row(a, row, big_row, seqsh);
  }
}

}  // namespace ms

extern "C" hipError_t ms_launch_sample(const ms::SampleArgs* a, bool any_nucleus, hipStream_t stream) {
  dim3 grid(a->chunks, a->rows);
  hipLaunchKernelGGL(ms::sample_stream_kernel, grid, dim3(ms::kBlock), 0, stream, *a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (any_nucleus) {
    hipLaunchKernelGGL(ms::nucleus_finish_kernel, dim3(a->rows), dim3(ms::kFinishBlock),
                       ms::kNucleusCap * sizeof(ms::u64), stream, *a);
    e = hipGetLastError();
  }
  return e;
}

extern "C" hipError_t ms_sample_init() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(ms::nucleus_finish_kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize,
                             ms::kNucleusCap * sizeof(ms::u64));
}
