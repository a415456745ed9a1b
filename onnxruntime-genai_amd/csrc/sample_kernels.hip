// Finish kernels of the nucleus / large-k sampling paths, the fp32 streaming kernels and the launch logic of
// mi355x_sample (the streaming kernels of fp16 and bf16 rows are instantiated in sample_kernels_f16.hip and
// sample_kernels_bf16.hip from the same templates).
#include "sample_stream.h"

extern "C" {
hipError_t ms_launch_stream(const ms::SampleArgs* a, const ms::InlineParams* table, int which, hipStream_t stream);
hipError_t ms_launch_stream_f16(const ms::SampleArgs* a, const ms::InlineParams* table, int which, hipStream_t stream);
hipError_t ms_launch_stream_bf16(const ms::SampleArgs* a, const ms::InlineParams* table, int which, hipStream_t stream);
}

namespace ms {

// Sorts n keys (kFinishBlock < n <= kNucleusCap) in LDS, descending, by a block of kFinishBlock
// threads: a counting pass over kSortBuckets buckets that are linear in the score (bucket 0 holds the
// best scores) groups the keys, then every key finds its rank inside its bucket by comparing whole
// keys.  The bucket of a score is a monotone function of it, so the result is the exact key order.
// Returns false -- keys untouched in value, possibly permuted -- when a bucket holds more than
// kBucketCap keys (heavy ties); the caller then uses the sorting network.
constexpr int kSortBuckets = 4096;
constexpr int kBucketCap = 64;
constexpr size_t kFinishLds = kNucleusCap * sizeof(u64) + (kSortBuckets + 1) * sizeof(uint32_t);

__device__ __noinline__ bool bucket_sort_desc(u64* keys, uint32_t* start, int n, float fmax, float fthr, uint32_t* red) {
  constexpr int R = kNucleusCap / kFinishBlock;
  const int t = threadIdx.x;
  u64 k[R];
  uint32_t info[R];  // bucket << 8 | slot inside the bucket, later the final position
#pragma unroll
  for (int r = 0; r < R; ++r) k[r] = r * kFinishBlock + t < n ? keys[r * kFinishBlock + t] : 0;
  for (int b = t; b <= kSortBuckets; b += kFinishBlock) start[b] = 0u;
  __syncthreads();
  const float span = fmax - fthr;
  const float scale = span > 0.0f ? static_cast<float>(kSortBuckets) / span : 0.0f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r * kFinishBlock + t < n) {
      const float x = key_to_float(key64_okey(k[r]));
      float bf = (fmax - x) * scale;
      bf = bf < static_cast<float>(kSortBuckets - 1) ? bf : static_cast<float>(kSortBuckets - 1);  // also NaN-safe
      const uint32_t b = bf > 0.0f ? static_cast<uint32_t>(bf) : 0u;
      const uint32_t slot = atomicAdd(&start[b], 1u);
      info[r] = (b << 8) | (slot < 255u ? slot : 255u);
    }
  }
  __syncthreads();
  // exclusive scan of the bucket counts (4 consecutive buckets per thread) and the size check
  constexpr int kPer = kSortBuckets / kFinishBlock;
  uint32_t cnt[kPer], local = 0u, big = 0u;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    cnt[i] = start[t * kPer + i];
    local += cnt[i];
    big |= cnt[i] > static_cast<uint32_t>(kBucketCap) ? 1u : 0u;
  }
  uint32_t inc = local;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t y = __shfl_up(inc, d, 64);
    if ((t & 63) >= d) inc += y;
  }
  const uint32_t any_big = block_max<uint32_t>(big, red);
  if ((t & 63) == 63) red[t >> 6] = inc;
  __syncthreads();
  if (any_big) return false;
  uint32_t base = inc - local;
  for (int w = 0; w < (t >> 6); ++w) base += red[w];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    start[t * kPer + i] = base;
    base += cnt[i];
  }
  if (t == kFinishBlock - 1) start[kSortBuckets] = base;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (r * kFinishBlock + t < n) keys[start[info[r] >> 8] + (info[r] & 255u)] = k[r];
  __syncthreads();
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r * kFinishBlock + t < n) {
      const uint32_t b = info[r] >> 8;
      const uint32_t lo = start[b], hi = start[b + 1];
      uint32_t rank = 0u;
      for (uint32_t j = lo; j < hi; ++j) rank += keys[j] > k[r] ? 1u : 0u;
      info[r] = lo + rank;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (r * kFinishBlock + t < n) keys[info[r]] = k[r];
  __syncthreads();
  return true;
}

// Sorts n2 keys (a power of two, at least two tiles) in global memory, descending, by a block of
// kFinishBlock threads with a tile of kNucleusCap keys in LDS: every tile is sorted in LDS (alternating
// directions), then the remaining levels of the bitonic network run their long-distance steps in
// global memory and the 14 short-distance steps of each level tile by tile in LDS.  About twice as
// fast as the same network entirely in global memory.
__device__ __forceinline__ void tiled_sort_desc(u64* g, int n2, u64* lds) {
  constexpr int T = kNucleusCap;
  const int tid = threadIdx.x;
  const int tiles = n2 / T;
  for (int t = 0; t < tiles; ++t) {
    u64* src = g + static_cast<size_t>(t) * T;
    for (int i = tid; i < T; i += kFinishBlock) lds[i] = src[i];
    __syncthreads();
    // the whole tile, zeros last; the plain network, inline: a call to one of the faster out-of-line sorts inside
    // this loop makes the kernel spill, and a kernel that uses scratch memory at all starts 2.5 us later
    block_sort_desc(lds, T);
#pragma unroll 4
    for (int i = tid; i < T; i += kFinishBlock) src[(t & 1) ? T - 1 - i : i] = lds[i];
    __syncthreads();
  }
  for (int k = 2 * T; k <= n2; k <<= 1) {
    for (int j = k >> 1; j >= T; j >>= 1) {
#pragma unroll 2
      for (int p = tid; p < n2 / 2; p += kFinishBlock) {
        const int i = ((p & ~(j - 1)) << 1) | (p & (j - 1));  // bit j clear
        const u64 x = g[i], y = g[i | j];
        const bool desc = (i & k) == 0;
        if ((x < y) == desc) {
          g[i] = y;
          g[i | j] = x;
        }
      }
      __syncthreads();
    }
    for (int t = 0; t < tiles; ++t) {
      u64* src = g + static_cast<size_t>(t) * T;
#pragma unroll 4
      for (int i = tid; i < T; i += kFinishBlock) lds[i] = src[i];
      __syncthreads();
      const bool desc = ((t * T) & k) == 0;  // one direction per tile: k >= 2 T
      for (int j = T >> 1; j >= 1; j >>= 1) {
#pragma unroll 2
        for (int p = tid; p < T / 2; p += kFinishBlock) {
          const int i = ((p & ~(j - 1)) << 1) | (p & (j - 1));
          const u64 x = lds[i], y = lds[i | j];
          if ((x < y) == desc) {
            lds[i] = y;
            lds[i | j] = x;
          }
        }
        __syncthreads();
      }
#pragma unroll 4
      for (int i = tid; i < T; i += kFinishBlock) src[i] = lds[i];
      __syncthreads();
    }
  }
}

// Per-row finish of the nucleus path: gathers the candidates the streaming pass left in `big`,
// sorts them in LDS and runs the exact epilogue.  One block of kFinishBlock threads per row;
// dynamic LDS: kNucleusCap key64s + the bucket table of the sort.
template <bool INLINE, bool LARGEK>
__device__ __forceinline__ void nucleus_finish_body(const SampleArgs& a) {
  extern __shared__ u64 lds_keys[];
  uint32_t* bucket_start = reinterpret_cast<uint32_t*>(lds_keys + kNucleusCap);  // kSortBuckets + 1 entries
  __shared__ SeqShared seqsh;
  __shared__ uint32_t sh_count;
  __shared__ uint32_t red32[16];
  __shared__ u64 red64[16];
  const int row = blockIdx.x;
  const int V = a.vocab;
  const int tid = threadIdx.x;
  const mi355x_sample_params prm = row_params<INLINE>(a, row);
  if (row_mode(prm, V, a.chunks) != (LARGEK ? kModeTopkLarge : kModeNucleus)) return;
  constexpr bool large_k = LARGEK;  // then every listed element is a candidate and no element after them is needed
  u64* big_row = a.big + static_cast<size_t>(row) * a.big_stride;
  const size_t cbase = static_cast<size_t>(row) * a.chunks;
  // The head of every chunk's list (kAhead entries per thread) is requested before the counts are
  // known -- whatever lies past a list's end is discarded later -- so that these loads overlap the
  // round trip for the counts.  Rows of more than kAheadChunks chunks, and rows whose lists hold more
  // than the sort has room for, read everything afterwards.
  constexpr int kGather = 8, kAheadChunks = 8, kAhead = 2;  // kGather: entries a thread has in flight
  static_assert((kAheadChunks * kAhead) % kGather == 0, "the head is consumed in whole batches");
  u64 pre[kAheadChunks * kAhead];
#pragma unroll
  for (int c = 0; c < kAheadChunks; ++c)
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
      pre[c * kAhead + u] =
          (a.chunks <= kAheadChunks && c < a.chunks) ? big_row[static_cast<size_t>(c) * kSChunk + u * kFinishBlock + tid] : 0;
  // Thread c reads everything chunk c left behind; the barriers of the first reduction publish the counts.
  __shared__ uint32_t sh_cnt[kAllCap / kSmallCap];       // candidates per chunk
  __shared__ uint32_t sh_first[kAllCap / kSmallCap + 1];  // their prefix sums
  __shared__ int sh_trim;
  __shared__ uint32_t sh_head, sh_all;
  uint32_t m = 0u;
  u64 best_below = 0;
  if (tid < a.chunks) {
    const uint32_t cnt = a.chunk_cnt[cbase + tid];
    m = cnt == kChunkCntOverflow ? 0xffffffffu : a.chunk_max[cbase + tid];  // above every key: the exact path
    best_below = large_k ? 0 : a.chunk_next[cbase + tid];
    sh_cnt[tid] = cnt;
  }
  if (tid == 0) sh_count = 0u;
  const uint32_t rmax = block_max<uint32_t>(m, red32);
  const bool gave_up = rmax == 0xffffffffu;
  uint32_t thr = 0u;
  if (rmax != 0u && !large_k) thr = order_key(key_to_float(rmax) - nucleus_depth(prm, V));
  if (tid == 0) {
    uint32_t all = 0u;
    for (int c = 0; c < a.chunks; ++c) all += gave_up ? 0u : sh_cnt[c];
    const uint32_t head =
        (a.chunks <= kAheadChunks && all < static_cast<uint32_t>(kNucleusCap)) ? kAhead * kFinishBlock : 0u;
    uint32_t run = 0u;
    for (int c = 0; c < a.chunks; ++c) {
      sh_first[c] = run;
      run += (gave_up || sh_cnt[c] <= head) ? 0u : sh_cnt[c] - head;
    }
    sh_first[a.chunks] = run;
    sh_head = head;
    sh_all = all;
  }
  __syncthreads();
  const int lane = lane_id();
  // Calls fn(entries, valid) for batches of kGather entries per thread of the flat sequence made of the
  // chunks' lists past their heads (sh_first[c] = such entries of the chunks before c).
  const uint32_t head = sh_head;
  auto flat_batches = [&](auto fn) {
    const uint32_t total = sh_first[a.chunks];
    for (uint32_t f0 = 0; f0 < total; f0 += kGather * blockDim.x) {
      u64 raw[kGather];
      bool valid[kGather];
#pragma unroll
      for (int u = 0; u < kGather; ++u) {
        const uint32_t f = f0 + u * blockDim.x + tid;
        raw[u] = 0;
        valid[u] = f < total;
        if (valid[u]) {
          int c = 0;
          for (int cc = 1; cc < a.chunks; ++cc) c += f >= sh_first[cc] ? 1 : 0;
          raw[u] = big_row[static_cast<size_t>(c) * kSChunk + head + (f - sh_first[c])];
        }
      }
      fn(raw, valid);
    }
  };
  // More candidates listed than the sort holds (a flat distribution): the threshold is raised to the
  // lowest score that still leaves room, found from a histogram of the candidates over the sort's
  // score-linear buckets.  The nucleus test of the epilogue only looks at the elements it is given, in
  // rank order, and reports when they do not contain the nucleus; only then does the row need the
  // exact path.
  bool trim_failed = false;
  if (!large_k && sh_all >= static_cast<uint32_t>(kNucleusCap)) {  // head == 0 here
    const float fmax = key_to_float(rmax), fthr = key_to_float(thr);
    const float span = fmax - fthr;
    const float scale = span > 0.0f ? static_cast<float>(kSortBuckets) / span : 0.0f;
    auto bucket_of = [=](float x) {
      float bf = (fmax - x) * scale;
      bf = bf < static_cast<float>(kSortBuckets - 1) ? bf : static_cast<float>(kSortBuckets - 1);
      return bf > 0.0f ? static_cast<int>(bf) : 0;
    };
    for (int b = tid; b < kSortBuckets; b += kFinishBlock) bucket_start[b] = 0u;
    __syncthreads();
    const uint32_t thr0 = thr;
    flat_batches([&](const u64 (&raw)[kGather], const bool (&valid)[kGather]) {
#pragma unroll
      for (int u = 0; u < kGather; ++u) {
        const float x = __uint_as_float(static_cast<uint32_t>(raw[u] >> 32));
        if (valid[u] && order_key(x) >= thr0) atomicAdd(&bucket_start[bucket_of(x)], 1u);
      }
    });
    __syncthreads();
    // last bucket up to which the candidates fit (one slot stays free for the element after them)
    if (tid < 64) {
      constexpr int kPer = kSortBuckets / 64;
      const uint32_t limit = static_cast<uint32_t>(kNucleusCap - 2);
      uint32_t own = 0u;
      for (int i = 0; i < kPer; ++i) own += bucket_start[tid * kPer + i];
      uint32_t inc = own;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t y = __shfl_up(inc, d, 64);
        if (lane >= d) inc += y;
      }
      const int crossing = first_lane(__ballot(inc > limit));  // -1: everything fits
      if (crossing < 0) {
        if (tid == 0) sh_trim = kSortBuckets - 1;
      } else if (tid == crossing) {
        uint32_t run = inc - own;
        int last = tid * kPer - 1;
        for (int i = 0; i < kPer; ++i) {
          run += bucket_start[tid * kPer + i];
          if (run > limit) break;
          last = tid * kPer + i;
        }
        sh_trim = last;
      }
    }
    __syncthreads();
    const int last_bucket = sh_trim;
    if (last_bucket < 0) {
      trim_failed = true;  // the best bucket alone does not fit (heavy ties)
    } else if (last_bucket < kSortBuckets - 1) {
      // the lowest score whose bucket is still kept: the bucket is a non-increasing function of the score
      uint32_t lo = thr, hi = rmax;
      while (lo < hi) {
        const uint32_t mid = lo + ((hi - lo) >> 1);
        if (bucket_of(key_to_float(mid)) <= last_bucket) hi = mid;
        else lo = mid + 1u;
      }
      thr = hi;
    }
  }
  // A batch of kGather entries per thread: float bits become order keys, candidates (at or above the
  // row's threshold) go to LDS at slots a wave reserves with one atomic per batch, the best of the
  // others is kept.
  uint32_t lowest = 0xffffffffu;  // lowest candidate key this thread has seen
  auto consume = [&](const u64 (&raw)[kGather], const bool (&valid)[kGather]) {
    u64 k64[kGather], hits[kGather];
    uint32_t wcnt = 0u;
#pragma unroll
    for (int u = 0; u < kGather; ++u) {
      k64[u] = valid[u] ? (static_cast<u64>(order_key(__uint_as_float(static_cast<uint32_t>(raw[u] >> 32)))) << 32) |
                              (raw[u] & 0xffffffffull)
                        : 0;
      const bool cand = valid[u] && key64_okey(k64[u]) >= thr;
      hits[u] = __ballot(cand);
      wcnt += static_cast<uint32_t>(__popcll(hits[u]));
      if (!cand) best_below = k64[u] > best_below ? k64[u] : best_below;
      if (cand && key64_okey(k64[u]) < lowest) lowest = key64_okey(k64[u]);
    }
    uint32_t base = 0u;
    if (lane == 0 && wcnt != 0u) base = atomicAdd(&sh_count, wcnt);
    base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
    for (int u = 0; u < kGather; ++u) {
      const uint32_t pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(hits[u] >> 32),
                                                     __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(hits[u]), base));
      if (((hits[u] >> lane) & 1ull) && pos < kNucleusCap) lds_keys[pos] = k64[u];
      base += static_cast<uint32_t>(__popcll(hits[u]));
    }
  };
  if (head != 0u) {
#pragma unroll
    for (int b = 0; b < kAheadChunks * kAhead / kGather; ++b) {
      if (b * kGather / kAhead < a.chunks) {
        u64 raw[kGather];
        bool valid[kGather];
#pragma unroll
        for (int u = 0; u < kGather; ++u) {
          const int q = b * kGather + u, c = q / kAhead;
          raw[u] = pre[q];
          valid[u] = c < a.chunks && static_cast<uint32_t>((q % kAhead) * kFinishBlock + tid) < sh_cnt[c < a.chunks ? c : 0];
        }
        consume(raw, valid);
      }
    }
  }
  flat_batches(consume);
  best_below = block_max<u64>(best_below, red64);  // barriers inside also publish sh_count
  uint32_t n_c = sh_count;
  bool ok = !gave_up && !trim_failed && n_c < kNucleusCap;  // room for the next-best element too
  if (large_k) thr = ~block_max<uint32_t>(~lowest, red32);  // the lowest candidate score: the sort scales its buckets by it
  if (ok) {
    if (best_below != 0 && tid == 0) lds_keys[n_c] = best_below;
    if (best_below != 0) n_c += 1;
    __syncthreads();
    bool sorted_done = false;
    if (n_c > static_cast<uint32_t>(kFinishBlock) && rmax != 0u) {
      sorted_done = bucket_sort_desc(lds_keys, bucket_start, static_cast<int>(n_c), key_to_float(rmax),
                                     key_to_float(thr), red32);
    }
    if (!sorted_done) {
      const int n2 = next_pow2(static_cast<int>(n_c));
      for (int p = static_cast<int>(n_c) + tid; p < n2; p += blockDim.x) lds_keys[p] = 0;
      __syncthreads();
      switch (n2 / kFinishBlock) {
        case 0:
        case 1: block_sort_desc(lds_keys, n2); break;
        case 2: block_sort_desc_regs<2>(lds_keys); break;
        case 4: block_sort_desc_regs<4>(lds_keys); break;
        case 8: block_sort_desc_regs<8>(lds_keys); break;
        default: block_sort_desc_regs<16>(lds_keys); break;
      }
    }
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
    const u64* lk = lds_keys;
    auto sorted = [=](int i) { return lk[i]; };
    auto exps = [=](int i) { return __uint_as_float(static_cast<uint32_t>(lk[i] >> 32)); };
    ok = block_sample_epilogue<4>(sorted, exps, static_cast<int>(n_c), V, prm, a.uniforms[row], row_outputs(a, row), seqsh);
  }
  if (!ok) {
    __syncthreads();
    u64* const tile = lds_keys;
    general_row<AnyDtype>(a, row, row_start<INLINE>(a, row, dtype_bytes(a.dtype)), prm, big_row, seqsh, [=](u64* keys, int n2, int n_real) {
      if (n2 >= 2 * kNucleusCap) tiled_sort_desc(keys, n2, tile);
      else block_sort_desc(keys, n2);
    });
  }
}

__global__ __launch_bounds__(kFinishBlock) void nucleus_finish_kernel(const SampleArgs a) { nucleus_finish_body<false, false>(a); }
__global__ __launch_bounds__(kFinishBlock) void nucleus_finish_rows_kernel(const SampleArgs a, const InlineParams) {
  nucleus_finish_body<true, false>(a);
}
__global__ __launch_bounds__(kFinishBlock) void largek_finish_kernel(const SampleArgs a) { nucleus_finish_body<false, true>(a); }
__global__ __launch_bounds__(kFinishBlock) void largek_finish_rows_kernel(const SampleArgs a, const InlineParams) {
  nucleus_finish_body<true, true>(a);
}

}  // namespace ms

MS_STREAM_KERNELS(, float)  // the fp32 streaming kernels live here, next to the finish kernels

extern "C" hipError_t ms_launch_sample(const ms::SampleArgs* a, const ms::InlineParams* table, bool any_other,
                                       bool any_nucleus, bool any_large_k, hipStream_t stream) {
  const dim3 fgrid(a->rows), fblock(ms::kFinishBlock);
  auto launch_stream = a->dtype == MI355X_F16 ? ms_launch_stream_f16 : a->dtype == MI355X_BF16 ? ms_launch_stream_bf16 : ms_launch_stream;
  hipError_t e = hipSuccess;
  if (any_other) {
    e = launch_stream(a, table, 0, stream);
    if (e != hipSuccess) return e;
  }
  if (any_nucleus) {
    e = launch_stream(a, table, 1, stream);
    if (e != hipSuccess) return e;
    if (table) hipLaunchKernelGGL(ms::nucleus_finish_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a, *table);
    else hipLaunchKernelGGL(ms::nucleus_finish_kernel, fgrid, fblock, ms::kFinishLds, stream, *a);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (any_large_k) {
    e = launch_stream(a, table, 2, stream);
    if (e != hipSuccess) return e;
    if (table) hipLaunchKernelGGL(ms::largek_finish_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a, *table);
    else hipLaunchKernelGGL(ms::largek_finish_kernel, fgrid, fblock, ms::kFinishLds, stream, *a);
    e = hipGetLastError();
  }
  return e;
}

extern "C" hipError_t ms_sample_init() {
  const void* finish[] = {reinterpret_cast<const void*>(ms::nucleus_finish_kernel),
                          reinterpret_cast<const void*>(ms::nucleus_finish_rows_kernel),
                          reinterpret_cast<const void*>(ms::largek_finish_kernel),
                          reinterpret_cast<const void*>(ms::largek_finish_rows_kernel)};
  for (const void* f : finish) {
    const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, ms::kFinishLds);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}
