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
constexpr int kSortBuckets = 7168;  // what fits next to the keys in 160 KB of LDS; a multiple of kFinishBlock
constexpr int kBucketCap = 64;
constexpr size_t kFinishLds = kNucleusCap * sizeof(u64) + (kSortBuckets + 1) * sizeof(uint32_t);

// R: keys per thread the code provides for (n <= R * kFinishBlock); a list of a quarter or half of the capacity
// gets code whose unrolled loops are that much shorter.
template <int R>
__device__ __noinline__ bool bucket_sort_desc_sized(u64* keys, uint32_t* start, int n, float fmax, float fthr, uint32_t* red) {
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
  uint32_t inc = wave_prefix_sum<uint32_t>(local);
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
  // info becomes: where the bucket starts | keys in the bucket << 16 (a bucket holds at most kBucketCap keys)
  static_assert(kBucketCap < 256 && kNucleusCap <= 65536, "the packing of info");
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r * kFinishBlock + t < n) {
      const uint32_t b = info[r] >> 8;
      const uint32_t lo = start[b];
      keys[lo + (info[r] & 255u)] = k[r];
      info[r] = lo | ((start[b + 1] - lo) << 16);
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r * kFinishBlock + t < n) {
      const uint32_t lo = info[r] & 0xffffu, hi = lo + (info[r] >> 16);
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

__device__ __forceinline__ bool bucket_sort_desc(u64* keys, uint32_t* start, int n, float fmax, float fthr, uint32_t* red) {
  constexpr int kFull = kNucleusCap / kFinishBlock;
  if (n <= kFull / 4 * kFinishBlock) return bucket_sort_desc_sized<kFull / 4>(keys, start, n, fmax, fthr, red);
  if (n <= kFull / 2 * kFinishBlock) return bucket_sort_desc_sized<kFull / 2>(keys, start, n, fmax, fthr, red);
  return bucket_sort_desc_sized<kFull>(keys, start, n, fmax, fthr, red);
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

// Sorts n distinct keys in global memory, descending, by a block of kFinishBlock threads that has kFinishLds
// bytes of LDS, with a second global buffer `alt` of n keys: a most-significant-digit radix sort with
// kRadixDigits digits.  The first level's digit is linear in the score between the row's largest and smallest
// ordinary value (everything at or below lowest() and every NaN lands in the last digit), which spreads a
// smooth distribution evenly; a refinement level's digit is linear in the 64-bit key between the largest and
// smallest key of its range.  Per level: one pass counts the keys per digit, one scatters them into `alt`
// digit by digit, then runs of consecutive digits that fit the LDS tile are loaded, every key finds its rank
// among the keys of its digit by comparing, and goes to its final place.  A digit of more than kRankCap keys
// goes back unsorted and is refined over its own, narrower key range.  Every key moves through memory three
// times per level (the seventeen levels of a sorting network over a 128K row move it forty times).  All
// inline: an out-of-line call in here makes the calling kernels use scratch memory.  Returns false, with
// `keys` some permutation of its input, when more ranges need refinement than the list holds.
constexpr int kRadixDigits = 16384;
constexpr int kRadixTile = static_cast<int>(kFinishLds / sizeof(u64)) - (kRadixDigits + 2) / 2;  // keys of a run
constexpr int kRankCap = 512;
constexpr int kRadixStack = 32;
static_assert(kRadixTile * sizeof(u64) >= kRadixDigits * sizeof(uint32_t), "the scatter cursors use the tile");

// Runs BODY with K = SRC[I] for I in [0, CNT), eight loads per thread in flight.  A macro: closures that capture
// the loop's state by reference end up in scratch memory here.
#define MS_FOR_KEYS(SRC, CNT, K, I, BODY)                                                                   \
  for (uint32_t i0_ = threadIdx.x; i0_ < (CNT); i0_ += 8 * kFinishBlock) {                                  \
    u64 kb_[8];                                                                                             \
    _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_)                                                        \
        kb_[u_] = i0_ + u_ * kFinishBlock < (CNT) ? (SRC)[i0_ + u_ * kFinishBlock] : 0;                     \
    _Pragma("unroll") for (int u_ = 0; u_ < 8; ++u_) {                                                      \
      if (i0_ + u_ * kFinishBlock < (CNT)) {                                                                \
        const u64 K = kb_[u_];                                                                              \
        const uint32_t I = i0_ + u_ * kFinishBlock;                                                         \
        BODY                                                                                                \
      }                                                                                                     \
    }                                                                                                       \
  }

__device__ __forceinline__ bool radix_rank_sort_desc(u64* keys, u64* alt, int n, u64* lds, uint32_t* red32, u64* red64) {
  __shared__ uint32_t stack_pos[kRadixStack], stack_cnt[kRadixStack];
  __shared__ int stack_n, failed;
  const int tid = threadIdx.x;
  uint32_t* const hist = reinterpret_cast<uint32_t*>(lds);  // kRadixDigits + 1 running totals
  u64* const tile = lds + (kRadixDigits + 2) / 2;
  uint32_t* const cursor = reinterpret_cast<uint32_t*>(tile);  // while a range is scattered
  if (tid == 0) {
    stack_n = 1;
    stack_pos[0] = 0u;
    stack_cnt[0] = static_cast<uint32_t>(n);
    failed = 0;
  }
  for (int level = 0; level < 64 * kRadixStack; ++level) {
    __syncthreads();
    const int sn = stack_n;
    if (sn == 0 || failed) break;
    const uint32_t pos = stack_pos[sn - 1], cnt = stack_cnt[sn - 1];
    __syncthreads();
    if (tid == 0) stack_n = sn - 1;
    u64* const src = keys + pos;
    u64* const dst = alt + pos;
    // the range of the keys, and of the ordinary scores among them
    const uint32_t ordinary = order_key(-1e30f);
    u64 kmin = ~0ull, kmax = 0ull;
    uint32_t omin = 0xffffffffu;
    MS_FOR_KEYS(src, cnt, k, i, {
      (void)i;
      kmin = k < kmin ? k : kmin;
      kmax = k > kmax ? k : kmax;
      const uint32_t o = key64_okey(k);
      omin = (o > ordinary && o < omin) ? o : omin;
    })
    kmax = block_max<u64>(kmax, red64);
    kmin = ~block_max<u64>(~kmin, red64);
    omin = ~block_max<uint32_t>(~omin, red32);
    const u64 span = kmax - kmin;
    if (span == 0ull && cnt > 1u) {  // equal keys cannot be told apart: not a row of (score, id) keys
      if (tid == 0) failed = 1;
      continue;
    }
    const float fmax = key_to_float(key64_okey(kmax));
    const float fmin = key_to_float(omin);
    const float fspan = fmax - fmin;
    const bool by_score = level == 0 && fmax < 3.0e38f && omin != 0xffffffffu && fspan > 0.0f && fspan < 3.0e38f;
    const float scale = by_score ? static_cast<float>(kRadixDigits) / fspan : 0.0f;
    const int bits = span != 0ull ? 64 - __clzll(span) : 0;
    const int shift = bits > 14 ? bits - 14 : 0;  // (kmax - k) >> shift < kRadixDigits
    static_assert(kRadixDigits == 1 << 14, "the shift above");
    auto digit = [=](u64 k) -> uint32_t {
      if (by_score) {
        float bf = (fmax - key_to_float(key64_okey(k))) * scale;
        bf = bf < static_cast<float>(kRadixDigits - 1) ? bf : static_cast<float>(kRadixDigits - 1);  // also NaN-safe
        return bf > 0.0f ? static_cast<uint32_t>(bf) : 0u;
      }
      return static_cast<uint32_t>((kmax - k) >> shift);
    };
    for (int b = tid; b <= kRadixDigits; b += kFinishBlock) hist[b] = 0u;
    __syncthreads();
    const bool one_digit = cnt <= static_cast<uint32_t>(kRankCap);
    if (one_digit) {
      if (tid == 0) hist[0] = cnt;  // one digit holds the whole range
    } else {
      MS_FOR_KEYS(src, cnt, k, i, {
        (void)i;
        atomicAdd(&hist[digit(k)], 1u);
      })
    }
    __syncthreads();
    {  // exclusive scan of the digit counts: wave w owns kPer * 64 consecutive digits, 64 at a time; oversize
       // digits join the list
      constexpr int kPer = kRadixDigits / kFinishBlock;
      const int lane = tid & 63, wave = tid >> 6;
      uint32_t own = 0u;
#pragma unroll 4
      for (int i = 0; i < kPer; ++i) own += hist[(wave * kPer + i) * 64 + lane];
      own = wave_sum<uint32_t>(own);
      if (lane == 0) red32[wave] = own;
      __syncthreads();
      uint32_t run = 0u;
      for (int w = 0; w < wave; ++w) run += red32[w];
#pragma unroll 2
      for (int i = 0; i < kPer; ++i) {
        const int d0 = (wave * kPer + i) * 64 + lane;
        const uint32_t c = hist[d0];
        uint32_t inc = wave_prefix_sum<uint32_t>(c);
        const uint32_t base = run + inc - c;
        hist[d0] = base;
        cursor[d0] = base;
        if (c > static_cast<uint32_t>(kRankCap)) {
          const int at = atomicAdd(&stack_n, 1);
          if (at < kRadixStack) {
            stack_pos[at] = pos + base;
            stack_cnt[at] = c;
          } else {
            failed = 1;
          }
        }
        run += wave_read_lane(inc, 63);
      }
      if (tid == kFinishBlock - 1) hist[kRadixDigits] = run;
    }
    __syncthreads();
    if (failed) break;  // nothing has moved yet
    MS_FOR_KEYS(src, cnt, k, i, { dst[one_digit ? i : atomicAdd(&cursor[digit(k)], 1u)] = k; })
    __syncthreads();
    int b0 = 0;
    while (b0 < kRadixDigits) {
      const uint32_t base = hist[b0];
      int lo = b0, hi = kRadixDigits;  // the last digit boundary up to which the keys from b0 on fit the tile
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (hist[mid] - base <= static_cast<uint32_t>(kRadixTile)) lo = mid;
        else hi = mid - 1;
      }
      if (lo == b0) {  // a digit larger than the tile: back unsorted (it is on the list)
        const uint32_t c = hist[b0 + 1] - base;
        MS_FOR_KEYS(dst + base, c, k, i, { src[base + i] = k; })
        b0 += 1;
        continue;
      }
      const uint32_t c = hist[lo] - base;
      if (c != 0u) {
        MS_FOR_KEYS(dst + base, c, k, i, { tile[i] = k; })
        __syncthreads();
        for (uint32_t i = tid; i < c; i += kFinishBlock) {
          const u64 k = tile[i];
          const uint32_t d = one_digit ? 0u : digit(k);
          const uint32_t first = hist[d], last = hist[d + 1];
          uint32_t at = base + i;  // an oversize digit stays where it is
          if (last - first <= static_cast<uint32_t>(kRankCap)) {
            uint32_t rank = 0u, j = first - base;
            const uint32_t end = last - base;
            for (; j + 4 <= end; j += 4) {  // four independent reads in flight
              const u64 x0 = tile[j], x1 = tile[j + 1], x2 = tile[j + 2], x3 = tile[j + 3];
              rank += (x0 > k ? 1u : 0u) + (x1 > k ? 1u : 0u) + (x2 > k ? 1u : 0u) + (x3 > k ? 1u : 0u);
            }
            for (; j < end; ++j) rank += tile[j] > k ? 1u : 0u;
            at = first + rank;
          }
          src[at] = k;
        }
        __syncthreads();
      }
      b0 = lo;
    }
  }
  __syncthreads();
  return failed == 0;
}

// The sort of the exact path in kernels that have the finish kernels' LDS: the radix sort above, else the network.
struct SortWithTile {
  u64* alt;
  u64* tile;  // the kernel's dynamic LDS (kFinishLds bytes)
  uint32_t* red32;
  u64* red64;
  __device__ __forceinline__ void operator()(u64* keys, int n2, int n_real) const {
    if (alt != nullptr && radix_rank_sort_desc(keys, alt, n_real, tile, red32, red64)) return;
    if (n2 >= 2 * kNucleusCap) tiled_sort_desc(keys, n2, tile);
    else block_sort_desc(keys, n2);
  }
};

// Where entry i of the sorted list lives once its exponential is cached in it: the epilogue's threads each read
// eight consecutive entries, 64 bytes apart from lane to lane, so entry i moves inside its group of eight to slot
// (i ^ (i >> 4)) & 7, which spreads those reads over all banks.
__device__ __forceinline__ uint32_t exp_slot(uint32_t i) { return (i & ~7u) | ((i ^ (i >> 4)) & 7u); }

// Where DeviceInterface::TopKScores wants a row's k best: ids and raw scores, best first (tokens null: not asked for).
struct EmitTopk {
  int32_t* tokens = nullptr;
  float* scores = nullptr;
  const void* row0 = nullptr;  // the row's logits, of type dtype
  int dtype = 0;
  __device__ __forceinline__ bool on() const { return tokens != nullptr; }
};

// The tail shared by the finish kernels: lds_keys[0 .. n_c) hold a row's candidates as key64s in any order,
// best_below (0: none) is the best element of the row that is not among them.  Sorts them together in LDS,
// caches the exponentials and runs the exact epilogue.  With cut_at_best_below the candidates that rank
// after best_below are dropped first (they are not a prefix of the row's order).  rmax / thr: order keys of
// the best and of (a bound below) the lowest candidate, which scale the buckets of the sort.  Returns false
// when the row needs the exact path (the epilogue found no end of the nucleus among the elements given).
// presorted: lds_keys[0 .. n_c) are sorted and hold their exponentials already (sort_gathered), only the epilogue is left.
__device__ __forceinline__ bool finish_candidates(u64* lds_keys, uint32_t* bucket_start, uint32_t n_c, u64 best_below,
                                                  uint32_t rmax, uint32_t thr, bool cut_at_best_below,
                                                  mi355x_sample_params prm, int V, double u, const RowOutputs& out,
                                                  SeqShared& seqsh, uint32_t* red32, EmitTopk emit = EmitTopk{},
                                                  bool presorted = false, u64 second_below = 0) {
  const int tid = threadIdx.x;
  const u64* lk = lds_keys;
  auto sorted = [=](int i) { return lk[exp_slot(static_cast<uint32_t>(i))]; };
  auto exps = [=](int i) { return __uint_as_float(static_cast<uint32_t>(lk[exp_slot(static_cast<uint32_t>(i))] >> 32)); };
  // (presorted: the list is sorted and carries its exponentials already; one call of the epilogue serves both cases)
  if (presorted && emit.on()) {
    const int kk = prm.k < V ? prm.k : V;
    if (n_c < static_cast<uint32_t>(kk)) return false;
    const RowPtr<AnyDtype> lrow(emit.row0, emit.dtype);
    for (int j = tid; j < kk; j += blockDim.x) {
      const uint32_t id = key64_index(lk[exp_slot(static_cast<uint32_t>(j))]);
      emit.tokens[j] = static_cast<int32_t>(id);
      emit.scores[j] = lrow[id];
    }
    return true;
  }
  if (!presorted) {
    if (best_below != 0 && tid == 0) {
      lds_keys[n_c] = best_below;
      if (second_below != 0) lds_keys[n_c + 1u] = second_below;  // (the element behind it, for lists that need it)
    }
    if (best_below != 0) n_c += second_below != 0 ? 2u : 1u;
    __syncthreads();
    bool sorted_done = false;
    if (n_c > static_cast<uint32_t>(kFinishBlock) && rmax != 0u) {
      sorted_done = bucket_sort_desc(lds_keys, bucket_start, static_cast<int>(n_c), key_to_float(rmax), key_to_float(thr), red32);
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
    if (emit.on()) {
      // DeviceInterface::TopKScores: the k best ids and their raw scores, best first (the value itself is read again:
      // keys do not tell -0 from +0); fewer than k numbers among the candidates: the exact path decides
      const int kk = prm.k < V ? prm.k : V;
      if (n_c < static_cast<uint32_t>(kk) || lds_keys[kk - 1] == 0) return false;
      const RowPtr<AnyDtype> lrow(emit.row0, emit.dtype);
      for (int j = tid; j < kk; j += blockDim.x) {
        const uint32_t id = key64_index(lds_keys[j]);
        emit.tokens[j] = static_cast<int32_t>(id);
        emit.scores[j] = lrow[id];
      }
      return true;
    }
    if (cut_at_best_below && best_below != 0) {
      // keys are distinct: exactly one thread finds it
      __shared__ uint32_t cut;
      for (uint32_t i = tid; i < n_c; i += blockDim.x)
        if (lds_keys[i] == best_below) cut = i + 1u;
      __syncthreads();
      n_c = cut;
    }
    // cache exp((s - max)/T) in the score half of every entry.  The epilogue's threads each read eight consecutive
    // entries, 64 bytes apart from lane to lane; entry i therefore moves inside its group of eight to slot
    // (i ^ (i >> 4)) & 7, which spreads those reads over all banks.  A group is read and rewritten by eight
    // neighbouring lanes in one pass of the loop, so the exchange happens in place.
    const float max_score = key_to_float(key64_okey(lds_keys[0]));
    __syncthreads();
    const float inv_temp = 1.0f / prm.temperature;
    auto slot_of = [](uint32_t i) { return exp_slot(i); };
    static_assert(kFinishBlock % 8 == 0 && kNucleusCap % 8 == 0, "whole groups per pass");
    for (uint32_t i = tid; i < ((n_c + 7u) & ~7u); i += blockDim.x) {
      const u64 k64 = i < n_c ? lds_keys[i] : 0;
      const float e = em::expf_exact((key_to_float(key64_okey(k64)) - max_score) * inv_temp);
      lds_keys[slot_of(i)] = (static_cast<u64>(__float_as_uint(e)) << 32) | (k64 & 0xffffffffull);
    }
    __syncthreads();
  }
  return block_sample_epilogue<8>(sorted, exps, static_cast<int>(n_c), V, prm, u, out, seqsh, true);  // (a barrier has just passed)
}

// Drops the candidates that certainly lie past the end of the nucleus, so that only the rest is sorted.
// FindNucleus stops at the first element i (in rank order) with prefix_i >= p * (prefix_i + (V - i - 1) * e_i).  A
// histogram of the candidates over the sort's score-linear buckets bounds both sides: after all elements of buckets
// 0 .. b the prefix is at least the sum of count * exp(lower edge), and the element that ends bucket b is at most
// exp(upper edge of b), so once  lower_bound(prefix) * (1 - p) >= p * (V - count so far) * exp(upper edge)  -- with 2 %
// to spare for the rounding of the reference's fp32 sums and of this estimate -- the stop lies at or before the end of
// bucket b.  Candidates of later buckets are dropped (the best of them becomes the element after the candidates),
// and thr rises to the lowest score of the buckets kept.  Only an estimate is at stake: the epilogue still decides
// on exact values and reports when the nucleus does not end among the elements it is given (then the exact path
// takes the row).  lds_keys[0 .. n_c) are the candidates in any order; table: kSortBuckets words.
constexpr uint32_t kTrimMin = 2048;  // shorter lists are sorted whole

__device__ __forceinline__ void trim_to_nucleus(u64* lds_keys, uint32_t* table, uint32_t& n_c, u64& best_below, uint32_t rmax,
                                                uint32_t& thr, mi355x_sample_params prm, int V, uint32_t* red32, u64* red64,
                                                uint32_t* counter) {
  if (n_c < kTrimMin || !(prm.p > 0.0f && prm.p < 1.0f)) return;
  constexpr int R = kNucleusCap / kFinishBlock;
  __shared__ int cut_bucket;
  const int tid = threadIdx.x, lane = tid & 63;
  const float fmax = key_to_float(rmax), fthr = key_to_float(thr);
  const float span = fmax - fthr;
  if (!(span > 0.0f) || !(span < 3.0e38f)) return;
  const float scale = static_cast<float>(kSortBuckets) / span;
  auto bucket_of = [=](float x) {
    float bf = (fmax - x) * scale;
    bf = bf < static_cast<float>(kSortBuckets - 1) ? bf : static_cast<float>(kSortBuckets - 1);
    return bf > 0.0f ? static_cast<int>(bf) : 0;
  };
  for (int b = tid; b < kSortBuckets; b += kFinishBlock) table[b] = 0u;
  if (tid == 0) cut_bucket = kSortBuckets;
  __syncthreads();
  if (tid == 0) *counter = 0u;  // (after the barrier: every thread has read the count of the list it came with)
  u64 k[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t i = static_cast<uint32_t>(r * kFinishBlock + tid);
    k[r] = i < n_c ? lds_keys[i] : 0;
    if (i < n_c) atomicAdd(&table[bucket_of(key_to_float(key64_okey(k[r])))], 1u);
  }
  __syncthreads();
  {
    // thread t owns buckets t * kPer .. (t + 1) * kPer - 1; bucket b spans scores fmax - (b + 1) / scale .. fmax - b / scale
    constexpr int kPer = kSortBuckets / kFinishBlock;
    __shared__ double scan_cnt[16], scan_mass[16];
    const int wave = tid >> 6;
    const float step = (1.0f / prm.temperature) / scale;  // exponent per bucket; the hardware's exp2 is exact enough for bounds
    const double p = static_cast<double>(prm.p);
    double cb[kPer], mb[kPer], cnt = 0.0, mass = 0.0;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int b = tid * kPer + i;
      cb[i] = static_cast<double>(table[b]);
      mb[i] = cb[i] * static_cast<double>(__expf(-static_cast<float>(b + 1) * step));
      cnt += cb[i];
      mass += mb[i];
    }
    const double cnt_inc = wave_scan_add(cnt), mass_inc = wave_scan_add(mass);
    if (lane == 63) {
      scan_cnt[wave] = cnt_inc;
      scan_mass[wave] = mass_inc;
    }
    __syncthreads();
    const double wc = row_scan_add(lane < kFinishBlock / 64 ? scan_cnt[lane] : 0.0);
    const double wm = row_scan_add(lane < kFinishBlock / 64 ? scan_mass[lane] : 0.0);
    double c = (wave > 0 ? wave_read_lane(wc, wave - 1) : 0.0) + (cnt_inc - cnt);
    double m = (wave > 0 ? wave_read_lane(wm, wave - 1) : 0.0) + (mass_inc - mass);
    uint32_t mine = static_cast<uint32_t>(kSortBuckets);
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int b = tid * kPer + i;
      c += cb[i];
      m += mb[i];
      // the stop lies at or before the end of bucket b
      const bool closed = m * (1.0 - p) >= 1.02 * p * (static_cast<double>(V) - c) * static_cast<double>(__expf(-static_cast<float>(b) * step));
      if (closed && mine == static_cast<uint32_t>(kSortBuckets)) mine = static_cast<uint32_t>(b);
    }
    const uint32_t first_closed = ~block_max<uint32_t>(~mine, red32);
    if (tid == 0) cut_bucket = static_cast<int>(first_closed);
  }
  __syncthreads();
  const int last_bucket = cut_bucket;
  if (last_bucket >= kSortBuckets - 1) return;  // nothing to drop
  // Everything down to half a bucket below the last kept bucket stays (a few keys more than needed: what matters is
  // that no key of a kept bucket is dropped, whatever the rounding of the bucket function).
  const uint32_t edge = order_key(fmax - (static_cast<float>(last_bucket) + 1.5f) / scale);
  const uint32_t thr2 = edge > thr ? edge : thr;
  // compaction: the candidates at or above thr2 go back to the front of the list (a wave reserves its range with
  // one atomic), the best of the others is kept
  uint32_t wave_total = 0u;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const bool have = k[r] != 0;
    const bool cand = have && key64_okey(k[r]) >= thr2;
    wave_total += static_cast<uint32_t>(__popcll(__ballot(cand)));
    if (have && !cand) best_below = k[r] > best_below ? k[r] : best_below;
  }
  uint32_t base = 0u;
  if (lane == 0 && wave_total != 0u) base = atomicAdd(counter, wave_total);
  base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const bool cand = k[r] != 0 && key64_okey(k[r]) >= thr2;
    const u64 bal = __ballot(cand);
    const uint32_t pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(bal >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(bal), base));
    if (cand) lds_keys[pos] = k[r];
    base += static_cast<uint32_t>(__popcll(bal));
  }
  best_below = block_max<u64>(best_below, red64);  // its barriers also publish the counter and the list
  n_c = *counter;
  thr = thr2;
}

// ---- the bucket sort in parts, with the trimming inside ---------------------------------------------------------
// The buckets of bucket_sort_desc, linear in the score below `top` (the score of order key rtop) down to the score of
// thr; scores above `top` share bucket 0 (whole keys are compared inside a bucket, so any monotone assignment sorts
// exactly).
struct ScoreBuckets {
  float top, scale;  // bucket = (top - score) * scale, within 0 .. kSortBuckets - 1
  __device__ __forceinline__ ScoreBuckets(uint32_t rtop, uint32_t thr) {
    top = key_to_float(rtop);
    const float span = top - key_to_float(thr);
    scale = span > 0.0f ? static_cast<float>(kSortBuckets) / span : 0.0f;
  }
  __device__ __forceinline__ uint32_t of_score(float score) const {  // (-0 and +0 share a bucket, as they share an order key)
    float bf = (top - score) * scale;
    bf = bf < static_cast<float>(kSortBuckets - 1) ? bf : static_cast<float>(kSortBuckets - 1);  // also NaN-safe
    return bf > 0.0f ? static_cast<uint32_t>(bf) : 0u;
  }
  __device__ __forceinline__ uint32_t operator()(uint32_t okey) const { return of_score(key_to_float(okey)); }
};

// What the scan keeps: the keys of buckets 0 .. last_bucket, n_sorted of them, in a list of n entries (one more
// when best_below, the best element below every candidate, follows them).  n = 0: the first thread's run of buckets
// alone overflows the room or holds a bucket of more than bucket_cap keys; the caller sorts another way.
struct TrimmedBuckets {
  uint32_t last_bucket, n_sorted, n;
  u64 best_below;
  // not 0: the kept buckets end short of the bucket where the nucleus certainly ends, so the list does not hold the
  // whole nucleus: 1: the room ends there, 2: the next thread's run has a bucket of more than bucket_cap keys
  uint32_t more;
  // the element after best_below in the row's order, when the caller found it (0: not in the list): entry n - 1 then
  u64 second_below;
};

// After a counting pass has left the number of candidates per bucket in start[0 .. kSortBuckets): turns the counts
// into the buckets' first places (start[kSortBuckets] = their total) and decides how many buckets the sort keeps.
// The histogram bounds where the nucleus certainly ends (the bound of trim_to_nucleus, in fp32 and per thread's run
// of buckets: it only has to be a bound, the epilogue decides on exact values and reports a nucleus that does not end
// among the entries it is given), so the buckets past that point need neither places nor ranks; and no more buckets
// are kept than fill room - 2 entries.  best_below: this thread's best element below the threshold (0: none); when
// every bucket is kept, the block's best such element follows the candidates.  want > 0: the row asks for its `want`
// best keys, whatever their mass: the kept buckets end with the thread's run that holds the want-th key.  Contains
// barriers; every thread gets the same result.  bucket_cap: the most keys of one bucket the caller ranks.
__device__ __forceinline__ TrimmedBuckets scan_buckets_and_trim(uint32_t* start, const ScoreBuckets& bucket_of, u64 best_below,
                                                                mi355x_sample_params prm, int V, int room, uint32_t* red32,
                                                                u64* red64, int want = 0, int bucket_cap = kBucketCap) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // exclusive scan of the counts (consecutive buckets per thread) with a lower bound of the mass next to it: every
  // key of bucket b weighs at least exp(-(b + 1) * step) times the weight of `top`
  constexpr int kPer = kSortBuckets / kFinishBlock;
  const float step = bucket_of.scale > 0.0f ? (1.0f / prm.temperature) / bucket_of.scale : 0.0f;  // exponent per bucket
  const bool trim = want == 0 && prm.p > 0.0f && prm.p < 1.0f && bucket_of.scale > 0.0f;
  const float ratio = __expf(-step);
  float edge = __expf(-static_cast<float>(t * kPer + 1) * step);
  uint32_t cnt[kPer], local = 0u, big = 0u;
  float mass = 0.0f;
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    cnt[i] = start[t * kPer + i];
    local += cnt[i];
    big |= cnt[i] > static_cast<uint32_t>(bucket_cap) ? 1u : 0u;
    mass += static_cast<float>(cnt[i]) * edge;
    edge *= ratio;
  }
  const uint32_t inc = wave_prefix_sum<uint32_t>(local);
  const float minc = wave_prefix_sum<float>(mass);
  if (lane == 63) red64[wave] = (static_cast<u64>(__float_as_uint(minc)) << 32) | inc;
  __syncthreads();
  const u64 of_wave = lane < kFinishBlock / 64 ? red64[lane] : 0;
  const uint32_t cw = wave_prefix_sum<uint32_t>(static_cast<uint32_t>(of_wave));
  const float mw = wave_prefix_sum<float>(__uint_as_float(static_cast<uint32_t>(of_wave >> 32)));
  const uint32_t n_cand = wave_read_lane(cw, kFinishBlock / 64 - 1);
  uint32_t c = (wave > 0 ? wave_read_lane(cw, wave - 1) : 0u) + inc - local;
  const float m = (wave > 0 ? wave_read_lane(mw, wave - 1) : 0.0f) + (minc - mass);
  // The stop of the nucleus search lies at or before the last element of bucket b once
  //   mass(0..b) * (1 - p) >= p * (V - count(0..b)) * exp(upper edge of b)
  // (2 % to spare for the roundings); when b is empty, the element that satisfies the rule is the first one of the
  // next bucket that is not.  A thread tests the bucket before its own: the first thread that finds the property
  // there and has a key of its own owns the last buckets the sort keeps.  (Bucket 0 may hold keys above its upper
  // edge: the test starts with thread 1.)  A thread whose buckets end beyond the room, or that has a bucket too full
  // to rank, ends the kept ones before it.  (`mine` holds four times the thread that ends them, plus TrimmedBuckets::more:
  // the lowest value wins, so the nucleus' own end goes first among equals.)
  uint32_t mine = 4u * static_cast<uint32_t>(kFinishBlock);
  if (trim && t > 0 && local != 0u) {
    const float pf = prm.p;
    if (m * (1.0f - pf) >= 1.02f * pf * static_cast<float>(static_cast<uint32_t>(V) - c) * __expf(-static_cast<float>(t * kPer - 1) * step))
      mine = 4u * static_cast<uint32_t>(t);
  }
  if (want > 0 && c < static_cast<uint32_t>(want) && c + local >= static_cast<uint32_t>(want)) mine = 4u * static_cast<uint32_t>(t);
  const bool run_fits = !(c + local > static_cast<uint32_t>(room - 2) || big != 0u);  // (this thread's run, with all before it)
  if (!run_fits) {
    const uint32_t before = 4u * static_cast<uint32_t>(t) - (big != 0u ? 2u : 3u);  // (thread t - 1, and why)
    big = t == 0 ? 1u : 0u;
    if (t != 0) mine = before < mine ? before : mine;
  }
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    start[t * kPer + i] = c;
    c += cnt[i];
  }
  if (t == kFinishBlock - 1) start[kSortBuckets] = c;
  // (its barrier also publishes the starts; red32 is not written again before the callers' next barrier)
  const uint32_t red = block_max<uint32_t>(big ? 0xffffffffu : ~mine, red32, false);
  TrimmedBuckets r{static_cast<uint32_t>(kSortBuckets), n_cand, 0u, 0, 0u};
  if (red == 0xffffffffu) return r;
  const uint32_t last_thread = (~red) >> 2;
  r.more = (~red) & 3u;
  if (last_thread < static_cast<uint32_t>(kFinishBlock)) {
    r.last_bucket = last_thread * kPer + (kPer - 1);
    r.n_sorted = r.n = start[r.last_bucket + 1u];
    // The reference's search notices a stop on the 16th, 64th, 256th ... element of a row only one element later
    // (src/sampling_distribution.h:166-181), so a list that ends exactly there may be one element short: it also gets
    // the next thread's run of buckets that holds a key, or, when nothing else is listed, the best element below.
    const uint32_t n = r.n_sorted;
    if (want == 0 && r.more == 0u && n >= 16u && (n & (n - 1u)) == 0u && ((__ffs(static_cast<int>(n)) - 1) & 1) == 0) {
      if (n == n_cand) {
        r.best_below = block_max<u64>(best_below, red64);
        r.n = n + (r.best_below != 0 ? 1u : 0u);
      } else {
        __syncthreads();  // (the reduction above left red32 to its readers)
        const bool later = static_cast<uint32_t>(t) > last_thread && local != 0u;
        const uint32_t nearest =
            block_max<uint32_t>(later ? (static_cast<uint32_t>(kFinishBlock - t) << 1) | (run_fits ? 1u : 0u) : 0u, red32);
        if (nearest & 1u) {  // (a run that does not fit the room, or has a bucket too full: the list stays as it is)
          const uint32_t next_thread = static_cast<uint32_t>(kFinishBlock) - (nearest >> 1);
          r.last_bucket = next_thread * kPer + (kPer - 1);
          r.n_sorted = r.n = start[r.last_bucket + 1u];
        }
      }
    }
  } else {
    r.best_below = block_max<u64>(best_below, red64);  // ranks after every candidate
    r.n = n_cand + (r.best_below != 0 ? 1u : 0u);
  }
  return r;
}

// The last part, once every kept key lies somewhere inside its bucket's places: the list is read back position by
// position (a thread's neighbours hold the neighbouring positions, so the lanes of a wave look at the same few
// buckets), a key's rank inside its bucket comes from comparing whole keys, and the pass that writes the final places
// caches exp((score - max) / T) in the score half of every entry, at exp_slot(rank), the way the epilogue reads the
// list (rmax: order key of the row's maximum).  SHIFTED: the keys were placed by counting start[b] up, so bucket b
// now lies between start[b - 1] and start[b]; otherwise between start[b] and start[b + 1].
template <bool SHIFTED>
__device__ __forceinline__ void rank_and_cache_exps(u64* keys, const uint32_t* start, const ScoreBuckets& bucket_of,
                                                    const TrimmedBuckets& kept, uint32_t rmax, float inv_temp) {
  const int t = threadIdx.x;
  constexpr int R = kNucleusCap / kFinishBlock;
  const uint32_t n_pad = (kept.n + 7u) & ~7u;
  u64 k[R];
  uint32_t fin[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (static_cast<uint32_t>(r * kFinishBlock) < n_pad) {
      const uint32_t pos = static_cast<uint32_t>(r * kFinishBlock + t);
      k[r] = pos == kept.n_sorted && pos < kept.n ? kept.best_below : 0;
      if (pos == kept.n_sorted + 1u && pos < kept.n) k[r] = kept.second_below;
      fin[r] = pos;
      if (pos < kept.n_sorted) {
        k[r] = keys[pos];
        const uint32_t b = bucket_of(key64_okey(k[r]));
        const uint32_t lo = SHIFTED ? (b > 0u ? start[b - 1u] : 0u) : start[b];
        const uint32_t hi = SHIFTED ? start[b] : start[b + 1u];
        uint32_t rank = 0u;
        for (uint32_t j = lo; j < hi; ++j) rank += keys[j] > k[r] ? 1u : 0u;
        fin[r] = lo + rank;
      }
    }
  }
  __syncthreads();
  // (the last group of eight is filled up with empty entries)
  const float fmax = key_to_float(rmax);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (static_cast<uint32_t>(r * kFinishBlock) < n_pad) {
      const uint32_t pos = static_cast<uint32_t>(r * kFinishBlock + t);
      if (pos < n_pad) {
        const float e = em::expf_exact((key_to_float(key64_okey(k[r])) - fmax) * inv_temp);
        keys[exp_slot(fin[r])] = (static_cast<u64>(__float_as_uint(e)) << 32) | (k[r] & 0xffffffffull);
      }
    }
  }
  __syncthreads();
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
  if (row_mode(prm, V, a.chunks, a.emit_topk) != (LARGEK ? kModeTopkLarge : kModeNucleus)) return;
  if (!LARGEK && a.xf.mask && a.row_done && a.row_done[row] != 0u) return;  // finished by the sparse-mask kernel
  constexpr bool large_k = LARGEK;  // then every listed element is a candidate and no element after them is needed
  u64* big_row = a.big + static_cast<size_t>(row) * a.big_stride;
  const size_t cbase = static_cast<size_t>(row) * a.chunks;
  // The head of every chunk's list (a few entries per thread) is requested before the counts are
  // known -- whatever lies past a list's end is discarded later -- so that these loads overlap the
  // round trip for the counts.  Rows of more than kAheadChunks chunks, and rows whose lists hold more
  // than the sort has room for, read everything afterwards.
  constexpr int kGather = 8, kAheadChunks = 8, kHeadSlots = 16;  // kGather: entries a thread has in flight
  static_assert(kHeadSlots % kGather == 0 && kHeadSlots >= 2 * kAheadChunks, "the head is consumed in whole batches");
  // (the fewer chunks, the more of each list fits the head: slot q holds entry (q & (per - 1)) * kFinishBlock + tid
  // of chunk q >> head_shift, per = 1 << head_shift)
  const int head_shift = a.chunks <= 1 ? 4 : a.chunks <= 2 ? 3 : a.chunks <= 4 ? 2 : 1;
  u64 pre[kHeadSlots];
#pragma unroll
  for (int q = 0; q < kHeadSlots; ++q) {
    const int c = q >> head_shift, u = q & ((1 << head_shift) - 1);
    pre[q] = (a.chunks <= kAheadChunks && c < a.chunks) ? big_row[static_cast<size_t>(c) * kSChunk + u * kFinishBlock + tid] : 0;
  }
  for (int b = tid; b <= kSortBuckets; b += kFinishBlock) bucket_start[b] = 0u;  // the sort's table, while the loads are on their way
  // Lane c of every wave reads what chunk c left behind (at most 16 chunks), so the row's maximum and threshold
  // are reductions inside the wave, with no exchange between the waves; wave 0 publishes the counts and where
  // every list's rows begin, behind the one barrier that follows.
  __shared__ uint32_t sh_cnt[kAllCap / kSmallCap];       // candidates per chunk
  __shared__ uint32_t sh_first[kAllCap / kSmallCap + 1];  // rows of kFinishBlock entries the lists past their heads take, prefix sums
  __shared__ int sh_trim;
  __shared__ uint32_t sh_head, sh_all;
  static_assert(kAllCap / kSmallCap < 64, "a lane per chunk, and one more");
  const int lane = lane_id();
  uint32_t cnt = 0u, m = 0u, cthr = 0u;
  u64 best_below = 0;
  if (lane < a.chunks) {
    cnt = a.chunk_cnt[cbase + lane];
    m = cnt == kChunkCntOverflow ? 0xffffffffu : a.chunk_max[cbase + lane];  // above every key: the exact path
    cthr = a.chunk_thr[cbase + lane];
  }
  if (tid < a.chunks) {
    best_below = large_k ? 0 : a.chunk_next[cbase + tid];
    sh_cnt[tid] = cnt;
  }
  if (tid == 0) sh_count = 0u;
  const uint32_t rmax = wave_max<uint32_t>(m);
  const bool gave_up = rmax == 0xffffffffu;
  // Every chunk's threshold holds for the whole row (no element of the row below it lies strictly inside the
  // nucleus; a chunk alone has k elements at or above its own), so the highest one is the row's: every element at
  // or above it is in its chunk's list.
  uint32_t thr = wave_max<uint32_t>(cthr);
  if (rmax == 0u) thr = 0u;  // (no number in the row)
  if (tid < 64) {
    const uint32_t listed = gave_up ? 0u : cnt;
    const uint32_t all = wave_sum<uint32_t>(listed);
    const uint32_t head =
        (a.chunks <= kAheadChunks && all < static_cast<uint32_t>(kNucleusCap)) ? static_cast<uint32_t>(kFinishBlock) << head_shift : 0u;
    // (in rows of kFinishBlock entries: a row lies in one chunk's list, so its chunk is found once for all threads)
    const uint32_t rows = listed <= head ? 0u : (listed - head + kFinishBlock - 1u) / kFinishBlock;
    const uint32_t before = wave_prefix_sum<uint32_t>(rows) - rows;
    if (lane <= a.chunks) sh_first[lane] = before;  // (lane a.chunks: all of them)
    if (lane == 0) {
      sh_head = head;
      sh_all = all;
    }
  }
  __syncthreads();
  // The chunks' lists past their heads, as a sequence of rows of kFinishBlock entries (sh_first[c] = rows of the
  // chunks before c; a list's last row may be short).  A cursor walks the rows in order; which chunk a row lies in
  // is the same for every thread, so finding it costs the threads nothing.
  const uint32_t head = sh_head;
  struct ListCursor {
    int chunk = -1;
    uint32_t next_first = 0u, base = 0u, cnt = 0u;  // rows before the next chunk / before this one, entries of this one's list
  };
  // Loads the rows g0 .. g0 + n_slots - 1 (n_slots <= kGather, rows that exist) into raw[]; bit u of the result: the
  // thread has an entry in row g0 + u.
  auto load_rows = [&](ListCursor& cur, uint32_t g0, int n_slots, u64 (&raw)[kGather]) __attribute__((always_inline)) {
    uint32_t have = 0u;
#pragma unroll
    for (int u = 0; u < kGather; ++u) {
      raw[u] = 0;
      if (u < n_slots) {
        const uint32_t g = g0 + u;
        while (g >= cur.next_first) {  // (ends: g is below the rows of all chunks)
          ++cur.chunk;
          cur.base = cur.next_first;
          cur.next_first = __builtin_amdgcn_readfirstlane(sh_first[cur.chunk + 1]);
          cur.cnt = __builtin_amdgcn_readfirstlane(sh_cnt[cur.chunk]);
        }
        const uint32_t i = head + (g - cur.base) * kFinishBlock + tid;
        if (i < cur.cnt) {
          raw[u] = big_row[static_cast<size_t>(cur.chunk) * kSChunk + i];
          have |= 1u << u;
        }
      }
    }
    return have;
  };
  // Calls fn(entries, valid, used) for batches of kGather entries per thread (bit u of `used` clear: slot u is empty
  // in every thread) of that sequence.
  auto flat_batches = [&](auto fn) __attribute__((always_inline)) {
    const uint32_t total = sh_first[a.chunks];
    ListCursor cur;
    for (uint32_t g0 = 0; g0 < total; g0 += kGather) {
      u64 raw[kGather];
      bool valid[kGather];
      const int n_slots = total - g0 < static_cast<uint32_t>(kGather) ? static_cast<int>(total - g0) : kGather;
      const uint32_t have = load_rows(cur, g0, n_slots, raw);
#pragma unroll
      for (int u = 0; u < kGather; ++u) valid[u] = (have >> u) & 1u;
      fn(raw, valid, (1u << n_slots) - 1u);
    }
  };
  // More candidates listed than the sort holds (a flat distribution): the threshold is raised to the
  // lowest score that still leaves room, found from a histogram of the candidates over the sort's
  // score-linear buckets.  The nucleus test of the epilogue only looks at the elements it is given, in
  // rank order, and reports when they do not contain the nucleus; only then does the row need the
  // exact path.
  // The entries of the head (in registers) and then of the rest of the lists, in batches: fn(entries, valid, used),
  // bit u of `used` clear: no thread has an entry in slot u.
  auto listed_batches = [&](auto fn) __attribute__((always_inline)) {
    if (head != 0u) {
#pragma unroll
      for (int b = 0; b < kHeadSlots / kGather; ++b) {
        if ((b * kGather) >> head_shift < a.chunks) {
          u64 raw[kGather];
          bool valid[kGather];
          uint32_t used = 0u;
#pragma unroll
          for (int u = 0; u < kGather; ++u) {
            const int q = b * kGather + u, c = q >> head_shift;
            const uint32_t first = static_cast<uint32_t>(q & ((1 << head_shift) - 1)) * kFinishBlock;
            const uint32_t cnt = c < a.chunks ? __builtin_amdgcn_readfirstlane(sh_cnt[c < a.chunks ? c : 0]) : 0u;
            raw[u] = pre[q];
            valid[u] = first + tid < cnt;
            used |= first < cnt ? 1u << u : 0u;
          }
          fn(raw, valid, used);
        }
      }
    }
    flat_batches(fn);
  };
  // A nucleus row's usual way: a counting sort over the lists where they lie.  A first pass over them counts the
  // candidates (at or above the row's threshold) into the sort's buckets; the histogram tells how many buckets the
  // nucleus can reach at all (and how many fit the sort); a second pass gives every key of those buckets a place in
  // LDS.  However long the lists are, only what is kept has to fit.  A bucket with too many keys (heavy ties) leaves
  // the row to the steps below: the list in LDS, trimmed, and the sorting network.
  bool presorted = false, ok = false;
  // A row that goes the way of nuclei wider than the sort (decided after the first scan, done behind the usual
  // path's code; kept in LDS, not in registers, in between): the threads whose runs of buckets the nucleus needs (0: not such a
  // row), the entries of its list, and the best element below the candidates when it follows them.
  __shared__ uint32_t sh_wide_end_t, sh_wide_n;
  __shared__ u64 sh_wide_below;
  if (tid == 0) sh_wide_end_t = 0u;  // (barriers follow before it is looked at)
  bool wide = false, wide_ok = false;  // such a row / finished that way
  uint32_t n_c = 0u;
  const int k_wanted = large_k ? (prm.k < V ? prm.k : V) : 0;
  if (!gave_up && rmax != 0u) {
    const ScoreBuckets bucket_of(rmax, thr);  // (the table is zero: cleared at the start, barriers since)
    const float thr_score = key_to_float(thr);
    u64 below = best_below;
    listed_batches([&](const u64 (&raw)[kGather], const bool (&valid)[kGather], uint32_t used) {
#pragma unroll
      for (int u = 0; u < kGather; ++u) {
        if (((used >> u) & 1u) && valid[u]) {
          const float score = __uint_as_float(static_cast<uint32_t>(raw[u] >> 32));
          if (score >= thr_score) {  // (the same test as on order keys: false for NaN, true for either zero against a zero)
            atomicAdd(&bucket_start[bucket_of.of_score(score)], 1u);
          } else {
            const u64 k64 = (static_cast<u64>(order_key(score)) << 32) | (raw[u] & 0xffffffffull);
            below = k64 > below ? k64 : below;
          }
        }
      }
    });
    __syncthreads();
    TrimmedBuckets kept = scan_buckets_and_trim(bucket_start, bucket_of, below, prm, V, kNucleusCap, red32, red64, k_wanted);
    if constexpr (!LARGEK) {
      // The list ends with the one element below the candidates and has 16, 64, 256 ... entries: should the search
      // stop on that last element, the reference notices it one element later (src/sampling_distribution.h:166-181),
      // and that element is in no list.  Rare enough to look for it in the row itself: the best key below
      // best_below.  (Rows whose logits are processed on the way in would need that processing here: the exact path
      // keeps those.)
      const uint32_t n_list = kept.n;
      if (kept.best_below != 0 && n_list == kept.n_sorted + 1u && kept.more == 0u && n_list >= 16u && (n_list & (n_list - 1u)) == 0u &&
          ((__ffs(static_cast<int>(n_list)) - 1) & 1) == 0 && !a.xf.active()) {
        const RowPtr<AnyDtype> lrow(row_start<INLINE>(a, row, dtype_bytes(a.dtype)), a.dtype);
        u64 second = 0;
        for (int i = tid; i < V; i += kFinishBlock) {
          const u64 key = make_key64(order_key(lrow[i]), static_cast<uint32_t>(i));
          if (key < kept.best_below && key > second && key64_okey(key) != 0u) second = key;  // (order key 0: not a number)
        }
        second = block_max<u64>(second, red64);
        if (second != 0) {
          kept.second_below = second;
          kept.n = n_list + 1u;
        }
      }
      // The nucleus may need more keys than the sort has room for (a flat distribution, a high temperature), or a
      // bucket too full for the usual ranking.  The same sort then runs over the row's second key buffer in global
      // memory: every needed key goes to a place of its bucket's there, the buckets are ranked in rounds through LDS,
      // and the epilogue reads the list from there.  Still a fraction of the exact path's work: the histogram's bound
      // of the nucleus says which buckets are needed.  Decided here, done behind the usual path's code.  (Lists short enough
      // for the head in registers fit the room: there only a bucket too full gets here, and the steps below take
      // the row, as they do when a bucket is too full even for the rounds.)
      if (kept.more != 0u && head == 0u && a.big2 != nullptr) {
        constexpr int kPer = kSortBuckets / kFinishBlock;
        constexpr int kWideBucketCap = 256;  // (a key's rank costs a compare per key of its bucket)
        // back from first places to counts, and scanned again with room for everything: where the nucleus ends
        uint32_t s[kPer + 1];
#pragma unroll
        for (int i = 0; i <= kPer; ++i) s[i] = bucket_start[tid * kPer + i];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kPer; ++i) bucket_start[tid * kPer + i] = s[i + 1] - s[i];
        __syncthreads();
        const TrimmedBuckets all_kept = scan_buckets_and_trim(bucket_start, bucket_of, below, prm, V, 0x7fffffff, red32, red64, 0, kWideBucketCap);
        // (the table holds first places again; a row that does not go this way goes on as if nothing had happened)
        wide = all_kept.n != 0u && all_kept.more == 0u && static_cast<size_t>((all_kept.n + 7u) & ~7u) <= a.big_stride;
        if (wide && tid == 0) {
          sh_wide_end_t = all_kept.last_bucket < static_cast<uint32_t>(kSortBuckets) ? all_kept.last_bucket / kPer + 1u
                                                                                      : static_cast<uint32_t>(kFinishBlock);
          sh_wide_n = all_kept.n;
          sh_wide_below = all_kept.best_below;
        }
      }
    }
    if (!wide && kept.more != 2u && kept.n != 0u && kept.n_sorted >= static_cast<uint32_t>(k_wanted)) {  // (fewer than k numbers listed: the steps below decide)
      listed_batches([&](const u64 (&raw)[kGather], const bool (&valid)[kGather], uint32_t used) {
#pragma unroll
        for (int u = 0; u < kGather; ++u) {
          if (((used >> u) & 1u) && valid[u]) {
            const float score = __uint_as_float(static_cast<uint32_t>(raw[u] >> 32));
            if (score >= thr_score) {
              const uint32_t b = bucket_of.of_score(score);
              if (b <= kept.last_bucket)
                lds_keys[atomicAdd(&bucket_start[b], 1u)] = (static_cast<u64>(order_key(score)) << 32) | (raw[u] & 0xffffffffull);
            }
          }
        }
      });
      __syncthreads();
      rank_and_cache_exps<true>(lds_keys, bucket_start, bucket_of, kept, rmax, 1.0f / prm.temperature);
      presorted = ok = true;
      n_c = kept.n;
    }
  }
  if constexpr (!LARGEK) {
    __syncthreads();
    const uint32_t wide_end_t = sh_wide_end_t;
    if (wide_end_t != 0u) {  // (decided after the first scan; the table holds the buckets' first places)
      const uint32_t wide_n = sh_wide_n;
      const u64 wide_below = sh_wide_below;
      constexpr int kPer = kSortBuckets / kFinishBlock;
      u64* const far = a.big2 + static_cast<size_t>(row) * a.big_stride;
      const ScoreBuckets bucket_of(rmax, thr);
      const float thr_score = key_to_float(thr);
      const float fmax = key_to_float(rmax), inv_temp = 1.0f / prm.temperature;
      bool in_rounds = true;
      {
        // One more pass over the lists gives every key of the needed buckets a place of its bucket's in the global
        // buffer (the atomics of a batch are issued together).
        const uint32_t end_b = wide_end_t * kPer;
        flat_batches([&](const u64 (&raw)[kGather], const bool (&valid)[kGather], uint32_t) {
          uint32_t bucket[kGather], place[kGather];
#pragma unroll
          for (int u = 0; u < kGather; ++u) {
            const float score = __uint_as_float(static_cast<uint32_t>(raw[u] >> 32));
            const uint32_t b = bucket_of.of_score(score);
            bucket[u] = (valid[u] && score >= thr_score && b < end_b) ? b : 0xffffffffu;
          }
#pragma unroll
          for (int u = 0; u < kGather; ++u)
            if (bucket[u] != 0xffffffffu) place[u] = atomicAdd(&bucket_start[bucket[u]], 1u);
#pragma unroll
          for (int u = 0; u < kGather; ++u) {
            if (bucket[u] != 0xffffffffu)
              far[place[u]] = (static_cast<u64>(order_key(__uint_as_float(static_cast<uint32_t>(raw[u] >> 32)))) << 32) | (raw[u] & 0xffffffffull);
          }
        });
        __syncthreads();
      }
      // (Placing has counted every bucket's first place up to the next one's: bucket b now lies between start[b - 1]
      // and start[b].)  The rounds: the next threads' runs of buckets that fit the room come to LDS as they lie, a
      // key's rank inside its bucket comes from comparing whole keys, and the entry -- the exponential cached in
      // it -- goes back to its final place.
      uint32_t first_t = 0u, done = 0u;
      while (in_rounds && first_t < wide_end_t) {
        const uint32_t run_end = bucket_start[(tid + 1) * kPer - 1];
        const bool over = static_cast<uint32_t>(tid) >= first_t && static_cast<uint32_t>(tid) < wide_end_t &&
                          run_end - done > static_cast<uint32_t>(kNucleusCap);
        const uint32_t first_over = block_max<uint32_t>(over ? static_cast<uint32_t>(kFinishBlock - tid) : 0u, red32);
        const uint32_t last_t = first_over != 0u ? static_cast<uint32_t>(kFinishBlock) - first_over : wide_end_t;
        if (last_t == first_t) {  // one thread's buckets alone do not fit
          in_rounds = false;
          break;
        }
        const uint32_t n_round = bucket_start[last_t * kPer - 1u] - done;
        constexpr int kPerThread = kNucleusCap / kFinishBlock;
        u64 mine[kPerThread];
#pragma unroll
        for (int r = 0; r < kPerThread; ++r) {
          const uint32_t pos = static_cast<uint32_t>(r * kFinishBlock + tid);
          mine[r] = pos < n_round ? far[done + pos] : 0;
        }
#pragma unroll
        for (int r = 0; r < kPerThread; ++r) lds_keys[r * kFinishBlock + tid] = mine[r];
        __syncthreads();
#pragma unroll 1
        for (int r = 0; r < kPerThread; ++r) {
          const uint32_t pos = static_cast<uint32_t>(r * kFinishBlock + tid);
          if (pos < n_round) {
            const u64 k = lds_keys[pos];
            const uint32_t b = bucket_of(key64_okey(k));
            const uint32_t lo = (b > 0u ? bucket_start[b - 1u] : 0u) - done, hi = bucket_start[b] - done;
            uint32_t rank = 0u, j = lo;
            for (; j + 4u <= hi; j += 4u) {  // (four reads under way at a time)
              const u64 k0 = lds_keys[j], k1 = lds_keys[j + 1u], k2 = lds_keys[j + 2u], k3 = lds_keys[j + 3u];
              rank += (k0 > k ? 1u : 0u) + (k1 > k ? 1u : 0u) + (k2 > k ? 1u : 0u) + (k3 > k ? 1u : 0u);
            }
            for (; j < hi; ++j) rank += lds_keys[j] > k ? 1u : 0u;
            const float e = em::expf_exact((key_to_float(key64_okey(k)) - fmax) * inv_temp);
            far[done + lo + rank] = (static_cast<u64>(__float_as_uint(e)) << 32) | (k & 0xffffffffull);
          }
        }
        __syncthreads();
        done += n_round;
        first_t = last_t;
      }
      if (in_rounds) {
        // the best element below the candidates follows them when every bucket was needed; empty entries fill the
        // last group of eight
        const uint32_t n_list = wide_n;
        if (static_cast<uint32_t>(tid) < ((n_list + 7u) & ~7u) - done) {
          u64 entry = 0;
          if (tid == 0 && done < n_list) {
            const float e = em::expf_exact((key_to_float(key64_okey(wide_below)) - fmax) * inv_temp);
            entry = (static_cast<u64>(__float_as_uint(e)) << 32) | (wide_below & 0xffffffffull);
          }
          far[done + tid] = entry;
        }
        __syncthreads();
        const u64* list = far;
        wide_ok = block_sample_epilogue<8>([=](int i) { return list[i]; },
                                           [=](int i) { return __uint_as_float(static_cast<uint32_t>(list[i] >> 32)); },
                                           static_cast<int>(n_list), V, prm, a.uniforms[row], row_outputs(a, row), seqsh, true);
      }
    }
  }
  if (!presorted && !wide) {
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
      flat_batches([&](const u64 (&raw)[kGather], const bool (&valid)[kGather], uint32_t) {
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
        uint32_t inc = wave_prefix_sum<uint32_t>(own);
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
    auto consume = [&](const u64 (&raw)[kGather], const bool (&valid)[kGather], uint32_t) {
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
    listed_batches(consume);
    best_below = block_max<u64>(best_below, red64);  // barriers inside also publish sh_count
    n_c = sh_count;
    ok = !gave_up && !trim_failed && n_c < kNucleusCap;  // room for the next-best element too
    if (large_k) thr = ~block_max<uint32_t>(~lowest, red32);  // the lowest candidate score: the sort scales its buckets by it
    if (ok && !large_k) trim_to_nucleus(lds_keys, bucket_start, n_c, best_below, rmax, thr, prm, V, red32, red64, &sh_count);
  }
  if (ok) {
    const bool emit = large_k && a.emit_topk == 1;
    EmitTopk target;  // (by value: a pointer to the kernel's arguments would put all of them on the stack)
    if (emit) target = EmitTopk{a.out_tokens + static_cast<size_t>(row) * prm.k, a.out_scores + static_cast<size_t>(row) * prm.k,
                                row_start<INLINE>(a, row, dtype_bytes(a.dtype)), a.dtype};
    ok = finish_candidates(lds_keys, bucket_start, n_c, presorted ? 0 : best_below, rmax, thr, false, prm, V,
                           emit ? 0.0 : a.uniforms[row], row_outputs(a, row), seqsh, red32, target, presorted);
  }
  if (!ok && !wide_ok) {
    __syncthreads();
    general_row<AnyDtype, SortWithTile>(a, row, row_start<INLINE>(a, row, dtype_bytes(a.dtype)), prm, big_row, seqsh,
                          SortWithTile{a.big2 ? a.big2 + static_cast<size_t>(row) * a.big_stride : nullptr, lds_keys, red32, red64});
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

// ---- nucleus rows under a sparse grammar mask ------------------------------------------------------------
// A row whose mask lets through fewer ids than the finish kernels can sort needs none of its masked logits:
// a masked id is lowest() whatever its logit was.  One workgroup per row enumerates the allowed ids from the
// mask words, gathers exactly those logits, adds the row's history ids with their processed values (the
// reference's order: mask, min-length, penalty, n-gram ban), applies the nucleus threshold and finishes the
// row like the finish kernel does.  The best element outside the candidates is the better of the best listed
// element below the threshold and the first masked id that is not in the history (every such id scores
// lowest()).  row_done[row] tells the streaming and finish kernels launched afterwards whether the row is
// finished (1) or theirs to do (0: the mask lets too many ids through, too many history ids, or the nucleus
// did not close inside the candidates).
constexpr int kSparseWords = 16;                              // mask words per thread: vocabularies up to 524288
constexpr int kSparseIds = kNucleusCap / kFinishBlock;        // gathered ids per thread
constexpr int kSparseExtraRegs = 2;                           // processed history ids a thread takes on as candidates
constexpr int kSparseExtras = kSparseExtraRegs * kFinishBlock;  // distinct history ids (their list uses the bucket table's LDS)
static_assert(2 * kSparseExtras <= kSortBuckets + 1, "the list of processed history ids fits the bucket table");

// A logit as the bits it is stored in (fp32: the word, 16-bit types: the half word), so that the loads of a gather
// are plain loads issued back to back whatever the type, and the value of such bits.
__device__ __forceinline__ uint32_t logit_bits(const void* row0, int dtype, uint32_t i) {
  return dtype == MI355X_F32 ? static_cast<const uint32_t*>(row0)[i] : static_cast<uint32_t>(static_cast<const uint16_t*>(row0)[i]);
}
__device__ __forceinline__ float logit_of_bits(uint32_t bits, int dtype) {
  if (dtype == MI355X_F16) return half_bits_to_float(static_cast<uint16_t>(bits));
  if (dtype == MI355X_BF16) return bf16_bits_to_float(static_cast<uint16_t>(bits));
  return __uint_as_float(bits);
}

constexpr int kSparseRegs = kSparseIds + kSparseExtraRegs;
// Slot u of the threads' registers holds elements at all (the same answer for every thread: whole slots are skipped):
// gathered ids fill the first kSparseIds slots thread by thread, processed history ids the slots after them.
__device__ __forceinline__ bool sparse_slot_used(int u, uint32_t n_gathered, uint32_t n_extra) {
  return u < kSparseIds ? static_cast<uint32_t>(u * kFinishBlock) < n_gathered
                        : static_cast<uint32_t>((u - kSparseIds) * kFinishBlock) < n_extra;
}
constexpr uint32_t kSparseDirectMin = 2 * kFinishBlock;  // shorter lists take the general tail (a sorting network)

// The bucket sort of a row whose elements the block's threads hold in registers (ids[u] with the order key ok[u] of
// its score; 0xffffffff: no element; n_gathered / n_extra as for sparse_slot_used): counted slot by slot, then
// scanned, placed and ranked.
constexpr uint32_t kGatheredIdBits = 20, kGatheredIdMask = (1u << kGatheredIdBits) - 1u, kGatheredIsCand = 1u << 31;
static_assert(kFinishBlock * kSparseWords * 32 <= (1 << kGatheredIdBits) && kBucketCap < 255, "the packing of id and slot");

// Part one, for the slots U0 .. U1 - 1: a candidate (order key at or above thr) takes a slot in its bucket's count
// (`start`, kSortBuckets + 1 words, zero before the first call), which rides on its id from here on (ids stay below
// 1 << 20), with a mark; the others leave (id 0) after updating best_below, the thread's best element below the
// threshold.  Slots can be counted as soon as their values are there, while later ones are still on their way.
template <int U0, int U1>
__device__ __forceinline__ void count_gathered(uint32_t* start, uint32_t (&ids)[kSparseRegs], const uint32_t (&ok)[kSparseRegs],
                                               const ScoreBuckets& bucket_of, uint32_t thr, u64& best_below,
                                               uint32_t n_gathered, uint32_t n_extra) {
#pragma unroll
  for (int u = U0; u < U1; ++u) {
    if (!sparse_slot_used(u, n_gathered, n_extra)) {
      ids[u] = 0u;
      continue;
    }
    const bool have = ids[u] != 0xffffffffu;
    if (have && ok[u] >= thr) {
      const uint32_t slot = atomicAdd(&start[bucket_of(ok[u])], 1u);
      ids[u] |= kGatheredIsCand | ((slot < 255u ? slot : 255u) << kGatheredIdBits);
    } else {
      if (have) {
        const u64 k64 = make_key64(ok[u], ids[u]);
        best_below = k64 > best_below ? k64 : best_below;
      }
      ids[u] = 0u;
    }
  }
}

// Part two, once every slot is counted: scan and trimming, the places, ranks and exponentials.  Returns the number
// of sorted entries `keys` then holds, the way the epilogue reads them; 0: a bucket holds more than kBucketCap keys,
// nothing but `start` was written, the caller takes the general tail.  rmax: order key of the row's maximum;
// best_below: the thread's best element below the threshold (0: none).
__device__ __forceinline__ uint32_t sort_counted(u64* keys, uint32_t* start, const uint32_t (&ids)[kSparseRegs],
                                                 const uint32_t (&ok)[kSparseRegs], const ScoreBuckets& bucket_of, uint32_t rmax,
                                                 u64 best_below, uint32_t n_gathered, uint32_t n_extra, mi355x_sample_params prm,
                                                 int V, uint32_t* red32, u64* red64) {
  __syncthreads();
  const TrimmedBuckets kept = scan_buckets_and_trim(start, bucket_of, best_below, prm, V, kNucleusCap, red32, red64);
  if (kept.n == 0u || kept.more == 2u) return 0u;  // (a bucket too full to rank among those the row needs)
  // every kept key to its bucket, in the order of arrival
#pragma unroll
  for (int u = 0; u < kSparseRegs; ++u) {
    if (sparse_slot_used(u, n_gathered, n_extra) && (ids[u] & kGatheredIsCand)) {
      const uint32_t b = bucket_of(ok[u]);
      if (b <= kept.last_bucket) keys[start[b] + ((ids[u] >> kGatheredIdBits) & 255u)] = make_key64(ok[u], ids[u] & kGatheredIdMask);
    }
  }
  __syncthreads();
  rank_and_cache_exps<false>(keys, start, bucket_of, kept, rmax, 1.0f / prm.temperature);
  return kept.n;
}

// Returns 1 when the row is finished, 0 when it is not, -1 when it is not a nucleus row.
template <bool INLINE>
__device__ __forceinline__ int nucleus_sparse_body(const SampleArgs& a) {
  extern __shared__ u64 lds_keys[];
  uint32_t* const bucket_start = reinterpret_cast<uint32_t*>(lds_keys + kNucleusCap);
  uint32_t* const hist_bits = reinterpret_cast<uint32_t*>(lds_keys);                  // first half: history bitmap of the row
  constexpr int kStashWords = kNucleusCap / 2;  // rows of up to that many mask words also keep their allowed ids as bits there
  uint32_t* const allowed_bits = hist_bits + kStashWords;
  uint32_t* const id_list = reinterpret_cast<uint32_t*>(lds_keys + kNucleusCap / 2);  // second half: ids to gather
  float* const extra_val = reinterpret_cast<float*>(bucket_start);
  uint32_t* const extra_idx = bucket_start + kSparseExtras;
  __shared__ SeqShared seqsh;
  __shared__ uint32_t red32[16], red32_rest[16];  // (two: the reductions below follow each other without a barrier between)
  __shared__ u64 red64[16];
  __shared__ uint32_t sh_extra, sh_count;
  const int row = blockIdx.x, tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  const int V = a.vocab;
  const mi355x_sample_params prm = row_params<INLINE>(a, row);
  if (row_mode(prm, V, a.chunks) != kModeNucleus) return -1;
  const int words = (V - 1) / 32 + 1;
  const void* const row0 = row_start<INLINE>(a, row, dtype_bytes(a.dtype));
  // A row this kernel cannot finish is left to the dense kernels launched after it -- or, when the caller's
  // bound on the mask made this the only kernel, to the exact path (the caller of this function sees to that).
  auto leave = [&](bool done) { return done ? 1 : 0; };
  if (words > kFinishBlock * kSparseWords) return leave(false);
  const uint32_t* mrow = a.xf.mask + static_cast<size_t>(row) * words;
  const int n_eos = a.xf.eos_count(row);
  const bool pen = a.xf.use_penalty();
  // The gather of the allowed ids' logits is what takes the time, so it starts as early as it can: straight after
  // the mask words, with the history's ids still among the ids it fetches.  The history (ids, their logits and
  // mask words: dependent round trips to memory) is worked through while the gather is in flight; an id found in
  // it then leaves the gathered ones, its processed value joins as a candidate of its own.
  const int32_t* const h = pen ? a.xf.history + static_cast<size_t>(row) * a.xf.history_stride : nullptr;
  const int hlen = pen ? a.xf.hist_len(row) : 0;
  const int tok0 = (pen && tid < hlen) ? h[tid] : -1;
  // allowed ids of this thread's words: mask bits minus the EOS ids under min-length, nothing past the vocabulary
  uint32_t w[kSparseWords];
#pragma unroll
  for (int q = 0; q < kSparseWords; ++q) {
    const int wi = tid + q * kFinishBlock;
    uint32_t word = 0u;
    if (q * kFinishBlock < words) word = mrow[wi < words ? wi : 0];
    w[q] = wi < words ? word : 0u;
  }
  auto valid_bits = [&](int wi) {
    const int n_real = V - wi * 32;
    return wi >= words ? 0u : n_real >= 32 ? ~0u : ((1u << n_real) - 1u);
  };
  if (pen)
    for (int i = tid; i < words; i += kFinishBlock) hist_bits[i] = 0u;
  if (tid == 0) {
    sh_extra = 0u;
    sh_count = 0u;
  }
  uint32_t count = 0u;
#pragma unroll
  for (int q = 0; q < kSparseWords; ++q) {
    if (q * kFinishBlock < words) {
      const int wi = tid + q * kFinishBlock;
      uint32_t m = w[q];
      for (int e = 0; e < n_eos; ++e)
        if ((a.xf.eos[e] >> 5) == wi) m &= ~(1u << (a.xf.eos[e] & 31));
      w[q] = m & valid_bits(wi);
      count += static_cast<uint32_t>(__popc(w[q]));
    }
  }
  // (the thread's first history id has arrived with the mask words: its logit and mask word are requested now)
  const bool tok0_ok = tok0 >= 0 && tok0 < V;
  const uint32_t mw0 = tok0_ok ? mrow[tok0 >> 5] : 0u;
  const uint32_t raw0 = tok0_ok ? logit_bits(row0, a.dtype, static_cast<uint32_t>(tok0)) : 0u;
  const uint32_t inc = wave_prefix_sum<uint32_t>(count);
  if (lane == 63) red32[wave] = inc;
  __syncthreads();
  const uint32_t per_wave = wave_prefix_sum<uint32_t>(lane < kFinishBlock / 64 ? red32[lane] : 0u);
  const uint32_t n_allowed = wave_read_lane(per_wave, kFinishBlock / 64 - 1);
  const uint32_t wave_base = wave > 0 ? wave_read_lane(per_wave, wave - 1) : 0u;
  if (n_allowed + 2u > static_cast<uint32_t>(kNucleusCap)) return leave(false);
  uint32_t pos = wave_base + inc - count;
#pragma unroll
  for (int q = 0; q < kSparseWords; ++q) {
    if (q * kFinishBlock < words) {
      uint32_t m = w[q];
      const uint32_t base_id = static_cast<uint32_t>(tid + q * kFinishBlock) * 32u;
      if (words <= kStashWords && tid + q * kFinishBlock < words) allowed_bits[tid + q * kFinishBlock] = m;  // (for this thread)
      while (m != 0u) {
        id_list[pos++] = base_id + static_cast<uint32_t>(__ffs(m) - 1);
        m &= m - 1u;
      }
    }
  }
  __syncthreads();
  // gather: every load of a thread is requested before the first is used
  uint32_t ids[kSparseIds + kSparseExtraRegs];
  uint32_t ok[kSparseRegs];  // the bits of a gathered logit, then the order key of the score (0: not a number, or no element)
#pragma unroll
  for (int u = 0; u < kSparseIds; ++u) {
    const uint32_t i = static_cast<uint32_t>(tid + u * kFinishBlock);
    ids[u] = i < n_allowed ? id_list[i] : 0xffffffffu;
  }
  // (The element type is resolved once, outside the loads, so that they are plain loads issued back to back; slots
  // without an id load element 0, so that the number of loads in flight does not depend on the row.)
  auto gather_slots = [&](auto first, auto last) {
    if (a.dtype == MI355X_F32) {
#pragma unroll
      for (int u = decltype(first)::value; u < decltype(last)::value; ++u)
        ok[u] = static_cast<const uint32_t*>(row0)[ids[u] != 0xffffffffu ? ids[u] : 0u];
    } else {
#pragma unroll
      for (int u = decltype(first)::value; u < decltype(last)::value; ++u)
        ok[u] = static_cast<const uint16_t*>(row0)[ids[u] != 0xffffffffu ? ids[u] : 0u];
    }
  };
  // The first loads keep the memory system busy for longer than the history takes: the rest follows after it.  (All
  // at once would have every wave wait at its load instructions, the queues being full, and reach the history
  // only when the gather is nearly over.)
  constexpr int kFirstLoads = 6;
  // (What the history needs of the loads requested further up has long arrived; the wait for it stands here, ahead
  // of the gather: behind it the compiler, which cannot count requests made under conditions, would wait for the
  // gather's loads as well.)
  asm volatile("" ::"v"(mw0), "v"(raw0));
  gather_slots(std::integral_constant<int, 0>{}, std::integral_constant<int, kFirstLoads>{});
  asm volatile("" ::: "memory");
  // history ids: marked in a bitmap of the whole row; whoever marks an id first computes its processed value
  if (pen) {
    const RowPtr<AnyDtype> lrow(row0, a.dtype);
    const uint32_t* ban_row = a.xf.ban_row(row, V);
    for (int j = tid; j < hlen; j += kFinishBlock) {
      const bool ahead = j == tid;  // fetched above
      const int tok = ahead ? tok0 : h[j];
      if (tok < 0 || tok >= V) continue;
      const uint32_t bit = 1u << (tok & 31);
      if (atomicOr(&hist_bits[tok >> 5], bit) & bit) continue;
      const uint32_t slot = atomicAdd(&sh_extra, 1u);
      if (slot < static_cast<uint32_t>(kSparseExtras)) {
        extra_val[slot] = xform_value(ahead ? logit_of_bits(raw0, a.dtype) : lrow[tok], a.xf.penalty, a.xf.eos, tok,
                                      ahead ? mw0 : mrow[tok >> 5], true, true, n_eos, ban_row);
        extra_idx[slot] = static_cast<uint32_t>(tok);
      }
    }
  }
  __syncthreads();
  const uint32_t n_extra = sh_extra;
  if (n_allowed + n_extra + 2u > static_cast<uint32_t>(kNucleusCap) || n_extra > static_cast<uint32_t>(kSparseExtras) ||
      n_allowed + n_extra == 0u)
    return leave(false);
  // the gathered ids that are in the history leave; the first masked id outside the history
  uint32_t first_masked = 0xffffffffu;
  if (pen) {
#pragma unroll
    for (int u = 0; u < kSparseIds; ++u) {
      if (static_cast<uint32_t>(u * kFinishBlock) < n_allowed) {
        const uint32_t id = ids[u] != 0xffffffffu ? ids[u] : 0u;
        if ((hist_bits[id >> 5] >> (id & 31u)) & 1u) ids[u] = 0xffffffffu;
      }
    }
  }
#pragma unroll
  for (int q = 0; q < kSparseWords; ++q) {
    if (q * kFinishBlock < words) {
      const int wi = tid + q * kFinishBlock;
      const uint32_t hb = (pen && wi < words) ? hist_bits[wi] : 0u;
      uint32_t allowed = 0u;
      if (wi < words) {
        if (words <= kStashWords) {
          allowed = allowed_bits[wi];
        } else {  // (no room to keep them: the mask word once more, behind the gather)
          allowed = mrow[wi];
          for (int e = 0; e < n_eos; ++e)
            if ((a.xf.eos[e] >> 5) == wi) allowed &= ~(1u << (a.xf.eos[e] & 31));
        }
      }
      const uint32_t masked = ~allowed & valid_bits(wi) & ~hb;
      if (masked != 0u) {
        const uint32_t id = static_cast<uint32_t>(wi) * 32u + static_cast<uint32_t>(__ffs(masked) - 1);
        first_masked = id < first_masked ? id : first_masked;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kSparseExtraRegs; ++u) {
    const uint32_t i = static_cast<uint32_t>(tid + u * kFinishBlock);
    ids[kSparseIds + u] = i < n_extra ? extra_idx[i] : 0xffffffffu;
    ok[kSparseIds + u] = i < n_extra ? order_key(extra_val[i]) : 0u;
  }
  first_masked = ~block_max<uint32_t>(~first_masked, red32);  // (its barriers: every thread has read its extras)
  const bool direct = n_allowed + n_extra > kSparseDirectMin;
  if (direct)
    for (int b = tid; b <= kSortBuckets; b += kFinishBlock) bucket_start[b] = 0u;  // while the gather is in flight
  asm volatile("" ::: "memory");
  gather_slots(std::integral_constant<int, kFirstLoads>{}, std::integral_constant<int, kSparseIds>{});
  // The slots of the first loads and the processed history ids are there before the rest: their maximum stands in
  // for the row's where only a reference point is needed (the threshold below it, the buckets of the sort), so that
  // they are counted into their buckets while the other loads are still on their way.
  auto keys_of_slots = [&](auto first, auto last) {
    uint32_t kmax = 0u;
#pragma unroll
    for (int u = decltype(first)::value; u < decltype(last)::value; ++u) {
      const uint32_t bits = ok[u];
      ok[u] = 0u;
      if (sparse_slot_used(u, n_allowed, n_extra)) {
        ok[u] = ids[u] != 0xffffffffu ? order_key(logit_of_bits(bits, a.dtype)) : 0u;
        kmax = ok[u] > kmax ? ok[u] : kmax;
      }
    }
    return kmax;
  };
  uint32_t kmax = keys_of_slots(std::integral_constant<int, 0>{}, std::integral_constant<int, kFirstLoads>{});
#pragma unroll
  for (int u = kSparseIds; u < kSparseRegs; ++u) kmax = ok[u] > kmax ? ok[u] : kmax;
  const uint32_t rtop = block_max<uint32_t>(kmax, red32, false);  // (red32 is next written behind a later barrier)
  if (rtop == 0u) return leave(false);
  const uint32_t thr = order_key(key_to_float(rtop) - nucleus_depth(prm, V));
  if (thr <= order_key(kLowest)) return leave(false);  // masked ids would be candidates themselves
  u64 best_below = first_masked != 0xffffffffu ? make_key64(order_key(kLowest), first_masked) : 0;
  const ScoreBuckets bucket_of(rtop, thr);
  if (direct) {
    count_gathered<0, kFirstLoads>(bucket_start, ids, ok, bucket_of, thr, best_below, n_allowed, n_extra);
    count_gathered<kSparseIds, kSparseRegs>(bucket_start, ids, ok, bucket_of, thr, best_below, n_allowed, n_extra);
  }
  uint32_t rmax = rtop;
  if (static_cast<uint32_t>(kFirstLoads * kFinishBlock) < n_allowed) {
    const uint32_t rest = block_max<uint32_t>(keys_of_slots(std::integral_constant<int, kFirstLoads>{}, std::integral_constant<int, kSparseIds>{}), red32_rest, false);
    rmax = rest > rmax ? rest : rmax;
    if (direct) count_gathered<kFirstLoads, kSparseIds>(bucket_start, ids, ok, bucket_of, thr, best_below, n_allowed, n_extra);
  } else {
#pragma unroll
    for (int u = kFirstLoads; u < kSparseIds; ++u) {
      ok[u] = 0u;
      if (direct) ids[u] = 0u;
    }
  }
  uint32_t n_c = 0u;
  u64 second_below = 0;
  if (direct) {
    n_c = sort_counted(lds_keys, bucket_start, ids, ok, bucket_of, rmax, best_below, n_allowed, n_extra, prm, V, red32, red64);
    if (n_c == 0u) {  // heavy ties: the general tail, the candidates as they were
#pragma unroll
      for (int u = 0; u < kSparseRegs; ++u) ids[u] = (ids[u] >> 31) ? (ids[u] & kGatheredIdMask) : 0xffffffffu;
    }
  }
  const bool presorted = n_c != 0u;
  if (!presorted) {
    // candidates (at or above the threshold) go to the sort buffer at slots a wave reserves with one atomic per
    // batch; the best of the others is kept
#pragma unroll
    for (int u0 = 0; u0 < kSparseIds + kSparseExtraRegs; u0 += 6) {
      u64 hits[6];
      uint32_t wcnt = 0u;
#pragma unroll
      for (int u = u0; u < u0 + 6 && u < kSparseIds + kSparseExtraRegs; ++u) {
        const bool have = ids[u] != 0xffffffffu;
        const uint32_t ok32 = have ? ok[u] : 0u;
        const bool cand = have && ok32 >= thr;
        hits[u - u0] = __ballot(cand);
        wcnt += static_cast<uint32_t>(__popcll(hits[u - u0]));
        if (have && !cand) {
          const u64 k64 = make_key64(ok32, ids[u]);
          best_below = k64 > best_below ? k64 : best_below;
        }
      }
      uint32_t base = 0u;
      if (lane == 0 && wcnt != 0u) base = atomicAdd(&sh_count, wcnt);
      base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
      for (int u = u0; u < u0 + 6 && u < kSparseIds + kSparseExtraRegs; ++u) {
        const u64 b = hits[u - u0];
        const uint32_t p = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(b >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(b), base));
        if ((b >> lane) & 1ull) lds_keys[p] = make_key64(ok[u], ids[u]);
        base += static_cast<uint32_t>(__popcll(b));
      }
    }
    best_below = block_max<u64>(best_below, red64);  // barriers inside also publish sh_count
    n_c = sh_count;
    // A list that ends with best_below on its 16th, 64th, 256th ... entry: should the search stop on that entry, the
    // reference notices it one element later (src/sampling_distribution.h:166-181).  That element is the best key
    // below best_below among the elements that are no candidates and the masked ids; rows that came here straight
    // (the short lists: a few allowed ids under a grammar) still have every element in its thread's registers.
    const uint32_t n_list = n_c + 1u;
    if (!direct && best_below != 0 && n_list >= 16u && (n_list & (n_list - 1u)) == 0u && ((__ffs(static_cast<int>(n_list)) - 1) & 1) == 0) {
      u64 s = 0;
#pragma unroll
      for (int u = 0; u < kSparseIds + kSparseExtraRegs; ++u) {
        const u64 k64 = make_key64(ok[u], ids[u]);
        if (ids[u] != 0xffffffffu && ok[u] != 0u && ok[u] < thr && k64 < best_below && k64 > s) s = k64;
      }
      // The row's second masked id outside the history is wanted once in a long while: it is looked for here, behind
      // the first, a block of ids at a time (the row's list is short: nearly every id is masked, the first batch has it).
      uint32_t second_masked = 0xffffffffu;
      if (first_masked != 0xffffffffu) {
        for (uint32_t start = first_masked + 1u; start < static_cast<uint32_t>(V) && second_masked == 0xffffffffu;
             start += static_cast<uint32_t>(kFinishBlock)) {
          const uint32_t id = start + static_cast<uint32_t>(tid);
          bool is_masked = false;
          if (id < static_cast<uint32_t>(V)) {
            uint32_t m = mrow[id >> 5];
            for (int e = 0; e < n_eos; ++e)
              if (a.xf.eos[e] == static_cast<int>(id)) m &= ~(1u << (id & 31u));
            is_masked = ((m >> (id & 31u)) & 1u) == 0u;
            for (int j = 0; is_masked && j < hlen; ++j) is_masked = h[j] != static_cast<int>(id);
          }
          second_masked = ~block_max<uint32_t>(is_masked ? ~id : 0u, red32);
        }
      }
      const u64 km1 = make_key64(order_key(kLowest), first_masked), km2 = make_key64(order_key(kLowest), second_masked);
      if (first_masked != 0xffffffffu && km1 < best_below && km1 > s) s = km1;
      if (second_masked != 0xffffffffu && km2 < best_below && km2 > s) s = km2;
      second_below = block_max<u64>(s, red64);
    }
  }
  return leave(finish_candidates(lds_keys, bucket_start, n_c, presorted ? 0 : best_below, rmax, thr, false, prm, V, a.uniforms[row],
                                 row_outputs(a, row), seqsh, red32, EmitTopk{}, presorted, presorted ? 0 : second_below));
}

template <bool INLINE>
__device__ __forceinline__ void nucleus_sparse_entry(const SampleArgs& a) {
  int done = nucleus_sparse_body<INLINE>(a);
  if (done < 0) return;
  const int row = blockIdx.x;
  if (done == 0 && a.sparse_only) {  // no dense kernels follow: the exact path, here
    extern __shared__ u64 lds_keys[];
    __shared__ SeqShared exact_sh;
    __shared__ uint32_t exact_red32[16];
    __shared__ u64 exact_red64[16];
    __syncthreads();
    general_row<AnyDtype, SortWithTile>(a, row, row_start<INLINE>(a, row, dtype_bytes(a.dtype)), row_params<INLINE>(a, row),
                          a.big + static_cast<size_t>(row) * a.big_stride, exact_sh,
                          SortWithTile{a.big2 ? a.big2 + static_cast<size_t>(row) * a.big_stride : nullptr, lds_keys, exact_red32,
                                       exact_red64});
    done = 1;
  }
  if (threadIdx.x == 0) a.row_done[row] = static_cast<uint32_t>(done);
}

__global__ __launch_bounds__(kFinishBlock) void nucleus_sparse_kernel(const SampleArgs a) { nucleus_sparse_entry<false>(a); }
__global__ __launch_bounds__(kFinishBlock) void nucleus_sparse_rows_kernel(const SampleArgs a, const InlineParams) {
  nucleus_sparse_entry<true>(a);
}

// Rows whose parameters alone put them on the exact path (k above kLargeKMax, more chunks than a finishing
// workgroup ranks): one workgroup per row with the finish kernels' LDS, so that the row is sorted by the radix
// sort instead of a sorting network in global memory.
template <bool INLINE>
__device__ __forceinline__ void exact_rows_body(const SampleArgs& a) {
  extern __shared__ u64 lds_keys[];
  __shared__ SeqShared seqsh;
  __shared__ uint32_t red32[16];
  __shared__ u64 red64[16];
  const int row = blockIdx.x;
  const mi355x_sample_params prm = row_params<INLINE>(a, row);
  if (row_mode(prm, a.vocab, a.chunks, a.emit_topk) != kModeGeneral) return;
  general_row<AnyDtype, SortWithTile, 8>(a, row, row_start<INLINE>(a, row, dtype_bytes(a.dtype)), prm, a.big + static_cast<size_t>(row) * a.big_stride,
                        seqsh,
                        SortWithTile{a.big2 ? a.big2 + static_cast<size_t>(row) * a.big_stride : nullptr, lds_keys, red32, red64});
}
__global__ __launch_bounds__(kFinishBlock) void exact_rows_kernel(const SampleArgs a) { exact_rows_body<false>(a); }
__global__ __launch_bounds__(kFinishBlock) void exact_rows_rows_kernel(const SampleArgs a, const InlineParams) { exact_rows_body<true>(a); }

}  // namespace ms

MS_STREAM_KERNELS(, float)  // the fp32 streaming kernels live here, next to the finish kernels

extern "C" hipError_t ms_launch_sample(const ms::SampleArgs* a, const ms::InlineParams* table, bool any_other,
                                       bool any_nucleus, bool any_large_k, hipStream_t stream,
                                       const ms::SideStreams* sides) {
  const dim3 fgrid(a->rows), fblock(ms::kFinishBlock);
  auto launch_stream = a->dtype == MI355X_F16 ? ms_launch_stream_f16 : a->dtype == MI355X_BF16 ? ms_launch_stream_bf16 : ms_launch_stream;
  // A call whose rows are in several modes launches the kernels of every mode present; one after the other their
  // chains of dependent phases add up (12 + 42 + 39 us for top-k, nucleus and large-k rows in one batch of 64 x
  // 128256), side by side the longest decides.  The nucleus rows' kernels, the longest chain, stay on the caller's
  // stream.
  const int modes = (any_other ? 1 : 0) + (any_nucleus ? 1 : 0) + (any_large_k ? 1 : 0);
  const bool fork = sides != nullptr && modes > 1;
  int forked = 0;
  hipError_t e = hipSuccess;
  auto stream_of_mode = [&](bool stays) -> hipStream_t {
    if (!fork || stays) return stream;
    hipStream_t s = sides->side[forked++];
    if (e == hipSuccess) e = hipStreamWaitEvent(s, sides->fork, 0);
    return s;
  };
  if (fork) {
    e = hipEventRecord(sides->fork, stream);
    if (e != hipSuccess) return e;
  }
  if (any_other) {
    const hipStream_t s = stream_of_mode(!any_nucleus && !any_large_k);
    if (e == hipSuccess) e = launch_stream(a, table, 0, s);
  }
  if (any_large_k && e == hipSuccess) {
    const hipStream_t s = stream_of_mode(!any_nucleus);
    if (e == hipSuccess) e = launch_stream(a, table, 2, s);
    if (e == hipSuccess) {
      if (table) hipLaunchKernelGGL(ms::largek_finish_rows_kernel, fgrid, fblock, ms::kFinishLds, s, *a, *table);
      else hipLaunchKernelGGL(ms::largek_finish_kernel, fgrid, fblock, ms::kFinishLds, s, *a);
      e = hipGetLastError();
    }
  }
  if (any_nucleus && e == hipSuccess) {
    if (a->xf.mask && a->row_done) {  // rows under a sparse grammar mask are finished here; the next two kernels skip them
      if (table) hipLaunchKernelGGL(ms::nucleus_sparse_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a, *table);
      else hipLaunchKernelGGL(ms::nucleus_sparse_kernel, fgrid, fblock, ms::kFinishLds, stream, *a);
      e = hipGetLastError();
    }
    if (e == hipSuccess && !(a->xf.mask && a->row_done && a->sparse_only)) {
      e = launch_stream(a, table, 1, stream);
      if (e == hipSuccess) {
        if (table) hipLaunchKernelGGL(ms::nucleus_finish_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a, *table);
        else hipLaunchKernelGGL(ms::nucleus_finish_kernel, fgrid, fblock, ms::kFinishLds, stream, *a);
        e = hipGetLastError();
      }
    }
  }
  // (the forked streams join even after an error: a stream left forked would poison a capture)
  for (int i = 0; i < forked; ++i) {
    hipError_t j = hipEventRecord(sides->join[i], sides->side[i]);
    if (j == hipSuccess) j = hipStreamWaitEvent(stream, sides->join[i], 0);
    if (e == hipSuccess) e = j;
  }
  if (e != hipSuccess) return e;
  if (a->exact_kernel) {
    if (table) hipLaunchKernelGGL(ms::exact_rows_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a, *table);
    else hipLaunchKernelGGL(ms::exact_rows_kernel, fgrid, fblock, ms::kFinishLds, stream, *a);
    e = hipGetLastError();
  }
  return e;
}

extern "C" hipError_t ms_sample_init() {
  const void* finish[] = {reinterpret_cast<const void*>(ms::nucleus_finish_kernel),
                          reinterpret_cast<const void*>(ms::nucleus_finish_rows_kernel),
                          reinterpret_cast<const void*>(ms::largek_finish_kernel),
                          reinterpret_cast<const void*>(ms::largek_finish_rows_kernel),
                          reinterpret_cast<const void*>(ms::nucleus_sparse_kernel),
                          reinterpret_cast<const void*>(ms::nucleus_sparse_rows_kernel),
                          reinterpret_cast<const void*>(ms::exact_rows_kernel),
                          reinterpret_cast<const void*>(ms::exact_rows_rows_kernel)};
  for (const void* f : finish) {
    const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, ms::kFinishLds);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}
