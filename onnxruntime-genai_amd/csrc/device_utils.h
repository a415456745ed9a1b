// Device-side building blocks shared by the selection kernels: order-preserving keys, wave64
// reductions / sorts, the element loader with fused logits processing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "exact_math.h"
#include "mi355x_search.h"

namespace ms {

constexpr int kBlock = 256;            // threads per streaming workgroup (4 wave64)
constexpr int kElems = 32;             // logits held in registers per thread
constexpr int kChunk = kBlock * kElems;  // logits per streaming workgroup
constexpr float kLowest = -3.402823466e+38f;

typedef unsigned long long u64;

__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Larger key <=> larger score.  +-0 share a key, NaN maps to 0 (below -inf, whose key is 0x007fffff).
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  if (f != f) return 0u;
  if ((b << 1) == 0u) return 0x80000000u;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float key_to_float(uint32_t k) {
  if (k == 0u) return __uint_as_float(0x7fc00000u);
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// (score key, index) packed so that a plain unsigned max / descending sort yields
// "score descending, index ascending".  0 is the padding value (below every real element).
__device__ __forceinline__ u64 make_key64(uint32_t okey, uint32_t idx) {
  return (static_cast<u64>(okey) << 32) | static_cast<u64>(0xffffffffu - idx);
}
__device__ __forceinline__ uint32_t key64_index(u64 k) { return 0xffffffffu - static_cast<uint32_t>(k); }
__device__ __forceinline__ uint32_t key64_okey(u64 k) { return static_cast<uint32_t>(k >> 32); }

// ---- cross-lane helpers -------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T shfl_xor_t(T v, int mask) {
  return __shfl_xor(v, mask, 64);
}
template <>
__device__ __forceinline__ u64 shfl_xor_t<u64>(u64 v, int mask) {
  const uint32_t lo = __shfl_xor(static_cast<uint32_t>(v), mask, 64);
  const uint32_t hi = __shfl_xor(static_cast<uint32_t>(v >> 32), mask, 64);
  return (static_cast<u64>(hi) << 32) | lo;
}
template <typename T>
__device__ __forceinline__ T shfl_t(T v, int lane) {
  return __shfl(v, lane, 64);
}
template <>
__device__ __forceinline__ u64 shfl_t<u64>(u64 v, int lane) {
  const uint32_t lo = __shfl(static_cast<uint32_t>(v), lane, 64);
  const uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), lane, 64);
  return (static_cast<u64>(hi) << 32) | lo;
}

// The value `d` lanes below (row_shr inside a row of 16 lanes, then the row broadcasts), `old` where there is
// no such lane; 4- and 8-byte types.  These lane-shifting moves are register operations; the general lane
// shuffles (__shfl*) go through the LDS crossbar and take several times as long.
template <int CTRL, int ROW_MASK, typename T>
__device__ __forceinline__ T dpp_from_below_or(T old, T x) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit values");
  if constexpr (sizeof(T) == 4) {
    const uint32_t r = __builtin_amdgcn_update_dpp(__builtin_bit_cast(uint32_t, old), __builtin_bit_cast(uint32_t, x), CTRL,
                                                   ROW_MASK, 0xf, false);
    return __builtin_bit_cast(T, r);
  } else {
    const u64 o = __builtin_bit_cast(u64, old), b = __builtin_bit_cast(u64, x);
    const uint32_t lo = __builtin_amdgcn_update_dpp(static_cast<uint32_t>(o), static_cast<uint32_t>(b), CTRL, ROW_MASK, 0xf, false);
    const uint32_t hi = __builtin_amdgcn_update_dpp(static_cast<uint32_t>(o >> 32), static_cast<uint32_t>(b >> 32), CTRL,
                                                   ROW_MASK, 0xf, false);
    return __builtin_bit_cast(T, (static_cast<u64>(hi) << 32) | lo);
  }
}

// Value of x in lane l (l uniform over the wave).
template <typename T>
__device__ __forceinline__ T wave_read_lane(T x, int l) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit values");
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), l));
  } else {
    const u64 b = __builtin_bit_cast(u64, x);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(b)), l));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(b >> 32)), l));
    return __builtin_bit_cast(T, (static_cast<u64>(hi) << 32) | lo);
  }
}

// Reductions over the wave; every lane gets the result.  Six lane-shifting steps leave it in lane 63.
template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#define MS_STEP(CTRL, MASK)                                  \
  {                                                          \
    const T o = dpp_from_below_or<CTRL, MASK, T>(v, v);      \
    v = o > v ? o : v;                                       \
  }
  MS_STEP(0x111, 0xf) MS_STEP(0x112, 0xf) MS_STEP(0x114, 0xf) MS_STEP(0x118, 0xf) MS_STEP(0x142, 0xa) MS_STEP(0x143, 0xc)
#undef MS_STEP
  return wave_read_lane(v, 63);
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
  const T zero = T(0);
  v += dpp_from_below_or<0x111, 0xf, T>(zero, v);  // row_shr:1
  v += dpp_from_below_or<0x112, 0xf, T>(zero, v);  // row_shr:2
  v += dpp_from_below_or<0x114, 0xf, T>(zero, v);  // row_shr:4
  v += dpp_from_below_or<0x118, 0xf, T>(zero, v);  // row_shr:8
  v += dpp_from_below_or<0x142, 0xa, T>(zero, v);  // row_bcast:15 into rows 1 and 3
  v += dpp_from_below_or<0x143, 0xc, T>(zero, v);  // row_bcast:31 into rows 2 and 3
  return wave_read_lane(v, 63);
}

// Inclusive prefix sums over the wave (tree order).
template <typename T>
__device__ __forceinline__ T wave_prefix_sum(T v) {
  const T zero = T(0);
  v += dpp_from_below_or<0x111, 0xf, T>(zero, v);  // row_shr:1
  v += dpp_from_below_or<0x112, 0xf, T>(zero, v);  // row_shr:2
  v += dpp_from_below_or<0x114, 0xf, T>(zero, v);  // row_shr:4
  v += dpp_from_below_or<0x118, 0xf, T>(zero, v);  // row_shr:8
  v += dpp_from_below_or<0x142, 0xa, T>(zero, v);  // row_bcast:15 into rows 1 and 3
  v += dpp_from_below_or<0x143, 0xc, T>(zero, v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Bitonic sort of one value per lane, descending by lane index (lane 0 ends with the maximum).
template <typename T>
__device__ __forceinline__ T wave_sort_desc(T x) {
  const int lane = lane_id();
#pragma unroll
  for (int k = 2; k <= 64; k <<= 1) {
#pragma unroll
    for (int j = k >> 1; j > 0; j >>= 1) {
      const T y = shfl_xor_t<T>(x, j);
      const bool desc_block = (lane & k) == 0;
      const bool lower = (lane & j) == 0;
      const T mx = x > y ? x : y;
      const T mn = x > y ? y : x;
      x = (lower == desc_block) ? mx : mn;
    }
  }
  return x;
}

// Maximum over the first sixteen lanes (four lane-shifting steps inside the row); every lane gets the result.
template <typename T>
__device__ __forceinline__ T row16_max(T v) {
#define MS_STEP(CTRL)                                        \
  {                                                          \
    const T o = dpp_from_below_or<CTRL, 0xf, T>(v, v);       \
    v = o > v ? o : v;                                       \
  }
  MS_STEP(0x111) MS_STEP(0x112) MS_STEP(0x114) MS_STEP(0x118)
#undef MS_STEP
  return wave_read_lane(v, 15);
}

// Block-wide maximum of unsigned values; every thread gets the result.  `scratch` holds >= blockDim/64 entries
// (at most sixteen waves).  Two barriers: the second one lets the caller write `scratch` again at once; a caller
// that leaves it alone until its next barrier passes reuse_at_once = false and saves it.
template <typename T>
__device__ __forceinline__ T block_max(T v, T* scratch, bool reuse_at_once = true) {
  v = wave_max(v);
  const int lane = lane_id(), wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  const T r = row16_max<T>(lane < nw ? scratch[lane] : T(0));  // lane w looks at wave w's
  if (reuse_at_once) __syncthreads();
  return r;
}

// A key tau such that at least k of the keys offered by the block's threads are >= tau
// (1 <= k <= 64; threads without an element offer 0).  Each wave sorts its 64 keys, the best
// 64/waves of every wave are pooled and sorted again; the k-th best of that pool is a valid bound
// and equals the block's true k-th best unless one wave holds more than its share of the top k.
// blockDim.x must be 256 (4 waves).  `pool` holds 64 entries.
__device__ __forceinline__ uint32_t block_kth_bound(uint32_t key, int k, uint32_t* pool) {
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const uint32_t sorted = wave_sort_desc<uint32_t>(key);
  if (lane < 16) pool[wave * 16 + lane] = sorted;
  __syncthreads();
  uint32_t v = pool[lane];
  v = wave_sort_desc<uint32_t>(v);
  const uint32_t tau = shfl_t<uint32_t>(v, k - 1);
  __syncthreads();
  return tau;
}

// Loads with agent-scope coherence, for data another workgroup of the same launch wrote.
__device__ __forceinline__ u64 load_coherent(const u64* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t load_coherent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- fp16 widening ------------------------------------------------------------------------------
// Same value as the reference's FastFloat16ToFloat32 (src/models/utils.cpp:103-109): IEEE for zeros,
// subnormals and normals; an exponent field of 31 (Inf/NaN in IEEE) is decoded as an ordinary
// exponent, giving +-65536*(1+m/1024).
__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  const uint32_t sign = (h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu;
  const uint32_t m = h & 0x3ffu;
  if (e != 0u) return __uint_as_float(sign | ((e + 112u) << 23) | (m << 13));
  // subnormal or zero: m * 2^-24, exact in fp32
  const float mag = static_cast<float>(m) * 5.9604644775390625e-08f;
  return __uint_as_float(sign | __float_as_uint(mag));
}

// Eight fp16 values in a 16-byte vector, widened as above.  The hardware conversion is exact for zeros,
// subnormals and normals; the rare vector that holds an exponent field of 31 is redone by the bit formula.
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void widen_half8(v4u q, float* o) {
  const uint32_t w[4] = {q.x, q.y, q.z, q.w};
  uint32_t suspicious = 0u;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    o[2 * c] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w[c] & 0xffffu)));
    o[2 * c + 1] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w[c] >> 16)));
    suspicious |= ((w[c] & 0x7c007c00u) + 0x04000400u) & 0x80008000u;  // a half whose exponent bits are all ones
  }
  if (__builtin_expect(suspicious != 0u, 0)) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      o[2 * c] = half_bits_to_float(w[c] & 0xffffu);
      o[2 * c + 1] = half_bits_to_float(w[c] >> 16);
    }
  }
}

// bfloat16 -> fp32 as BFloat16ToFloat32 does (src/models/utils.cpp:84-86 via :55-77): the bits moved to
// the upper half, except that every NaN becomes the canonical quiet NaN.
__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) {
  if ((h & 0x7f80u) == 0x7f80u && (h & 0x7fu) != 0u) return __uint_as_float(0x7fc00000u);
  return __uint_as_float(h << 16);
}

struct bf16_t {  // a bfloat16 bit pattern (uint16_t stands for IEEE binary16 throughout)
  uint16_t bits;
};
// One 16-bit element as fp32: binary16 for uint16_t, bfloat16 for bf16_t.
template <typename InT>
__device__ __forceinline__ float narrow_bits_to_float(uint32_t bits) {
  if constexpr (sizeof(InT) == sizeof(bf16_t) && !__is_same(InT, uint16_t)) return bf16_bits_to_float(bits);
  else return half_bits_to_float(bits);
}
// Eight bfloat16 values in a 16-byte vector.  NaNs keep their payload here (the canonical quiet NaN of
// bf16_bits_to_float is only needed where a value is written out): selection only asks whether a value is a NaN.
__device__ __forceinline__ void widen_bf16x8(v4u q, float* o) {
  const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    o[2 * c] = __uint_as_float(w[c] << 16);
    o[2 * c + 1] = __uint_as_float(w[c] & 0xffff0000u);
  }
}

// fp32 -> fp16 with FastFloat32ToFloat16's arithmetic (src/models/utils.cpp:111-118): the rounding
// bit is added before the fields are split, values beyond the fp16 range saturate to 0x7FFF.
__device__ __forceinline__ uint32_t float_to_half_bits(float v) {
  const uint32_t b = __float_as_uint(v) + 0x00001000u;
  const uint32_t e = (b & 0x7F800000u) >> 23;
  const uint32_t m = b & 0x007FFFFFu;
  uint32_t r = (b & 0x80000000u) >> 16;
  if (e > 112u) r |= (((e - 112u) << 10) & 0x7C00u) | (m >> 13);
  if (e < 113u && e > 101u) r |= (((0x007FF000u + m) >> (125u - e)) + 1u) >> 1;
  if (e > 143u) r |= 0x7FFFu;
  return r & 0xffffu;
}

// ---- fused logits processing --------------------------------------------------------------------
struct Xform {
  const uint32_t* mask;
  const int32_t* history;
  int history_stride;
  int history_len;
  float penalty;
  int n_eos;  // 0 unless min-length masking is active
  int eos[MI355X_MAX_EOS];
  const int32_t* history_lens;  // per-row number of valid history ids, or null (history_len for every row)
  int min_length;               // with history_lens: only rows shorter than this get the EOS masking
  const uint32_t* ban;          // per-row bitmap (mask layout) of ids the no-repeat-n-gram rule bans, or null
  __host__ __device__ __forceinline__ bool active() const { return mask || use_penalty() || n_eos > 0; }
  // true when elements must be tested against the row's history: a penalty to apply or banned ids to
  // look up (a banned id always occurs in the history; a penalty of 1.0f leaves a value unchanged)
  __host__ __device__ __forceinline__ bool use_penalty() const {
    return history && (history_lens || history_len > 0) && (penalty != 1.0f || ban);
  }
  // (The common length passes through a register before the branch: as a plain `lens ? lens[row] : len` the compiler
  // loads through a selected pointer, which for the common length is a round trip to the kernel arguments in memory
  // and, being a load that may go anywhere, makes every wait behind it a wait for all loads.)
  __device__ __forceinline__ int hist_len(int row) const {
    int n = history_len;
    asm volatile("" : "+s"(n));
    if (history_lens) n = history_lens[row];
    return n;
  }
  __device__ __forceinline__ int eos_count(int row) const {
    return (history_lens && min_length > 0 && history_lens[row] >= min_length) ? 0 : n_eos;
  }
  __device__ __forceinline__ const uint32_t* ban_row(int row, int vocab) const {
    return ban ? ban + static_cast<size_t>(row) * ((vocab - 1) / 32 + 1) : nullptr;
  }
};

// Kernel arguments live in memory and are read with scalar loads of a few hundred cycles each.  Left to
// the compiler, each is fetched where it is first needed, one wait after the other, which shows in
// latency-bound kernels.  arg_now() makes the value exist at the point of the call, so that a group of
// calls puts all those loads in flight together.
template <typename T>
__device__ __forceinline__ T arg_now(T x) {
  asm volatile("" : "+s"(x));
  return x;
}

// Marks, in an LDS bitmap covering vocabulary ids [base, base + kChunk), the ids present in the
// row's history.  bits: kChunk/32 words.  Ends with a barrier.
__device__ __forceinline__ void build_history_bitmap(const Xform& xf, int row, int base, uint32_t* bits) {
  for (int i = threadIdx.x; i < kChunk / 32; i += blockDim.x) bits[i] = 0u;
  __syncthreads();
  const int32_t* h = xf.history + static_cast<size_t>(row) * xf.history_stride;
  const int hlen = xf.hist_len(row);
  for (int i = threadIdx.x; i < hlen; i += blockDim.x) {
    const int rel = h[i] - base;
    if (rel >= 0 && rel < kChunk) atomicOr(&bits[rel >> 5], 1u << (rel & 31));
  }
  __syncthreads();
}

// The reference's order: mask -> min-length -> repetition penalty -> no-repeat-n-gram ban
// (src/standard_decoding_strategy.cpp:24-32, src/sampling_distribution.h:100-110).  n_eos and
// ban_row are the row's values (Xform::eos_count, Xform::ban_row).
__device__ __forceinline__ float xform_value(float x, float penalty, const int* eos, int idx, uint32_t mask_word,
                                             bool has_mask, bool in_history, int n_eos, const uint32_t* ban_row) {
  if (has_mask && !((mask_word >> (idx & 31)) & 1u)) x = kLowest;
  for (int e = 0; e < n_eos; ++e)
    if (eos[e] == idx) x = kLowest;
  if (in_history) {
    x = x < 0.0f ? x * penalty : x / penalty;
    if (ban_row && ((ban_row[idx >> 5] >> (idx & 31)) & 1u)) x = kLowest;
  }
  return x;
}

// 128-bit vectors that assume no more than their elements' alignment.  The hardware reads them from any address, so
// rows that do not start on a 16-byte boundary (odd vocabularies such as 50257, views into larger buffers) are read
// with the same loads as aligned rows; they only touch more cache lines.
typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t v4u_any __attribute__((ext_vector_type(4), aligned(2)));

// Loads the kElems logits a thread owns in chunk `chunk` of a row, widened to fp32 and processed.
// Thread t owns, for j = 0..NV-1, the VEC consecutive ids starting at
// chunk*kChunk + (j*kBlock + t)*VEC; ids >= vocab yield 0 and must be ignored by the caller.
template <typename InT>
struct Loader;

template <>
struct Loader<float> {
  static constexpr int VEC = 4;
  static constexpr int NV = kElems / VEC;
  __device__ static __forceinline__ int index_of(int chunk, int j, int c) {
    return chunk * kChunk + (j * kBlock + static_cast<int>(threadIdx.x)) * VEC + c;
  }
  __device__ static __forceinline__ void load(const float* row, int vocab, int chunk, float (&v)[kElems]) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i0 = index_of(chunk, j, 0);
      if (i0 + VEC <= vocab) {
        const v4f_any q = *reinterpret_cast<const v4f_any*>(row + i0);
        v[j * 4 + 0] = q.x;
        v[j * 4 + 1] = q.y;
        v[j * 4 + 2] = q.z;
        v[j * 4 + 3] = q.w;
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[j * 4 + c] = (i0 + c < vocab) ? row[i0 + c] : 0.0f;
      }
    }
  }
};

template <typename T16>
struct Loader16 {  // sixteen-bit elements: IEEE binary16 bit patterns (uint16_t) or bfloat16 (bf16_t)
  static constexpr int VEC = 8;
  static constexpr int NV = kElems / VEC;
  __device__ static __forceinline__ int index_of(int chunk, int j, int c) {
    return chunk * kChunk + (j * kBlock + static_cast<int>(threadIdx.x)) * VEC + c;
  }
  __device__ static __forceinline__ void load(const T16* row, int vocab, int chunk, float (&v)[kElems]) {
    const uint16_t* const bits = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i0 = index_of(chunk, j, 0);
      if (i0 + VEC <= vocab) {
        const v4u_any q = *reinterpret_cast<const v4u_any*>(bits + i0);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          v[j * 8 + 2 * c] = narrow_bits_to_float<T16>(w[c] & 0xffffu);
          v[j * 8 + 2 * c + 1] = narrow_bits_to_float<T16>(w[c] >> 16);
        }
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[j * 8 + c] = (i0 + c < vocab) ? narrow_bits_to_float<T16>(bits[i0 + c]) : 0.0f;
      }
    }
  }
};
template <>
struct Loader<uint16_t> : Loader16<uint16_t> {};
template <>
struct Loader<bf16_t> : Loader16<bf16_t> {};

// Applies the logits processing to the registers loaded by Loader<InT>::load.
template <typename InT>
__device__ __forceinline__ void xform_chunk(const Xform& xf, int row, int vocab, int chunk,
                                            const uint32_t* hist_bits, float (&v)[kElems]) {
  using L = Loader<InT>;
  const bool has_mask = xf.mask != nullptr;
  const bool pen = xf.use_penalty();
  const uint32_t* mrow = has_mask ? xf.mask + static_cast<size_t>(row) * ((vocab - 1) / 32 + 1) : nullptr;
  const int n_eos = xf.eos_count(row);
  const uint32_t* ban_row = xf.ban_row(row, vocab);
#pragma unroll
  for (int j = 0; j < L::NV; ++j) {
#pragma unroll
    for (int c = 0; c < L::VEC; ++c) {
      const int idx = L::index_of(chunk, j, c);
      if (idx < vocab) {
        const uint32_t mw = has_mask ? mrow[idx >> 5] : 0u;
        const int rel = idx - chunk * kChunk;
        const bool hit = pen && ((hist_bits[rel >> 5] >> (rel & 31)) & 1u);
        v[j * L::VEC + c] = xform_value(v[j * L::VEC + c], xf.penalty, xf.eos, idx, mw, has_mask, hit, n_eos, ban_row);
      }
    }
  }
}

// Single-element version for code that revisits a row outside the streaming layout.
template <typename InT>
__device__ __forceinline__ float load_one(const InT* row, int idx);
template <>
__device__ __forceinline__ float load_one<float>(const float* row, int idx) { return row[idx]; }
template <>
__device__ __forceinline__ float load_one<uint16_t>(const uint16_t* row, int idx) {
  return half_bits_to_float(row[idx]);
}
template <>
__device__ __forceinline__ float load_one<bf16_t>(const bf16_t* row, int idx) {
  return bf16_bits_to_float(row[idx].bits);
}

}  // namespace ms
