// Wave64 selection primitives: lane exchanges without LDS traffic, an in-register bitonic sort,
// k-th-largest by bisection, wave-aggregated slot allocation and the pooled block bound.
#pragma once
#include "device_utils.h"

namespace ms {

// ---- lane exchange primitives ---------------------------------------------------------------------
template <int M>
__device__ __forceinline__ uint32_t lane_xor(uint32_t x) {
  if constexpr (M == 1) {
    return __builtin_amdgcn_mov_dpp(x, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  } else if constexpr (M == 2) {
    return __builtin_amdgcn_mov_dpp(x, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  } else if constexpr (M == 4) {
    // banks of four lanes: even banks read four lanes up (row_shl:4), odd banks four lanes down
    const uint32_t t = __builtin_amdgcn_update_dpp(x, x, 0x104, 0xf, 0x5, false);
    return __builtin_amdgcn_update_dpp(t, x, 0x114, 0xf, 0xa, false);
  } else if constexpr (M == 8) {
    return __builtin_amdgcn_mov_dpp(x, 0x128, 0xf, 0xf, true);  // row_ror:8 == xor 8 inside a row of 16
  } else if constexpr (M == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    return (lane_id() & 16) ? r[0] : r[1];
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return (lane_id() & 32) ? r[0] : r[1];
  }
}

template <int M>
__device__ __forceinline__ u64 lane_xor64(u64 x) {
  const uint32_t lo = lane_xor<M>(static_cast<uint32_t>(x));
  const uint32_t hi = lane_xor<M>(static_cast<uint32_t>(x >> 32));
  return (static_cast<u64>(hi) << 32) | lo;
}
__device__ __forceinline__ uint32_t lane_xor_any(uint32_t x, int m) { return __shfl_xor(x, m, 64); }

// The pair (own key, key of the lane J away) of a compare-exchange step on 32-bit keys, in an order that suits the
// hardware: the two results of a permlane swap already are the pair's two members in every lane.
template <int J>
__device__ __forceinline__ void lane_pair(uint32_t x, uint32_t& a, uint32_t& b) {
  if constexpr (J == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    a = r[0];
    b = r[1];
  } else if constexpr (J == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    a = r[0];
    b = r[1];
  } else {
    a = x;
    b = lane_xor<J>(x);
  }
}

template <int K, int J, typename T>
__device__ __forceinline__ void sort_merge(T& x, int lane) {
  const bool keep_max = (((lane & K) == 0) == ((lane & J) == 0));
  if constexpr (sizeof(T) == 8) {
    const T y = lane_xor64<J>(x);
    x = ((y > x) == keep_max) ? y : x;
  } else {
    // maximum and minimum of the pair (the lane exchange folds into both instructions as a DPP operand), then
    // one select on a lane mask that does not depend on the data
    uint32_t a, b;
    lane_pair<J>(x, a, b);
    const uint32_t mx = a > b ? a : b, mn = a > b ? b : a;
    x = keep_max ? mx : mn;
  }
  if constexpr (J > 1) sort_merge<K, J / 2, T>(x, lane);
}

// The two members of the pair (lane, lane ^ J) of a compare-exchange step on 64-bit keys: lo = the key of the lane
// whose bit J is clear, hi = the other one, both in both lanes.  For J = 16 and 32 the two results of a permlane
// swap are exactly that; for the shorter distances a lane reads its partner and sorts out which is which.
template <int J>
__device__ __forceinline__ void lane_pair64(u64 x, int lane, u64& lo, u64& hi) {
  const uint32_t x0 = static_cast<uint32_t>(x), x1 = static_cast<uint32_t>(x >> 32);
  if constexpr (J == 16) {
    const auto r0 = __builtin_amdgcn_permlane16_swap(x0, x0, false, false);
    const auto r1 = __builtin_amdgcn_permlane16_swap(x1, x1, false, false);
    lo = (static_cast<u64>(r1[0]) << 32) | r0[0];
    hi = (static_cast<u64>(r1[1]) << 32) | r0[1];
  } else if constexpr (J == 32) {
    const auto r0 = __builtin_amdgcn_permlane32_swap(x0, x0, false, false);
    const auto r1 = __builtin_amdgcn_permlane32_swap(x1, x1, false, false);
    lo = (static_cast<u64>(r1[0]) << 32) | r0[0];
    hi = (static_cast<u64>(r1[1]) << 32) | r0[1];
  } else {
    const u64 y = lane_xor64<J>(x);
    const bool upper = (lane & J) != 0;
    lo = upper ? y : x;
    hi = upper ? x : y;
  }
}

// Bitonic merge of a bitonic sequence held one key per lane: the result is sorted by lane, descending,
// or ascending if ASC.
template <int J, bool ASC, typename T>
__device__ __forceinline__ void bitonic_merge(T& x, int lane) {
  if constexpr (sizeof(T) == 8 && J >= 16) {
    u64 lo, hi;
    lane_pair64<J>(x, lane, lo, hi);
    const bool upper = (lane & J) != 0;
    x = ((hi > lo) != (upper != ASC)) ? hi : lo;  // descending: the lower lane keeps the larger key
  } else {
    T y;
    if constexpr (sizeof(T) == 8) y = lane_xor64<J>(x);
    else y = lane_xor<J>(x);
    const bool keep_max = ((lane & J) == 0) != ASC;
    x = ((y > x) == keep_max) ? y : x;
  }
  if constexpr (J > 1) bitonic_merge<J / 2, ASC, T>(x, lane);
}

// The same for two independent sequences at once, a descending and b ascending: the two dependent chains
// are written step by step side by side, so that the instructions of one fill the waits of the other.
template <int J>
__device__ __forceinline__ void bitonic_merge_two(u64& a, u64& b, int lane) {
  const bool upper = (lane & J) != 0;
  if constexpr (J >= 16) {
    u64 alo, ahi, blo, bhi;
    lane_pair64<J>(a, lane, alo, ahi);
    lane_pair64<J>(b, lane, blo, bhi);
    const bool ta = (ahi > alo) != upper;
    const bool tb = (bhi > blo) == upper;
    a = ta ? ahi : alo;
    b = tb ? bhi : blo;
  } else {
    const u64 ya = lane_xor64<J>(a);
    const u64 yb = lane_xor64<J>(b);
    const bool ta = (ya > a) != upper;
    const bool tb = (yb > b) == upper;
    a = ta ? ya : a;
    b = tb ? yb : b;
  }
  if constexpr (J > 1) bitonic_merge_two<J / 2>(a, b, lane);
}

// The 64 largest of four lists of 64 keys, each sorted descending (list(c, i) = i-th best of list c, 0 for
// a missing list), one result per lane, sorted descending.  A descending list against an ascending
// one is a bitonic pair whose lane-wise maximum holds the 64 best of both; the two first-level
// merges are independent and the second one is produced ascending so that no lane reversal is needed.
template <typename List>
__device__ __forceinline__ u64 wave_merge4(List list, int lane) {
  const u64 a0 = list(0, lane), a1 = list(1, 63 - lane), b0 = list(2, 63 - lane), b1 = list(3, lane);
  u64 a = a1 > a0 ? a1 : a0;
  u64 b = b1 > b0 ? b1 : b0;
  bitonic_merge_two<32>(a, b, lane);
  u64 g = b > a ? b : a;
  bitonic_merge<32, false, u64>(g, lane);
  return g;
}

// Bitonic sort of one key per lane, descending by lane (lane 0 ends with the maximum).
template <typename T>
__device__ __forceinline__ T wave_sort_desc_fast(T x) {
  const int lane = lane_id();
  sort_merge<2, 1, T>(x, lane);
  sort_merge<4, 2, T>(x, lane);
  sort_merge<8, 4, T>(x, lane);
  sort_merge<16, 8, T>(x, lane);
  sort_merge<32, 16, T>(x, lane);
  sort_merge<64, 32, T>(x, lane);
  return x;
}

// k-th largest of the wave's R keys per lane (0 if fewer than k keys are non-zero): bisection on the
// key bits with wave-wide population counts.
template <int R>
__device__ __forceinline__ uint32_t wave_kth_largest(const uint32_t (&key)[R], int k) {
  uint32_t prefix = 0u;
#pragma unroll 1
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t cand = prefix | (1u << bit);
    int cnt = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) cnt += __popcll(__ballot(key[r] >= cand));
    if (cnt >= k) prefix = cand;
  }
  return prefix;
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
  base = wave_read_lane(base, leader);
  return base + static_cast<uint32_t>(__popcll(b & ((1ull << lane) - 1ull)));
}

__device__ __forceinline__ int first_lane(u64 ballot) { return ballot ? __ffsll(static_cast<long long>(ballot)) - 1 : -1; }

__device__ __forceinline__ void store_coherent(u64* p, u64 v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A key tau such that at least k of the keys offered by the block's threads are >= tau (0 if there
// are fewer than k offers).  One offer per thread (0 = none); only the first nw waves hold offers.
// Every wave sorts its 64 offers and pools its best 64/nw; the pool's k-th entry is the exact k-th
// best offer unless one wave holds more than its share of the top k.  Waves write their shares in
// alternating directions, so the pool arrives as sorted runs that only the last merge levels of the
// sorting network have to join, and every wave sorts the pool for itself: one barrier, no broadcast.
// Any block of up to 16 waves, 1 <= k <= 64.
__device__ __forceinline__ uint32_t block_pool_bound(uint32_t offer, int k, int nw, uint32_t* pool) {
  const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
  if (nw < 1) nw = 1;
  const int c = 64 / nw;
  const uint32_t sorted = wave_sort_desc_fast<uint32_t>(offer);
  const bool runs = (nw == 8);  // shares of 8: the sorting network's state before its 16-merge level
  if (wave < nw && lane < c) pool[wave * c + ((runs && (wave & 1)) ? c - 1 - lane : lane)] = sorted;
  if (tid < 64 && tid >= nw * c) pool[tid] = 0u;
  __syncthreads();
  uint32_t ps = pool[lane];
  if (runs) {
    sort_merge<16, 8, uint32_t>(ps, lane);
    sort_merge<32, 16, uint32_t>(ps, lane);
    sort_merge<64, 32, uint32_t>(ps, lane);
  } else {
    ps = wave_sort_desc_fast<uint32_t>(ps);
  }
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(ps, k - 1));
}

}  // namespace ms
