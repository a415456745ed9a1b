// Segment-wise row access shared by the kernels that cut long rows into segments of kSegElems
// elements handled by 256-thread workgroups (exact sequential sums, beam-search candidates).
#pragma once
#include "kernels.h"
#include "device_utils.h"

namespace ms {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

constexpr int kSegBlock = 256;
constexpr int kSegPer = kSegElems / kSegBlock;  // 16 elements per thread

// Loads the 16 elements of thread t in segment `seg`: for j, the VEC consecutive ids starting at
// seg*kSegElems + (j*256 + t)*VEC (VEC = 4 for fp32, 8 for fp16 and bf16).  Ids >= vocab yield `fill`.
template <typename InT>
__device__ __forceinline__ void seg_load(const InT* row, int vocab, int seg, float fill, float (&v)[kSegPer]) {
  constexpr int VEC = sizeof(InT) == 4 ? 4 : 8;
  constexpr int NV = kSegPer / VEC;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i0 = seg * kSegElems + (j * kSegBlock + static_cast<int>(threadIdx.x)) * VEC;
    if (i0 + VEC <= vocab) {
      if constexpr (VEC == 4) {
        const v4f_any q = *reinterpret_cast<const v4f_any*>(row + i0);
        v[j * 4] = q.x, v[j * 4 + 1] = q.y, v[j * 4 + 2] = q.z, v[j * 4 + 3] = q.w;
      } else {
        const v4u q = *reinterpret_cast<const v4u_any*>(row + i0);
        if constexpr (__is_same(InT, uint16_t)) {
          widen_half8(q, &v[j * 8]);  // the hardware conversion, redone by the bit formula where it differs
        } else {
          const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            v[j * 8 + 2 * c] = narrow_bits_to_float<InT>(w[c] & 0xffffu);
            v[j * 8 + 2 * c + 1] = narrow_bits_to_float<InT>(w[c] >> 16);
          }
        }
      }
    } else {
#pragma unroll
      for (int c = 0; c < VEC; ++c) v[j * VEC + c] = (i0 + c < vocab) ? load_one<InT>(row, i0 + c) : fill;
    }
  }
}

template <typename InT>
__device__ __forceinline__ int seg_index(int seg, int e) {
  constexpr int VEC = sizeof(InT) == 4 ? 4 : 8;
  return seg * kSegElems + ((e / VEC) * kSegBlock + static_cast<int>(threadIdx.x)) * VEC + e % VEC;
}

}  // namespace ms
