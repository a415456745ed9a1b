// Greedy argmax with fused logits processing, and the in-place logits-processing kernel.
#include "kernels.h"

namespace ms {

// One workgroup per (chunk, row): block maximum of key64, folded into the row's slot with an atomic
// max; the last workgroup to arrive publishes the token and clears the slot for the next launch.
// Reproduces ArgMax's strict '>' scan (src/search.h:9-29): first maximum wins, a NaN at index 0 is
// never replaced, NaNs elsewhere never win.
template <typename InT>
__global__ __launch_bounds__(kBlock) void argmax_kernel(const ArgmaxArgs a) {
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int V = a.vocab;
  __shared__ uint32_t hist_bits[kChunk / 32];
  __shared__ u64 red64[4];
  const InT* lrow = static_cast<const InT*>(a.logits) + static_cast<size_t>(row) * a.row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(lrow) & 15u) == 0);
  float v[kElems];
  Loader<InT>::load(lrow, aligned, V, chunk, v);
  if (a.xf.active()) {
    if (a.xf.use_penalty()) build_history_bitmap(a.xf, row, chunk * kChunk, hist_bits);
    xform_chunk<InT>(a.xf, row, V, chunk, hist_bits, v);
  }
  u64 best = 0;
#pragma unroll
  for (int e = 0; e < kElems; ++e) {
    const int idx = Loader<InT>::index_of(chunk, e / Loader<InT>::VEC, e % Loader<InT>::VEC);
    if (idx < V) {
      u64 k = make_key64(order_key(v[e]), static_cast<uint32_t>(idx));
      if (idx == 0 && v[e] != v[e]) k = ~0ull;  // NaN at index 0 is sticky
      if (k == 0) k = 1;                         // keep real elements above the empty slot value
      best = k > best ? k : best;
    }
  }
  best = block_max<u64>(best, red64);
  if (threadIdx.x == 0) {
    atomicMax(&a.row_best[row], best);
    __threadfence();
    const uint32_t old = atomicAdd(&a.row_arrive[row], 1u);
    if (old == static_cast<uint32_t>(a.chunks) - 1u) {
      __threadfence();
      const u64 k = load_coherent(&a.row_best[row]);
      a.out_tokens[row] = static_cast<int32_t>(key64_index(k));
      a.row_best[row] = 0;
      a.row_arrive[row] = 0u;
    }
  }
}

// mask -> min-length -> repetition penalty, written back in place
// (LaunchAddLogitsMask / ApplyMinLength / ApplyRepetitionPenalty).
__global__ __launch_bounds__(kBlock) void process_logits_kernel(float* logits, int64_t row_stride, int vocab, const Xform xf) {
  const int row = blockIdx.y, chunk = blockIdx.x;
  __shared__ uint32_t hist_bits[kChunk / 32];
  float* lrow = logits + static_cast<size_t>(row) * row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(lrow) & 15u) == 0);
  float v[kElems];
  Loader<float>::load(lrow, aligned, vocab, chunk, v);
  if (xf.use_penalty()) build_history_bitmap(xf, row, chunk * kChunk, hist_bits);
  xform_chunk<float>(xf, row, vocab, chunk, hist_bits, v);
#pragma unroll
  for (int j = 0; j < Loader<float>::NV; ++j) {
    const int i0 = Loader<float>::index_of(chunk, j, 0);
    if (aligned && i0 + 4 <= vocab) {
      *reinterpret_cast<float4*>(lrow + i0) = make_float4(v[j * 4], v[j * 4 + 1], v[j * 4 + 2], v[j * 4 + 3]);
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (i0 + c < vocab) lrow[i0 + c] = v[j * 4 + c];
    }
  }
}

}  // namespace ms

extern "C" hipError_t ms_launch_argmax(const ms::ArgmaxArgs* a, int dtype, hipStream_t stream) {
  dim3 grid(a->chunks, a->rows);
  if (dtype == MI355X_F16)
    hipLaunchKernelGGL(ms::argmax_kernel<uint16_t>, grid, dim3(ms::kBlock), 0, stream, *a);
  else
    hipLaunchKernelGGL(ms::argmax_kernel<float>, grid, dim3(ms::kBlock), 0, stream, *a);
  return hipGetLastError();
}

extern "C" hipError_t ms_launch_process_logits(float* logits, int64_t row_stride, int rows, int vocab,
                                               const ms::Xform* xf, hipStream_t stream) {
  dim3 grid((vocab + ms::kChunk - 1) / ms::kChunk, rows);
  hipLaunchKernelGGL(ms::process_logits_kernel, grid, dim3(ms::kBlock), 0, stream, logits, row_stride, vocab, *xf);
  return hipGetLastError();
}
