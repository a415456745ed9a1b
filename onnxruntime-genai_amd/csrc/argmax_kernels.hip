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
  float v[kElems];
  Loader<InT>::load(lrow, V, chunk, v);
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

// Small problems (a few rows of at most kRowKernelMaxVocab logits) are latency-bound: one 1024-thread
// workgroup per row walks the whole row, so no cross-workgroup hand-over is needed.
constexpr int kRowKernelMaxVocab = 65536;

template <typename InT>
__global__ __launch_bounds__(1024) void argmax_row_kernel(const ArgmaxArgs a) {
  constexpr int VEC = Loader<InT>::VEC;
  constexpr int NB = 8;  // vectors a thread has in flight: all their loads are issued before any is used
  const int row = blockIdx.x, tid = threadIdx.x;
  // everything this latency-bound kernel reads from its arguments, fetched together
  const int V = arg_now(a.vocab);
  const int64_t row_stride = arg_now(a.row_stride);
  const InT* const logits = static_cast<const InT*>(arg_now(a.logits));
  int32_t* const out_tokens = arg_now(a.out_tokens);
  const uint32_t* const mask = arg_now(a.xf.mask);
  const int32_t* const history = arg_now(a.xf.history);
  const int32_t* const history_lens = arg_now(a.xf.history_lens);
  const uint32_t* const ban = arg_now(a.xf.ban);
  const int history_stride = arg_now(a.xf.history_stride);
  const int history_len = arg_now(a.xf.history_len);
  const int min_length = arg_now(a.xf.min_length);
  const int n_eos_all = arg_now(a.xf.n_eos);
  const float penalty = arg_now(a.xf.penalty);
  __shared__ uint32_t hist_bits[kRowKernelMaxVocab / 32];
  __shared__ u64 red64[16];
  const InT* lrow = logits + static_cast<size_t>(row) * row_stride;
  const bool pen = history && (history_lens || history_len > 0) && (penalty != 1.0f || ban);  // Xform::use_penalty
  const bool has_mask = mask != nullptr;
  const bool active = has_mask || pen || n_eos_all > 0;
  const uint32_t* mrow = has_mask ? mask + static_cast<size_t>(row) * ((V - 1) / 32 + 1) : nullptr;
  const int hlen = pen ? (history_lens ? history_lens[row] : history_len) : 0;
  const int n_eos = (history_lens && min_length > 0 && history_lens[row] >= min_length) ? 0 : n_eos_all;
  const uint32_t* ban_row = ban ? ban + static_cast<size_t>(row) * ((V - 1) / 32 + 1) : nullptr;
  u64 best = 0;
  for (int base = 0; base < V; base += 1024 * VEC * NB) {
    float v[NB][VEC];
    uint32_t mw[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int i0 = base + (j * 1024 + tid) * VEC;
      mw[j] = (has_mask && i0 < V) ? mrow[i0 >> 5] : 0u;  // VEC divides 32: one word covers the vector
      if (i0 + VEC <= V) {
        if constexpr (VEC == 4) {
          const v4f_any q = *reinterpret_cast<const v4f_any*>(lrow + i0);
          v[j][0] = q.x, v[j][1] = q.y, v[j][2] = q.z, v[j][3] = q.w;
        } else {
          const v4u_any q = *reinterpret_cast<const v4u_any*>(lrow + i0);
          const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            v[j][2 * c] = narrow_bits_to_float<InT>(w[c] & 0xffffu);
            v[j][2 * c + 1] = narrow_bits_to_float<InT>(w[c] >> 16);
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[j][c] = (i0 + c < V) ? load_one<InT>(lrow, i0 + c) : 0.0f;
      }
    }
    if (pen && base == 0) {  // built while the first batch of loads is in flight
      const int32_t* h = history + static_cast<size_t>(row) * history_stride;
      int hv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) hv[r] = (r * 1024 + tid < hlen) ? h[r * 1024 + tid] : -1;
      for (int i = tid; i < (V + 31) / 32; i += 1024) hist_bits[i] = 0u;
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (hv[r] >= 0 && hv[r] < V) atomicOr(&hist_bits[hv[r] >> 5], 1u << (hv[r] & 31));
      for (int i = 4096 + tid; i < hlen; i += 1024) {
        const int t = h[i];
        if (t >= 0 && t < V) atomicOr(&hist_bits[t >> 5], 1u << (t & 31));
      }
      __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int i0 = base + (j * 1024 + tid) * VEC;
      const uint32_t hw = (pen && i0 < V) ? hist_bits[i0 >> 5] : 0u;
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        const int idx = i0 + c;
        if (idx < V) {
          float x = v[j][c];
          if (active) x = xform_value(x, penalty, a.xf.eos, idx, mw[j], has_mask, (hw >> (idx & 31)) & 1u, n_eos, ban_row);
          u64 k = make_key64(order_key(x), static_cast<uint32_t>(idx));
          if (idx == 0 && x != x) k = ~0ull;  // NaN at index 0 is sticky
          if (k == 0) k = 1;
          best = k > best ? k : best;
        }
      }
    }
  }
  best = block_max<u64>(best, red64);
  if (tid == 0) out_tokens[row] = static_cast<int32_t>(key64_index(best));
}

// mask -> min-length -> repetition penalty, written back in place
// (LaunchAddLogitsMask / ApplyMinLength / ApplyRepetitionPenalty).
__global__ __launch_bounds__(kBlock) void process_logits_kernel(float* logits, int64_t row_stride, int vocab, const Xform xf) {
  const int row = blockIdx.y, chunk = blockIdx.x;
  __shared__ uint32_t hist_bits[kChunk / 32];
  float* lrow = logits + static_cast<size_t>(row) * row_stride;
  const bool aligned = ((reinterpret_cast<uintptr_t>(lrow) & 15u) == 0);
  float v[kElems];
  Loader<float>::load(lrow, vocab, chunk, v);
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
  if (a->vocab <= ms::kRowKernelMaxVocab && a->rows * a->chunks < 256) {
    if (dtype == MI355X_F16)
      hipLaunchKernelGGL(ms::argmax_row_kernel<uint16_t>, dim3(a->rows), dim3(1024), 0, stream, *a);
    else if (dtype == MI355X_BF16)
      hipLaunchKernelGGL(ms::argmax_row_kernel<ms::bf16_t>, dim3(a->rows), dim3(1024), 0, stream, *a);
    else
      hipLaunchKernelGGL(ms::argmax_row_kernel<float>, dim3(a->rows), dim3(1024), 0, stream, *a);
    return hipGetLastError();
  }
  dim3 grid(a->chunks, a->rows);
  if (dtype == MI355X_F16)
    hipLaunchKernelGGL(ms::argmax_kernel<uint16_t>, grid, dim3(ms::kBlock), 0, stream, *a);
  else if (dtype == MI355X_BF16)
    hipLaunchKernelGGL(ms::argmax_kernel<ms::bf16_t>, grid, dim3(ms::kBlock), 0, stream, *a);
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
