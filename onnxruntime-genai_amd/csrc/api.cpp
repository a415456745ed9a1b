// Host side of the C ABI declared in include/mi355x_search.h: argument validation, workspace
// management and kernel launches.  No computation happens here, and there is no CPU fallback: every
// entry point either launches the HIP kernels or fails.
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <new>
#include <string>
#include <vector>
#include "kernels.h"
#include "mi355x_search.h"

namespace {

thread_local std::string g_error;

int Fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
  return code;
}

#define HIP_TRY(expr)                                                                       \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess) return Fail(MI355X_E_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

int NextPow2(int v) {
  int p = 64;
  while (p < v) p <<= 1;
  return p;
}

}  // namespace

struct mi355x_search_ctx {
  int device{};
  int max_rows{}, max_vocab{}, max_chunks{};
  size_t bytes{};
  std::vector<void*> allocs;
  ms::u64* cand_small{};
  uint32_t* chunk_cnt{};
  uint32_t* chunk_max{};
  ms::u64* chunk_next{};
  uint32_t* row_arrive{};
  ms::u64* row_best{};
  ms::u64* big{};
  size_t big_stride{};
  uint32_t* fallback_rows{};
  mi355x_sample_params* params_dev{};
  void** ptr_table{};      // device copy of pointer tables (kv gather)
  size_t ptr_table_cap{};

  template <typename T>
  hipError_t Alloc(T** p, size_t count, bool zero) {
    void* q = nullptr;
    const size_t n = count * sizeof(T);
    hipError_t e = hipMalloc(&q, n ? n : 16);
    if (e != hipSuccess) return e;
    allocs.push_back(q);
    bytes += n;
    if (zero) {
      e = hipMemset(q, 0, n ? n : 16);
      if (e != hipSuccess) return e;
    }
    *p = static_cast<T*>(q);
    return hipSuccess;
  }
};

namespace {

int CheckRows(const mi355x_search_ctx* ctx, int rows, int vocab) {
  if (!ctx) return Fail(MI355X_E_INVALID, "null context");
  if (rows <= 0 || vocab <= 0) return Fail(MI355X_E_INVALID, "rows (%d) and vocab (%d) must be positive", rows, vocab);
  if (rows > ctx->max_rows || vocab > ctx->max_vocab)
    return Fail(MI355X_E_CAPACITY, "rows=%d vocab=%d exceed the context's capacity (%d, %d)", rows, vocab,
                ctx->max_rows, ctx->max_vocab);
  return MI355X_OK;
}

int MakeXform(const mi355x_logits_xform* in, ms::Xform* out) {
  std::memset(out, 0, sizeof(*out));
  out->penalty = 1.0f;
  if (!in) return MI355X_OK;
  out->mask = in->mask;
  out->history = in->history;
  out->history_stride = in->history_stride;
  out->history_len = in->history_len;
  out->penalty = in->repetition_penalty;
  if (in->history && in->history_len > in->history_stride)
    return Fail(MI355X_E_INVALID, "history_len (%d) exceeds history_stride (%d)", in->history_len, in->history_stride);
  if (in->history_len < 0) return Fail(MI355X_E_INVALID, "negative history_len");
  if (in->apply_min_length) {
    if (in->n_eos < 0 || in->n_eos > MI355X_MAX_EOS)
      return Fail(MI355X_E_INVALID, "n_eos (%d) out of range [0, %d]", in->n_eos, MI355X_MAX_EOS);
    out->n_eos = in->n_eos;
    for (int i = 0; i < in->n_eos; ++i) out->eos[i] = in->eos_ids[i];
  }
  return MI355X_OK;
}

}  // namespace

extern "C" {

const char* mi355x_search_last_error(void) { return g_error.c_str(); }

int mi355x_search_create(int device, int max_rows, int max_vocab, mi355x_search_ctx** out) {
  if (!out) return Fail(MI355X_E_INVALID, "null output pointer");
  *out = nullptr;
  if (max_rows <= 0 || max_vocab <= 0) return Fail(MI355X_E_INVALID, "max_rows and max_vocab must be positive");
  int count = 0;
  HIP_TRY(hipGetDeviceCount(&count));
  if (device < 0 || device >= count) return Fail(MI355X_E_INVALID, "device %d out of range (%d visible)", device, count);
  HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return Fail(MI355X_E_UNSUPPORTED, "kernels are built for gfx950 only; device %d is %s", device, prop.gcnArchName);
  auto* c = new (std::nothrow) mi355x_search_ctx;
  if (!c) return Fail(MI355X_E_INVALID, "out of host memory");
  c->device = device;
  c->max_rows = max_rows;
  c->max_vocab = max_vocab;
  c->max_chunks = (max_vocab + ms::kChunk - 1) / ms::kChunk;
  const size_t rc = static_cast<size_t>(max_rows) * c->max_chunks;
  c->big_stride = static_cast<size_t>(NextPow2(max_vocab));
  if (c->big_stride < static_cast<size_t>(c->max_chunks) * ms::kChunk) c->big_stride = static_cast<size_t>(c->max_chunks) * ms::kChunk;
  if (c->big_stride < static_cast<size_t>(ms::kSChunk)) c->big_stride = ms::kSChunk;
  hipError_t e = hipSuccess;
  auto ok = [&](hipError_t r) {
    if (e == hipSuccess) e = r;
  };
  const size_t sc = static_cast<size_t>(max_rows) * ((max_vocab + ms::kSChunk - 1) / ms::kSChunk);
  ok(c->Alloc(&c->cand_small, sc * ms::kSmallCap, true));  // all-zero between launches
  ok(c->Alloc(&c->chunk_cnt, rc, true));
  ok(c->Alloc(&c->chunk_max, rc, true));
  ok(c->Alloc(&c->chunk_next, rc, true));
  ok(c->Alloc(&c->row_arrive, static_cast<size_t>(max_rows), true));
  ok(c->Alloc(&c->row_best, static_cast<size_t>(max_rows), true));
  ok(c->Alloc(&c->big, static_cast<size_t>(max_rows) * c->big_stride, false));
  ok(c->Alloc(&c->fallback_rows, 1, true));
  ok(c->Alloc(&c->params_dev, static_cast<size_t>(max_rows), false));
  c->ptr_table_cap = 4096;
  ok(c->Alloc(&c->ptr_table, c->ptr_table_cap, false));
  if (e == hipSuccess) e = ms_sample_init();
  if (e != hipSuccess) {
    mi355x_search_destroy(c);
    return Fail(MI355X_E_HIP, "workspace allocation failed: %s", hipGetErrorString(e));
  }
  *out = c;
  return MI355X_OK;
}

void mi355x_search_destroy(mi355x_search_ctx* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  for (void* p : ctx->allocs) (void)hipFree(p);
  delete ctx;
}

size_t mi355x_search_workspace_bytes(const mi355x_search_ctx* ctx) { return ctx ? ctx->bytes : 0; }

int mi355x_process_logits(mi355x_search_ctx* ctx, void* stream, float* logits, int64_t row_stride, int rows,
                          int vocab, const mi355x_logits_xform* xf) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits) return Fail(MI355X_E_INVALID, "null logits");
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride (%lld) smaller than vocab (%d)", (long long)row_stride, vocab);
  ms::Xform x;
  if (int r = MakeXform(xf, &x)) return r;
  if (!x.active()) return MI355X_OK;
  HIP_TRY(ms_launch_process_logits(logits, row_stride, rows, vocab, &x, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_argmax(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                  int rows, int vocab, const mi355x_logits_xform* xf, int32_t* out_tokens) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits || !out_tokens) return Fail(MI355X_E_INVALID, "null logits or output");
  if (dtype != MI355X_F32 && dtype != MI355X_F16) return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  ms::ArgmaxArgs a{};
  if (int r = MakeXform(xf, &a.xf)) return r;
  a.logits = logits;
  a.row_stride = row_stride;
  a.rows = rows;
  a.vocab = vocab;
  a.chunks = (vocab + ms::kChunk - 1) / ms::kChunk;
  a.out_tokens = out_tokens;
  a.row_best = ctx->row_best;
  a.row_arrive = ctx->row_arrive;
  HIP_TRY(ms_launch_argmax(&a, dtype, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_sample(mi355x_search_ctx* ctx, void* stream, const float* logits, int64_t row_stride, int rows,
                  int vocab, const mi355x_logits_xform* xf, mi355x_sample_params params,
                  const mi355x_sample_params* per_row_params, const double* uniforms, int32_t* out_tokens,
                  int32_t* kept_count, int32_t* kept_ids, float* kept_probs, int kept_capacity) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits || !uniforms || !out_tokens) return Fail(MI355X_E_INVALID, "null logits, uniforms or output");
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  if ((kept_ids || kept_probs) && kept_capacity <= 0) return Fail(MI355X_E_INVALID, "kept_capacity must be positive");
  if (kept_probs && !kept_ids) return Fail(MI355X_E_INVALID, "kept_probs requires kept_ids");
  hipStream_t s = static_cast<hipStream_t>(stream);
  ms::SampleArgs a{};
  if (int r = MakeXform(xf, &a.xf)) return r;
  bool any_nucleus = false;
  auto check = [&](const mi355x_sample_params& p) -> int {
    if (!(p.temperature > 0.0f)) return Fail(MI355X_E_INVALID, "temperature must be positive (got %g)", p.temperature);
    if (p.k <= 1 && vocab > 64) any_nucleus = true;
    return MI355X_OK;
  };
  if (per_row_params) {
    for (int r = 0; r < rows; ++r)
      if (int rc = check(per_row_params[r])) return rc;
    HIP_TRY(hipMemcpyAsync(ctx->params_dev, per_row_params, sizeof(mi355x_sample_params) * rows,
                           hipMemcpyHostToDevice, s));
    a.per_row = ctx->params_dev;
  } else {
    if (int rc = check(params)) return rc;
  }
  a.logits = logits;
  a.row_stride = row_stride;
  a.rows = rows;
  a.vocab = vocab;
  a.chunks = (vocab + ms::kSChunk - 1) / ms::kSChunk;
  a.uniform = params;
  a.uniforms = uniforms;
  a.out_tokens = out_tokens;
  a.kept_count = kept_count;
  a.kept_ids = kept_ids;
  a.kept_probs = kept_probs;
  a.kept_capacity = kept_capacity;
  a.cand_small = ctx->cand_small;
  a.chunk_cnt = ctx->chunk_cnt;
  a.chunk_max = ctx->chunk_max;
  a.chunk_next = ctx->chunk_next;
  a.row_arrive = ctx->row_arrive;
  a.big = ctx->big;
  a.big_stride = ctx->big_stride;
  a.fallback_rows = ctx->fallback_rows;
#ifdef MS_DEBUG_STAGES
  a.debug_stage = getenv("MS_STAGE") ? atoi(getenv("MS_STAGE")) : 0;
#endif
  HIP_TRY(ms_launch_sample(&a, any_nucleus, s));
  return MI355X_OK;
}

int mi355x_search_fallback_rows(mi355x_search_ctx* ctx, void* stream, unsigned* rows) {
  if (!ctx || !rows) return Fail(MI355X_E_INVALID, "null argument");
  HIP_TRY(hipMemcpyAsync(rows, ctx->fallback_rows, sizeof(unsigned), hipMemcpyDeviceToHost,
                         static_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

}  // extern "C"
