// Host side of the C ABI declared in include/mi355x_search.h: argument validation, workspace
// management and kernel launches.  No computation happens here, and there is no CPU fallback: every
// entry point either launches the HIP kernels or fails.
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cmath>
#include <cstring>
#include <cstdlib>
#include <new>
#include <string>
#include <vector>
#include "api_internal.h"

namespace {

thread_local std::string g_error;

}  // namespace

int ms_vfail(int code, const char* fmt, va_list ap) {
  char buf[512];
  vsnprintf(buf, sizeof(buf), fmt, ap);
  g_error = buf;
  return code;
}

namespace {

int Fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  ms_vfail(code, fmt, ap);
  va_end(ap);
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
  uint32_t* chunk_thr{};
  ms::u64* chunk_next{};
  uint32_t* row_arrive{};
  ms::u64* row_best{};
  ms::u64* big{};
  ms::u64* big2{};
  size_t big_stride{};
  uint32_t* fallback_rows{};
  uint32_t* row_done{};
  int poll_limit{ms::kDefaultPollLimit};
  uint32_t* ban{};  // [max_rows, mask words]: ids banned by the no-repeat-n-gram rule
  mi355x_sample_params* params_dev{};
  void** ptr_table{};      // device copy of pointer tables (kv gather)
  size_t ptr_table_cap{};
  float* beam_row_scores{};
  ms::u64* seg_cand{};  // [max_rows][max_segs][kBeamMaxCand] beam-search candidates per segment
  int max_segs{};
  uint32_t* seg_max{};
  double* seg_sum{};
  int4* seg_step{};
  int4* sub_step{};
  int* sub_se{};
  float* row_max{};
  float* row_sum{};
  int32_t* row_index{};  // device copy of per-row host indices (logits hand-off)
  int32_t* beam_row_tokens{};
  // Pinned host staging for the calls that take a table from a caller's HOST array (per-row parameters of more
  // than 64 rows, the KV gather's pointer tables, token_index): the call copies the array into a slot here and
  // records a copy from the slot to the device table.  Slots of the ring are reused once the copy that read them
  // is done (an event per slot); a call on a capturing stream gets a slot of its own that is never reused, so the
  // copy node of its graph reads the same bytes at every replay.
  ms::SideStreams sides{};  // where the kernels of a call with rows in several modes run side by side
  static constexpr int kStageRing = 8, kStageCaptured = 56;
  char* stage{};
  size_t stage_slot_bytes{};
  hipEvent_t stage_event[kStageRing]{};
  bool stage_pending[kStageRing]{};
  int stage_next{}, stage_captured{};

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

// Validates the caller's logits-processing request and turns it into the kernels' form.  With a
// no-repeat-n-gram size it also launches the kernel that writes the rows' banned-id bitmaps into
// the context's workspace.
int MakeXform(mi355x_search_ctx* ctx, const mi355x_logits_xform* in, int rows, int vocab, hipStream_t stream,
              ms::Xform* out) {
  return ms_make_xform(ctx, in, rows, vocab, stream, out);
}

}  // namespace

// `ctx` may be null (an entry point without a context): the n-gram rule, whose bitmaps live in a
// context's workspace, is then refused.
int ms_make_xform(mi355x_search_ctx* ctx, const mi355x_logits_xform* in, int rows, int vocab, hipStream_t stream,
                  ms::Xform* out) {
  std::memset(out, 0, sizeof(*out));
  out->penalty = 1.0f;
  if (!in) return MI355X_OK;
  out->mask = in->mask;
  out->history = in->history;
  out->history_stride = in->history_stride;
  out->history_len = in->history_len;
  out->history_lens = in->history ? in->history_lens : nullptr;
  out->min_length = in->min_length;
  out->penalty = in->repetition_penalty;
  if (in->history && !in->history_lens && in->history_stride != 0 && in->history_len > in->history_stride)
    return Fail(MI355X_E_INVALID, "history_len (%d) exceeds history_stride (%d)", in->history_len, in->history_stride);
  if (in->history_len < 0 || in->history_stride < 0) return Fail(MI355X_E_INVALID, "negative history_len or history_stride");
  if (in->history_lens && !in->history) return Fail(MI355X_E_INVALID, "history_lens given without history");
  if (in->apply_min_length || (in->history_lens && in->min_length > 0)) {
    if (in->n_eos < 0 || in->n_eos > MI355X_MAX_EOS)
      return Fail(MI355X_E_INVALID, "n_eos (%d) out of range [0, %d]", in->n_eos, MI355X_MAX_EOS);
    out->n_eos = in->n_eos;
    for (int i = 0; i < in->n_eos; ++i) out->eos[i] = in->eos_ids[i];
  }
  if (in->no_repeat_ngram_size > 0) {
    if (!in->history) return Fail(MI355X_E_INVALID, "no_repeat_ngram_size needs a history");
    if (!ctx) return Fail(MI355X_E_UNSUPPORTED, "no_repeat_ngram_size needs a context (its bitmaps live in the workspace)");
    if (out->history_lens || out->history_len >= in->no_repeat_ngram_size) {
      HIP_TRY(ms_launch_ngram_ban(out, rows, vocab, in->no_repeat_ngram_size, ctx->ban, stream));
      out->ban = ctx->ban;
    }
  }
  return MI355X_OK;
}

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
  ok(c->Alloc(&c->chunk_thr, rc, true));
  ok(c->Alloc(&c->chunk_next, rc, true));
  ok(c->Alloc(&c->row_arrive, static_cast<size_t>(max_rows), true));
  ok(c->Alloc(&c->row_best, static_cast<size_t>(max_rows), true));
  ok(c->Alloc(&c->big, static_cast<size_t>(max_rows) * c->big_stride, false));
  ok(c->Alloc(&c->big2, static_cast<size_t>(max_rows) * c->big_stride, false));
  ok(c->Alloc(&c->row_done, static_cast<size_t>(max_rows), true));
  ok(c->Alloc(&c->fallback_rows, 4, true));  // [0] rows finished by the exact path, [1] a wait gave up, [2] exact-sum segments whose wait gave up
  ok(c->Alloc(&c->ban, static_cast<size_t>(max_rows) * ((max_vocab - 1) / 32 + 1), false));
  ok(c->Alloc(&c->params_dev, static_cast<size_t>(max_rows), false));
  ok(c->Alloc(&c->beam_row_scores, static_cast<size_t>(max_rows) * ms::kBeamMaxCand, false));
  ok(c->Alloc(&c->beam_row_tokens, static_cast<size_t>(max_rows) * ms::kBeamMaxCand, false));
  c->max_segs = (max_vocab + ms::kSegElems - 1) / ms::kSegElems;
  ok(c->Alloc(&c->seg_max, static_cast<size_t>(max_rows) * c->max_segs, false));
  ok(c->Alloc(&c->seg_sum, static_cast<size_t>(max_rows) * c->max_segs, false));
  // "not written yet" everywhere (all bits set): the state the exact-sum kernels expect and leave behind
  if (c->seg_sum) ok(hipMemset(c->seg_sum, 0xff, static_cast<size_t>(max_rows) * c->max_segs * sizeof(double)));
  ok(c->Alloc(&c->seg_cand, static_cast<size_t>(max_rows) * c->max_segs * ms::kBeamMaxCand, false));
  ok(c->Alloc(&c->seg_step, static_cast<size_t>(max_rows) * c->max_segs, false));
  ok(c->Alloc(&c->sub_step, static_cast<size_t>(max_rows) * c->max_segs * ms::kSegSubs, false));
  ok(c->Alloc(&c->sub_se, static_cast<size_t>(max_rows) * c->max_segs * ms::kSegSubs, false));
  ok(c->Alloc(&c->row_max, static_cast<size_t>(max_rows), false));
  ok(c->Alloc(&c->row_sum, static_cast<size_t>(max_rows), false));
  ok(c->Alloc(&c->row_index, static_cast<size_t>(max_rows), false));
  c->ptr_table_cap = 4096;
  ok(c->Alloc(&c->ptr_table, c->ptr_table_cap, false));
  c->stage_slot_bytes = std::max(c->ptr_table_cap * sizeof(void*), static_cast<size_t>(max_rows) * sizeof(mi355x_sample_params));
  c->stage_slot_bytes = (c->stage_slot_bytes + 255) & ~static_cast<size_t>(255);
  if (e == hipSuccess) {
    void* pinned = nullptr;
    e = hipHostMalloc(&pinned, c->stage_slot_bytes * (mi355x_search_ctx::kStageRing + mi355x_search_ctx::kStageCaptured), hipHostMallocDefault);
    c->stage = static_cast<char*>(pinned);
  }
  for (int i = 0; i < mi355x_search_ctx::kStageRing && e == hipSuccess; ++i)
    e = hipEventCreateWithFlags(&c->stage_event[i], hipEventDisableTiming);
  for (hipStream_t& st : c->sides.side)
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
  for (hipEvent_t* ev : {&c->sides.fork, &c->sides.join[0], &c->sides.join[1]})
    if (e == hipSuccess) e = hipEventCreateWithFlags(ev, hipEventDisableTiming);
  if (e == hipSuccess) e = ms_sample_init();
  if (e == hipSuccess) e = ms_static_scratch_setup();  // set-up of mi355x_argmax_static on this device
  // the fills above ran on the null stream: done before a caller's stream, which need not wait for it, uses them
  if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
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
  for (hipEvent_t ev : ctx->stage_event)
    if (ev) (void)hipEventDestroy(ev);
  for (hipStream_t st : ctx->sides.side)
    if (st) (void)hipStreamDestroy(st);
  for (hipEvent_t ev : {ctx->sides.fork, ctx->sides.join[0], ctx->sides.join[1]})
    if (ev) (void)hipEventDestroy(ev);
  if (ctx->stage) (void)hipHostFree(ctx->stage);
  delete ctx;
}

size_t mi355x_search_workspace_bytes(const mi355x_search_ctx* ctx) { return ctx ? ctx->bytes : 0; }

int mi355x_search_abi_version(void) { return MI355X_ABI_VERSION; }

int mi355x_process_logits(mi355x_search_ctx* ctx, void* stream, float* logits, int64_t row_stride, int rows,
                          int vocab, const mi355x_logits_xform* xf) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits) return Fail(MI355X_E_INVALID, "null logits");
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride (%lld) smaller than vocab (%d)", (long long)row_stride, vocab);
  ms::Xform x;
  if (int r = MakeXform(ctx, xf, rows, vocab, static_cast<hipStream_t>(stream), &x)) return r;
  if (!x.active()) return MI355X_OK;
  HIP_TRY(ms_launch_process_logits(logits, row_stride, rows, vocab, &x, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_argmax(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                  int rows, int vocab, const mi355x_logits_xform* xf, int32_t* out_tokens) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits || !out_tokens) return Fail(MI355X_E_INVALID, "null logits or output");
  if (dtype != MI355X_F32 && dtype != MI355X_F16 && dtype != MI355X_BF16)
    return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  // rows of more than 64 logits go through the fused selection kernel (k = 1, ids only), whatever their type
  const int fused_chunks = (vocab + ms::kSChunk - 1) / ms::kSChunk;
  const bool fused = vocab > 64 && fused_chunks * ms::kSmallCap <= ms::kAllCap && rows * fused_chunks >= ms::kArgmaxFusedMinBlocks;
  if (fused) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    ms::SampleArgs f{};
    if (int r = MakeXform(ctx, xf, rows, vocab, s, &f.xf)) return r;
    f.logits = logits;
    f.dtype = dtype;
    f.row_stride = row_stride;
    f.rows = rows;
    f.vocab = vocab;
    f.chunks = fused_chunks;
    f.uniform = mi355x_sample_params{1, 0.0f, 1.0f};
    f.out_tokens = out_tokens;
    f.emit_topk = ms::kEmitArgmax;
    f.cand_small = ctx->cand_small;
    f.chunk_cnt = ctx->chunk_cnt;
    f.chunk_max = ctx->chunk_max;
    f.chunk_thr = ctx->chunk_thr;
    f.chunk_next = ctx->chunk_next;
    f.big = ctx->big;
    f.big_stride = ctx->big_stride;
    f.fallback_rows = ctx->fallback_rows;
    f.poll_limit = ctx->poll_limit;
    HIP_TRY(ms_launch_sample(&f, nullptr, true, false, false, s, nullptr));
    return MI355X_OK;
  }
  ms::ArgmaxArgs a{};
  if (int r = MakeXform(ctx, xf, rows, vocab, static_cast<hipStream_t>(stream), &a.xf)) return r;
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
  return mi355x_sample_typed(ctx, stream, logits, MI355X_F32, row_stride, rows, vocab, xf, params, per_row_params,
                             uniforms, out_tokens, kept_count, kept_ids, kept_probs, kept_capacity);
}

namespace {

// True while `s` records into a graph: an entry point that reads a caller's HOST array with an asynchronous copy
// would leave a node that reads that array again at every replay.
bool Capturing(hipStream_t s) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(s, &status) == hipSuccess && status != hipStreamCaptureStatusNone;
}

// Records a copy of `bytes` bytes of the caller's host array `src` to the device table `dst` on stream s, through a
// pinned staging slot of the context (see mi355x_search_ctx::stage).
int StageToDevice(mi355x_search_ctx* ctx, hipStream_t s, void* dst, const void* src, size_t bytes) {
  if (bytes > ctx->stage_slot_bytes) return Fail(MI355X_E_CAPACITY, "a host table of %zu bytes exceeds the staging slot", bytes);
  const bool capturing = Capturing(s);
  int slot;
  if (capturing) {
    if (ctx->stage_captured == mi355x_search_ctx::kStageCaptured)
      return Fail(MI355X_E_UNSUPPORTED, "this context has staged %d host tables for graph capture, all it provides for",
                  mi355x_search_ctx::kStageCaptured);
    slot = mi355x_search_ctx::kStageRing + ctx->stage_captured++;
  } else {
    slot = ctx->stage_next;
    ctx->stage_next = (slot + 1) % mi355x_search_ctx::kStageRing;
    if (ctx->stage_pending[slot]) HIP_TRY(hipEventSynchronize(ctx->stage_event[slot]));
  }
  char* pinned = ctx->stage + static_cast<size_t>(slot) * ctx->stage_slot_bytes;
  std::memcpy(pinned, src, bytes);
  HIP_TRY(hipMemcpyAsync(dst, pinned, bytes, hipMemcpyHostToDevice, s));
  if (!capturing) {
    HIP_TRY(hipEventRecord(ctx->stage_event[slot], s));
    ctx->stage_pending[slot] = true;
  }
  return MI355X_OK;
}

// One launch set of the sampling path.  Rows lie row_stride elements apart from `logits`, or -- row_ptrs not
// null, at most kInlineParamRows rows -- start at the device pointers row_ptrs[0 .. rows).
int SampleImpl(mi355x_search_ctx* ctx, hipStream_t s, const void* logits, const void* const* row_ptrs, int dtype,
               int64_t row_stride, int rows, int vocab, const mi355x_logits_xform* xf, mi355x_sample_params params,
               const mi355x_sample_params* per_row_params, const double* uniforms, int32_t* out_tokens,
               int32_t* kept_count, int32_t* kept_ids, float* kept_probs, int kept_capacity) {
  ms::SampleArgs a{};
  if (int r = MakeXform(ctx, xf, rows, vocab, s, &a.xf)) return r;
  bool any_nucleus = false, any_other = false, any_large_k = false, any_exact = false;
  const int chunks = (vocab + ms::kSChunk - 1) / ms::kSChunk;
  ms::InlineParams table{};
  bool use_table = false;
  auto check = [&](const mi355x_sample_params& p) -> int {
    if (!(p.temperature > 0.0f)) return Fail(MI355X_E_INVALID, "temperature must be positive (got %g)", p.temperature);
    // the kernels' own rule (row_mode) decides; these flags only have to cover it
    const int kk = p.k < vocab ? p.k : vocab;
    const bool fits = vocab > 64 && chunks * ms::kSmallCap <= ms::kAllCap;
    const bool whole = p.k <= 1 && !(p.p < 1.0f);  // no top-k and no nucleus: the whole vocabulary
    const bool nucleus = p.k <= 1 && !whole, large_k = p.k > 1 && kk > 64 && kk <= ms::kLargeKMax;
    if (nucleus && vocab > 64) any_nucleus = true;
    if (large_k && vocab > 64) any_large_k = true;
    if (vocab > 64 && (!fits || whole || (p.k > 1 && kk > ms::kLargeKMax))) any_exact = true;
    else if (!((nucleus || large_k) && fits)) any_other = true;
    return MI355X_OK;
  };
  if (per_row_params) {
    for (int r = 0; r < rows; ++r)
      if (int rc = check(per_row_params[r])) return rc;
  } else {
    if (int rc = check(params)) return rc;
  }
  if (row_ptrs || (per_row_params && rows <= ms::kInlineParamRows)) {
    for (int r = 0; r < rows; ++r) {
      table.row[r] = per_row_params ? per_row_params[r] : params;
      table.row_ptr[r] = row_ptrs ? row_ptrs[r] : nullptr;
    }
    use_table = true;
  } else if (per_row_params) {
    if (int rc = StageToDevice(ctx, s, ctx->params_dev, per_row_params, sizeof(mi355x_sample_params) * rows)) return rc;
    a.per_row = ctx->params_dev;
  }
  a.logits = row_ptrs ? row_ptrs[0] : logits;
  a.dtype = dtype;
  a.row_stride = row_stride;
  a.rows = rows;
  a.vocab = vocab;
  a.chunks = chunks;
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
  a.chunk_thr = ctx->chunk_thr;
  a.chunk_next = ctx->chunk_next;
  a.big = ctx->big;
  a.big2 = ctx->big2;
  a.big_stride = ctx->big_stride;
  a.fallback_rows = ctx->fallback_rows;
  a.poll_limit = ctx->poll_limit;
  a.row_done = ctx->row_done;
  a.exact_kernel = any_exact ? 1 : 0;
  // a caller that bounds the number of allowed ids per row lets the sparse-mask kernel work alone
  if (xf && xf->mask && xf->mask_allowed_max > 0) {
    const int hist = a.xf.history_lens ? a.xf.history_stride : a.xf.history_len;
    const int64_t listed = static_cast<int64_t>(xf->mask_allowed_max) + (a.xf.use_penalty() ? hist : 0) + 2;
    a.sparse_only = listed <= ms::kNucleusCap && hist <= 2048;  // (what the kernel can list; beyond, all three kernels)
  }
  HIP_TRY(ms_launch_sample(&a, use_table ? &table : nullptr, any_other, any_nucleus, any_large_k, s, &ctx->sides));
  return MI355X_OK;
}

int CheckSampleArgs(int dtype, const double* uniforms, const int32_t* out_tokens, const int32_t* kept_ids,
                    const float* kept_probs, int kept_capacity) {
  if (!uniforms || !out_tokens) return Fail(MI355X_E_INVALID, "null logits, uniforms or output");
  if (dtype != MI355X_F32 && dtype != MI355X_F16 && dtype != MI355X_BF16)
    return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if ((kept_ids || kept_probs) && kept_capacity <= 0) return Fail(MI355X_E_INVALID, "kept_capacity must be positive");
  if (kept_probs && !kept_ids) return Fail(MI355X_E_INVALID, "kept_probs requires kept_ids");
  return MI355X_OK;
}

}  // namespace

int mi355x_sample_typed(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                        int rows, int vocab, const mi355x_logits_xform* xf, mi355x_sample_params params,
                        const mi355x_sample_params* per_row_params, const double* uniforms, int32_t* out_tokens,
                        int32_t* kept_count, int32_t* kept_ids, float* kept_probs, int kept_capacity) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits) return Fail(MI355X_E_INVALID, "null logits, uniforms or output");
  if (int r = CheckSampleArgs(dtype, uniforms, out_tokens, kept_ids, kept_probs, kept_capacity)) return r;
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  return SampleImpl(ctx, static_cast<hipStream_t>(stream), logits, nullptr, dtype, row_stride, rows, vocab, xf, params,
                    per_row_params, uniforms, out_tokens, kept_count, kept_ids, kept_probs, kept_capacity);
}

int mi355x_sample_scattered(mi355x_search_ctx* ctx, void* stream, const void* const* row_ptrs, int dtype, int rows,
                            int vocab, const mi355x_logits_xform* xf, mi355x_sample_params params,
                            const mi355x_sample_params* per_row_params, const double* uniforms, int32_t* out_tokens,
                            int32_t* kept_count, int32_t* kept_ids, float* kept_probs, int kept_capacity) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!row_ptrs) return Fail(MI355X_E_INVALID, "null row pointer array");
  for (int r = 0; r < rows; ++r)
    if (!row_ptrs[r]) return Fail(MI355X_E_INVALID, "row %d has a null pointer", r);
  if (int r = CheckSampleArgs(dtype, uniforms, out_tokens, kept_ids, kept_probs, kept_capacity)) return r;
  const int words = (vocab - 1) / 32 + 1;
  // the row pointers travel inside the kernel arguments, kInlineParamRows rows per launch
  for (int r0 = 0; r0 < rows; r0 += ms::kInlineParamRows) {
    const int n = rows - r0 < ms::kInlineParamRows ? rows - r0 : ms::kInlineParamRows;
    mi355x_logits_xform part;
    if (xf) {
      part = *xf;
      if (part.mask) part.mask += static_cast<size_t>(r0) * words;
      if (part.history) part.history += static_cast<size_t>(r0) * part.history_stride;
      if (part.history_lens) part.history_lens += r0;
    }
    if (int rc = SampleImpl(ctx, static_cast<hipStream_t>(stream), nullptr, row_ptrs + r0, dtype, vocab, n, vocab,
                            xf ? &part : nullptr, params, per_row_params ? per_row_params + r0 : nullptr, uniforms + r0,
                            out_tokens + r0, kept_count ? kept_count + r0 : nullptr,
                            kept_ids ? kept_ids + static_cast<size_t>(r0) * kept_capacity : nullptr,
                            kept_probs ? kept_probs + static_cast<size_t>(r0) * kept_capacity : nullptr, kept_capacity))
      return rc;
  }
  return MI355X_OK;
}

int mi355x_topk_scores(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                       int rows, int vocab, int k, int32_t* out_tokens, float* out_scores) {
  if (int r = CheckRows(ctx, rows, vocab)) return r;
  if (!logits || !out_tokens || !out_scores) return Fail(MI355X_E_INVALID, "null logits or output");
  if (dtype != MI355X_F32 && dtype != MI355X_F16 && dtype != MI355X_BF16)
    return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if (k < 1 || k > vocab) return Fail(MI355X_E_INVALID, "k (%d) must be in [1, vocab]", k);
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // sixteen-bit rows are read as they are and widened in registers (DeviceInterface::TopKScores makes an fp32
  // copy first, src/cuda/interface.cpp:440-451); the scores returned are the widened values
  ms::SampleArgs a{};
  if (int r = MakeXform(ctx, nullptr, rows, vocab, s, &a.xf)) return r;
  a.logits = logits;
  a.dtype = dtype;
  a.row_stride = row_stride;
  a.rows = rows;
  a.vocab = vocab;
  a.chunks = (vocab + ms::kSChunk - 1) / ms::kSChunk;
  a.uniform = mi355x_sample_params{k, 0.0f, 1.0f};
  a.out_tokens = out_tokens;
  a.out_scores = out_scores;
  a.emit_topk = 1;
  a.cand_small = ctx->cand_small;
  a.chunk_cnt = ctx->chunk_cnt;
  a.chunk_max = ctx->chunk_max;
  a.chunk_thr = ctx->chunk_thr;
  a.chunk_next = ctx->chunk_next;
  a.big = ctx->big;
  a.big2 = ctx->big2;
  a.big_stride = ctx->big_stride;
  a.fallback_rows = ctx->fallback_rows;
  a.poll_limit = ctx->poll_limit;
  // up to 64: the fused kernel's sorted candidate lists; up to kLargeKMax: the candidate lists of the large-k
  // sampling route with an epilogue that emits instead of drawing; beyond (and for rows of more chunks than a
  // finishing workgroup ranks): the exact path's whole-row sort.  The kernels' own rule (row_mode) decides.
  const bool fits = vocab > 64 && a.chunks * ms::kSmallCap <= ms::kAllCap;
  const bool large_k = fits && k > 64 && k <= ms::kLargeKMax;
  const bool exact = vocab > 64 && (!fits || k > ms::kLargeKMax);
  a.exact_kernel = exact ? 1 : 0;
  HIP_TRY(ms_launch_sample(&a, nullptr, !large_k && !exact, false, large_k, s, nullptr));
  return MI355X_OK;
}

// Fills the argument block of the multi-workgroup sequential sum when the shape calls for it and the
// context's workspace covers it (the exponentials go to the key buffer of the sampling paths, which
// never run at the same time on one context).
static bool FillSeqSum(mi355x_search_ctx* ctx, const void* x, int64_t row_stride, int rows, int vocab, float inv_temp,
                       ms::SeqSumArgs* q) {
  const int segs = (vocab + ms::kSegElems - 1) / ms::kSegElems;
  if (vocab < ms::kSeqSumMinVocab || rows > ctx->max_rows || vocab > ctx->max_vocab || segs > ms::kMaxSegs) return false;
  q->x = x;
  q->row_stride = row_stride;
  q->rows = rows;
  q->vocab = vocab;
  q->segs = segs;
  q->inv_temp = inv_temp;
  q->seg_max = ctx->seg_max;
  q->seg_sum = ctx->seg_sum;
  q->seg_step = ctx->seg_step;
  q->sub_step = ctx->sub_step;
  q->sub_se = ctx->sub_se;
  q->e = reinterpret_cast<float*>(ctx->big);
  q->e_stride = ctx->big_stride * 2;
  q->out_max = ctx->row_max;
  q->out_sum = ctx->row_sum;
  q->poll_limit = ctx->poll_limit;
  q->gave_up = ctx->fallback_rows + 2;
  return true;
}

int mi355x_softmax(mi355x_search_ctx* ctx, void* stream, float* scores, int64_t row_stride, int rows, int vocab,
                   float temperature, int log_softmax) {
  if (!ctx) return Fail(MI355X_E_INVALID, "null context");
  if (!scores || rows <= 0 || vocab <= 0) return Fail(MI355X_E_INVALID, "null scores or non-positive size");
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  if (!(temperature > 0.0f)) return Fail(MI355X_E_INVALID, "temperature must be positive (got %g)", temperature);
  hipStream_t s = static_cast<hipStream_t>(stream);
  ms::SeqSumArgs q{};
  if (FillSeqSum(ctx, scores, row_stride, rows, vocab, 1.0f / temperature, &q)) {
    // long rows: the exact sum is spread over the whole GPU, then an element-wise pass finishes
    HIP_TRY(ms_launch_seqsum(&q, MI355X_F32, s));
    HIP_TRY(ms_launch_softmax_apply(scores, row_stride, &q, log_softmax, s));
  } else {
    HIP_TRY(ms_launch_softmax(scores, row_stride, rows, vocab, temperature, log_softmax, s));
  }
  return MI355X_OK;
}

namespace {
// mi355x_beam_select; with `step`, the launch that finishes the selection also does the scorer step where the
// path taken has such a launch (*fused says whether it did).
int BeamSelectImpl(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                   int batch, int beams, int vocab, const float* beam_scores, float* out_scores,
                   int32_t* out_tokens, int32_t* out_beam_indices, const ms::ScorerStep* step, bool* fused) {
  if (batch <= 0 || beams <= 0) return Fail(MI355X_E_INVALID, "batch and beams must be positive");
  if (beams > ms::kBeamMaxCand / 2) return Fail(MI355X_E_UNSUPPORTED, "beams (%d) above the supported %d", beams, ms::kBeamMaxCand / 2);
  if (int r = CheckRows(ctx, batch * beams, vocab)) return r;
  if (!logits || !beam_scores || !out_scores || !out_tokens || !out_beam_indices)
    return Fail(MI355X_E_INVALID, "null argument");
  if (dtype != MI355X_F32 && dtype != MI355X_F16 && dtype != MI355X_BF16)
    return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if (row_stride < vocab) return Fail(MI355X_E_INVALID, "row_stride smaller than vocab");
  if (static_cast<long long>(beams) * vocab < 2LL * beams)
    return Fail(MI355X_E_INVALID, "beam search requires num_beams * vocab_size (%lld) >= 2 * num_beams (%d)",
                static_cast<long long>(beams) * vocab, 2 * beams);
  if (static_cast<unsigned long long>(beams) * static_cast<unsigned long long>(vocab) > 0xffffffffull)
    return Fail(MI355X_E_UNSUPPORTED, "beams * vocab exceeds 2^32");
  ms::BeamArgs a{};
  a.logits = logits;
  a.row_stride = row_stride;
  a.batch = batch;
  a.beams = beams;
  a.vocab = vocab;
  a.beam_scores = beam_scores;
  a.row_scores = ctx->beam_row_scores;
  a.row_tokens = ctx->beam_row_tokens;
  a.out_scores = out_scores;
  a.out_tokens = out_tokens;
  a.out_beams = out_beam_indices;
  ms::SeqSumArgs q{};
  if (FillSeqSum(ctx, logits, row_stride, batch * beams, vocab, 1.0f, &q)) {
    a.row_max = q.out_max;
    a.row_sum = q.out_sum;
    if (static_cast<long long>(beams) * q.segs * 2 * beams <= ms::kBeamFinCap) {
      // long rows: the segments list their best logits inside the launch that writes their exponentials, the
      // exact sums follow, and one workgroup per batch entry scores the listed candidates
      a.seg_cand = ctx->seg_cand;
      a.seg_max = q.seg_max;
      a.segs = q.segs;
      HIP_TRY(ms_launch_seqsum_max(&q, dtype, static_cast<hipStream_t>(stream)));
      HIP_TRY(ms_launch_beam_exp_step(&q, &a, dtype, static_cast<hipStream_t>(stream)));
      HIP_TRY(ms_launch_seqsum_walk(&q, static_cast<hipStream_t>(stream)));
      HIP_TRY(ms_launch_beam_finish(&a, dtype, step, static_cast<hipStream_t>(stream)));
      if (fused) *fused = step != nullptr;
      return MI355X_OK;
    }
    HIP_TRY(ms_launch_seqsum(&q, dtype, static_cast<hipStream_t>(stream)));
  }
  HIP_TRY(ms_launch_beam_select(&a, dtype, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}
}  // namespace

int mi355x_beam_select(mi355x_search_ctx* ctx, void* stream, const void* logits, int dtype, int64_t row_stride,
                       int batch, int beams, int vocab, const float* beam_scores, float* out_scores,
                       int32_t* out_tokens, int32_t* out_beam_indices) {
  return BeamSelectImpl(ctx, stream, logits, dtype, row_stride, batch, beams, vocab, beam_scores, out_scores, out_tokens,
                        out_beam_indices, nullptr, nullptr);
}

int mi355x_spec_verify_sparse(mi355x_search_ctx* ctx, void* stream, const int32_t* target_count,
                              const int32_t* target_ids, const float* target_probs, int target_capacity,
                              const int32_t* draft_count, const int32_t* draft_ids, const float* draft_probs,
                              int draft_capacity, const int32_t* proposal, const float* accept_u,
                              const double* sample_u, int batch, int K, int mode, int32_t* accepted_len,
                              int32_t* final_token, int32_t* engine_draws) {
  if (!ctx || !target_count || !target_ids || !proposal || !accepted_len || !final_token || !engine_draws)
    return Fail(MI355X_E_INVALID, "null argument");
  if (mode < 0 || mode > 2) return Fail(MI355X_E_INVALID, "mode (%d) must be 0, 1 or 2", mode);
  if (batch <= 0 || K < 1 || K > 64) return Fail(MI355X_E_INVALID, "batch (%d) must be positive and K (%d) in [1, 64]", batch, K);
  if (target_capacity <= 0) return Fail(MI355X_E_INVALID, "target_capacity must be positive");
  if (mode != 2 && (!target_probs || !sample_u)) return Fail(MI355X_E_INVALID, "null target_probs or sample_u");
  if (mode == 0 && (!draft_count || !draft_ids || !draft_probs || !accept_u || draft_capacity <= 0))
    return Fail(MI355X_E_INVALID, "mode 0 needs the draft distributions and accept_u");
  if (batch > ctx->max_rows) return Fail(MI355X_E_CAPACITY, "batch=%d exceeds the context's capacity (%d)", batch, ctx->max_rows);
  if (static_cast<size_t>(target_capacity) > 2 * ctx->big_stride)
    return Fail(MI355X_E_CAPACITY, "target_capacity=%d exceeds the context's workspace (%zu)", target_capacity, 2 * ctx->big_stride);
  ms::SpecSparseArgs a{};
  a.t_count = target_count;
  a.t_ids = target_ids;
  a.t_probs = target_probs;
  a.t_cap = target_capacity;
  a.d_count = draft_count;
  a.d_ids = draft_ids;
  a.d_probs = draft_probs;
  a.d_cap = draft_capacity;
  a.proposal = proposal;
  a.accept_u = accept_u;
  a.sample_u = sample_u;
  a.K = K;
  a.mode = mode;
  a.residual = reinterpret_cast<float*>(ctx->big);
  a.residual_stride = 2 * ctx->big_stride;
  a.accepted_len = accepted_len;
  a.final_token = final_token;
  a.engine_draws = engine_draws;
  HIP_TRY(ms_launch_spec_verify_sparse(&a, batch, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_draw_in_order(mi355x_search_ctx* ctx, void* stream, const int32_t* kept_count, const int32_t* kept_ids,
                         const float* kept_probs, int kept_capacity, int rows, const int32_t* skip_rows,
                         const double* uniform_pool, int32_t* out_tokens, int32_t* draws_used) {
  if (!ctx || !kept_count || !kept_ids || !kept_probs || !uniform_pool || !out_tokens)
    return Fail(MI355X_E_INVALID, "null argument");
  if (rows <= 0 || kept_capacity <= 0) return Fail(MI355X_E_INVALID, "rows and kept_capacity must be positive");
  HIP_TRY(ms_launch_draw_in_order(kept_count, kept_ids, kept_probs, kept_capacity, rows, skip_rows, uniform_pool, out_tokens,
                                  draws_used, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_greedy_tail(mi355x_search_ctx* ctx, void* stream, int32_t* next_tokens, int32_t* eos_seen, int batch,
                       const int32_t* eos_ids, int n_eos, int32_t pad_token_id, int32_t* sequences, int max_length,
                       int current_length, int32_t* done) {
  if (!ctx || !next_tokens || !eos_seen || !sequences || !done) return Fail(MI355X_E_INVALID, "null argument");
  if (batch <= 0 || max_length <= 0 || current_length < 0)
    return Fail(MI355X_E_INVALID, "batch (%d) and max_length (%d) must be positive, current_length (%d) not negative",
                batch, max_length, current_length);
  if (n_eos < 0 || n_eos > MI355X_MAX_EOS || (n_eos > 0 && !eos_ids))
    return Fail(MI355X_E_INVALID, "n_eos (%d) out of range [0, %d] or null eos_ids", n_eos, MI355X_MAX_EOS);
  HIP_TRY(ms_launch_greedy_tail(next_tokens, eos_seen, batch, eos_ids, n_eos, pad_token_id, sequences, max_length,
                                current_length, done, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_cast(mi355x_search_ctx* ctx, void* stream, const void* in, int in_dtype, void* out, int out_dtype,
                size_t count) {
  if (!ctx || !in || !out) return Fail(MI355X_E_INVALID, "null argument");
  if (in_dtype == out_dtype) return Fail(MI355X_E_INVALID, "Cast - input and output types are the same");
  int kind = -1;
  if (in_dtype == MI355X_F16 && out_dtype == MI355X_F32) kind = 0;
  else if (in_dtype == MI355X_BF16 && out_dtype == MI355X_F32) kind = 1;
  else if (in_dtype == MI355X_F32 && out_dtype == MI355X_F16) kind = 2;
  else if (in_dtype == MI355X_F32 && out_dtype == MI355X_BF16) kind = 3;
  else if (in_dtype == MI355X_I32 && out_dtype == MI355X_I64) kind = 4;
  if (kind < 0) return Fail(MI355X_E_UNSUPPORTED, "cast from type %d to type %d is not implemented", in_dtype, out_dtype);
  if (count == 0) return MI355X_OK;
  HIP_TRY(ms_launch_cast(in, out, count, kind, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_logits_handoff(mi355x_search_ctx* ctx, void* stream, const void* raw, int dtype, int rows, int seq_len,
                          int vocab, const int32_t* token_index, float* out, int64_t out_stride) {
  if (!ctx || !raw || !out) return Fail(MI355X_E_INVALID, "null argument");
  if (rows <= 0 || seq_len <= 0 || vocab <= 0) return Fail(MI355X_E_INVALID, "non-positive size");
  if (out_stride < vocab) return Fail(MI355X_E_INVALID, "out_stride smaller than vocab");
  if (rows > 65535) return Fail(MI355X_E_CAPACITY, "too many rows (%d)", rows);
  const int kind = dtype == MI355X_F16 ? 0 : dtype == MI355X_BF16 ? 1 : dtype == MI355X_F32 ? 2 : -1;
  if (kind < 0) return Fail(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int32_t* index_dev = nullptr;
  if (token_index) {
    if (rows > ctx->max_rows) return Fail(MI355X_E_CAPACITY, "rows (%d) exceed the context's %d", rows, ctx->max_rows);
    for (int r = 0; r < rows; ++r)
      if (token_index[r] < 0 || token_index[r] >= seq_len)
        return Fail(MI355X_E_INVALID, "token_index[%d] = %d outside [0, %d)", r, token_index[r], seq_len);
    if (int rc = StageToDevice(ctx, s, ctx->row_index, token_index, sizeof(int32_t) * rows)) return rc;
    index_dev = ctx->row_index;
  }
  HIP_TRY(ms_launch_logits_handoff(raw, kind, rows, seq_len, vocab, index_dev, out, out_stride, s));
  return MI355X_OK;
}

int mi355x_kv_gather(mi355x_search_ctx* ctx, void* stream, const void* const* present, void* const* past,
                     int n_tensors, const int32_t* beam_indices, int rows, size_t block_bytes) {
  if (!ctx || !present || !past || !beam_indices) return Fail(MI355X_E_INVALID, "null argument");
  if (n_tensors <= 0 || rows <= 0 || block_bytes == 0) return Fail(MI355X_E_INVALID, "non-positive size");
  if (static_cast<size_t>(n_tensors) * 2 > ctx->ptr_table_cap || n_tensors > 65535 || rows > 65535)
    return Fail(MI355X_E_CAPACITY, "too many tensors (%d) or rows (%d)", n_tensors, rows);
  // Widest power-of-two access (at most 16 bytes) that every block of every tensor is aligned to.
  uintptr_t align = static_cast<uintptr_t>(block_bytes);
  for (int t = 0; t < n_tensors; ++t) {
    if (!present[t] || !past[t]) return Fail(MI355X_E_INVALID, "null tensor pointer at %d", t);
    align |= reinterpret_cast<uintptr_t>(present[t]) | reinterpret_cast<uintptr_t>(past[t]);
  }
  int width = 16;
  while (align & static_cast<uintptr_t>(width - 1)) width >>= 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  {
    std::vector<const void*> both(static_cast<size_t>(n_tensors) * 2);  // one table: present pointers, then past pointers
    std::copy_n(present, n_tensors, both.begin());
    std::copy_n(past, n_tensors, both.begin() + n_tensors);
    if (int rc = StageToDevice(ctx, s, ctx->ptr_table, both.data(), sizeof(void*) * both.size())) return rc;
  }
  HIP_TRY(ms_launch_kv_gather(ctx->ptr_table, ctx->ptr_table + n_tensors, n_tensors, beam_indices, rows, block_bytes, width, s));
  return MI355X_OK;
}

int mi355x_spec_verify(mi355x_search_ctx* ctx, void* stream, const float* p_target, const float* p_draft,
                       const int32_t* draft_tokens, const float* accept_u, const double* sample_u, int batch, int K,
                       int vocab, int32_t* accepted_len, int32_t* final_token) {
  if (!ctx || !p_target || !p_draft || !draft_tokens || !accept_u || !sample_u || !accepted_len || !final_token)
    return Fail(MI355X_E_INVALID, "null argument");
  if (batch <= 0 || K <= 0 || vocab < 2) return Fail(MI355X_E_INVALID, "batch, K must be positive and vocab >= 2");
  HIP_TRY(ms_launch_spec_verify(p_target, p_draft, draft_tokens, accept_u, sample_u, batch, K, vocab, accepted_len,
                                final_token, static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_search_fallback_rows(mi355x_search_ctx* ctx, void* stream, unsigned* rows) {
  if (!ctx || !rows) return Fail(MI355X_E_INVALID, "null argument");
  HIP_TRY(hipMemcpyAsync(rows, ctx->fallback_rows, sizeof(unsigned), hipMemcpyDeviceToHost,
                         static_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_search_wait_gave_up(mi355x_search_ctx* ctx, void* stream, int* gave_up) {
  if (!ctx || !gave_up) return Fail(MI355X_E_INVALID, "null argument");
  unsigned word = 0;
  HIP_TRY(hipMemcpyAsync(&word, ctx->fallback_rows + 1, sizeof(unsigned), hipMemcpyDeviceToHost,
                         static_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  *gave_up = word != 0u;
  return MI355X_OK;
}

int mi355x_search_sum_waits_gave_up(mi355x_search_ctx* ctx, void* stream, unsigned* segments) {
  if (!ctx || !segments) return Fail(MI355X_E_INVALID, "null argument");
  HIP_TRY(hipMemcpyAsync(segments, ctx->fallback_rows + 2, sizeof(unsigned), hipMemcpyDeviceToHost,
                         static_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return MI355X_OK;
}

int mi355x_search_set_poll_limit(mi355x_search_ctx* ctx, int polls) {
  if (!ctx) return Fail(MI355X_E_INVALID, "null context");
  if (polls < 0) return Fail(MI355X_E_INVALID, "negative poll limit");
  ctx->poll_limit = polls;
  return MI355X_OK;
}

// ---- device-resident beam scorer ---------------------------------------------------------------------
struct mi355x_beam_scorer {
  mi355x_search_ctx* ctx{};
  ms::ScorerState st{};
  std::vector<void*> allocs;
  int32_t* seq[2]{};
  int cur{};
  int length{};
  bool finalized{};
  float* pow_dev{};
  float* cand_scores{};    // [batch, 2*beams]: the candidates of mi355x_beam_search_step
  int32_t* cand_tokens{};
  int32_t* cand_beams{};
};

int mi355x_beam_scorer_create(mi355x_search_ctx* ctx, int batch, int beams, int max_length, int pad_token_id,
                              const int32_t* eos_ids, int n_eos, float length_penalty, int early_stopping,
                              mi355x_beam_scorer** out) {
  if (!ctx || !out) return Fail(MI355X_E_INVALID, "null argument");
  *out = nullptr;
  if (batch <= 0 || beams <= 1 || max_length <= 0) return Fail(MI355X_E_INVALID, "batch, max_length must be positive and beams > 1");
  if (beams > ms::kBeamMaxCand / 2) return Fail(MI355X_E_UNSUPPORTED, "beams (%d) above the supported %d", beams, ms::kBeamMaxCand / 2);
  if (n_eos < 0 || n_eos > MI355X_MAX_EOS || (n_eos > 0 && !eos_ids)) return Fail(MI355X_E_INVALID, "bad eos list");
  HIP_TRY(hipSetDevice(ctx->device));
  auto* s = new (std::nothrow) mi355x_beam_scorer;
  if (!s) return Fail(MI355X_E_INVALID, "out of host memory");
  s->ctx = ctx;
  const size_t bb = static_cast<size_t>(batch) * beams;
  hipError_t e = hipSuccess;
  auto alloc = [&](void** p, size_t bytes) {
    if (e != hipSuccess) return;
    e = hipMalloc(p, bytes ? bytes : 16);
    if (e == hipSuccess) {
      s->allocs.push_back(*p);
      e = hipMemset(*p, 0, bytes ? bytes : 16);
    }
  };
  ms::ScorerState& st = s->st;
  st.batch = batch;
  st.beams = beams;
  st.max_length = max_length;
  st.pad = pad_token_id;
  st.early_stopping = early_stopping != 0;
  st.n_eos = n_eos;
  for (int i = 0; i < n_eos; ++i) st.eos[i] = eos_ids[i];
  alloc(reinterpret_cast<void**>(&st.next_scores), bb * sizeof(float));
  alloc(reinterpret_cast<void**>(&st.next_tokens), bb * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&st.next_indices), bb * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&st.hyp_score), bb * sizeof(float));
  alloc(reinterpret_cast<void**>(&st.hyp_len), bb * sizeof(int));
  alloc(reinterpret_cast<void**>(&st.hyp_slot), static_cast<size_t>(batch) * (beams + 1) * sizeof(int));
  alloc(reinterpret_cast<void**>(&st.hyp_tokens), static_cast<size_t>(batch) * (beams + 1) * max_length * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&st.hyp_used), batch * sizeof(int));
  alloc(reinterpret_cast<void**>(&st.done), batch * sizeof(int));
  alloc(reinterpret_cast<void**>(&st.not_done), sizeof(int));
  alloc(reinterpret_cast<void**>(&st.pending), batch * sizeof(int));
  alloc(reinterpret_cast<void**>(&st.arrive), sizeof(unsigned));
  alloc(reinterpret_cast<void**>(&s->pow_dev), (static_cast<size_t>(max_length) + 1) * sizeof(float));
  alloc(reinterpret_cast<void**>(&s->seq[0]), bb * max_length * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&s->seq[1]), bb * max_length * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&s->cand_scores), 2 * bb * sizeof(float));
  alloc(reinterpret_cast<void**>(&s->cand_tokens), 2 * bb * sizeof(int32_t));
  alloc(reinterpret_cast<void**>(&s->cand_beams), 2 * bb * sizeof(int32_t));
  if (e == hipSuccess) {
    // initial beam scores 0, -1e9, -1e9, ... per batch entry (src/beam_search_scorer.cpp:76-81); rank -> row
    // identity; pow(length, length_penalty) from the host libm, the function the reference calls.
    std::vector<float> init(bb, 0.0f), powt(static_cast<size_t>(max_length) + 1);
    for (int b = 0; b < batch; ++b)
      for (int j = 1; j < beams; ++j) init[static_cast<size_t>(b) * beams + j] = -1e9;
    std::vector<int> slots(static_cast<size_t>(batch) * (beams + 1));
    for (size_t i = 0; i < slots.size(); ++i) slots[i] = static_cast<int>(i % (beams + 1));
    for (int l = 0; l <= max_length; ++l) powt[l] = std::pow(static_cast<float>(l), length_penalty);
    e = hipMemcpy(st.next_scores, init.data(), bb * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(st.hyp_slot, slots.data(), slots.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(s->pow_dev, powt.data(), powt.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(st.not_done, &batch, sizeof(int), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);  // the fills are done before any stream uses the state
    st.pow_table = s->pow_dev;
  }
  if (e != hipSuccess) {
    mi355x_beam_scorer_destroy(s);
    return Fail(MI355X_E_HIP, "beam scorer allocation failed: %s", hipGetErrorString(e));
  }
  *out = s;
  return MI355X_OK;
}

void mi355x_beam_scorer_destroy(mi355x_beam_scorer* s) {
  if (!s) return;
  for (void* p : s->allocs) (void)hipFree(p);
  delete s;
}

int mi355x_beam_scorer_set_prompt(mi355x_beam_scorer* s, void* stream, const int32_t* tokens, int prompt_len) {
  if (!s || !tokens) return Fail(MI355X_E_INVALID, "null argument");
  if (prompt_len < 0 || prompt_len > s->st.max_length) return Fail(MI355X_E_INVALID, "User-defined tokens exceed max_length.");
  const int bb = s->st.batch * s->st.beams;
  std::vector<int32_t> host(static_cast<size_t>(bb) * s->st.max_length, 0);
  for (int i = 0; i < bb; ++i)
    std::memcpy(host.data() + static_cast<size_t>(i) * s->st.max_length,
                tokens + static_cast<size_t>(i / s->st.beams) * prompt_len, sizeof(int32_t) * prompt_len);
  hipStream_t st = static_cast<hipStream_t>(stream);
  HIP_TRY(hipMemcpyAsync(s->seq[s->cur], host.data(), host.size() * sizeof(int32_t), hipMemcpyHostToDevice, st));
  HIP_TRY(hipStreamSynchronize(st));  // `host` goes out of scope
  s->length = prompt_len;
  return MI355X_OK;
}

int mi355x_beam_scorer_step(mi355x_beam_scorer* s, void* stream, const float* cand_scores, const int32_t* cand_tokens,
                            const int32_t* cand_beam_indices) {
  if (!s || !cand_scores || !cand_tokens || !cand_beam_indices) return Fail(MI355X_E_INVALID, "null argument");
  if (s->length >= s->st.max_length) return Fail(MI355X_E_INVALID, "sequence already at max_length (%d)", s->st.max_length);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (Capturing(st))
    return Fail(MI355X_E_UNSUPPORTED, "a scorer step carries the sequence length and buffer of this very step: a graph replay would repeat it");
  HIP_TRY(ms_launch_scorer_step(&s->st, s->seq[s->cur], s->seq[1 - s->cur], s->length, cand_scores, cand_tokens,
                                cand_beam_indices, st));
  s->cur = 1 - s->cur;
  s->length += 1;
  return MI355X_OK;
}

int mi355x_beam_search_step(mi355x_beam_scorer* s, void* stream, const void* logits, int dtype, int64_t row_stride,
                            int vocab) {
  if (!s) return Fail(MI355X_E_INVALID, "null argument");
  if (s->length >= s->st.max_length) return Fail(MI355X_E_INVALID, "sequence already at max_length (%d)", s->st.max_length);
  if (Capturing(static_cast<hipStream_t>(stream)))
    return Fail(MI355X_E_UNSUPPORTED, "a search step carries the sequence length and buffer of this very step: a graph replay would repeat it");
  ms::ScorerStep step{s->st, s->seq[s->cur], s->seq[1 - s->cur], s->length};
  bool fused = false;
  if (int r = BeamSelectImpl(s->ctx, stream, logits, dtype, row_stride, s->st.batch, s->st.beams, vocab, s->st.next_scores,
                             s->cand_scores, s->cand_tokens, s->cand_beams, &step, &fused))
    return r;
  if (!fused) return mi355x_beam_scorer_step(s, stream, s->cand_scores, s->cand_tokens, s->cand_beams);
  s->cur = 1 - s->cur;
  s->length += 1;
  return MI355X_OK;
}

const float* mi355x_beam_scorer_next_scores(const mi355x_beam_scorer* s) { return s ? s->st.next_scores : nullptr; }
const int32_t* mi355x_beam_scorer_next_tokens(const mi355x_beam_scorer* s) { return s ? s->st.next_tokens : nullptr; }
const int32_t* mi355x_beam_scorer_next_indices(const mi355x_beam_scorer* s) { return s ? s->st.next_indices : nullptr; }
const int32_t* mi355x_beam_scorer_sequences(const mi355x_beam_scorer* s, int* length) {
  if (!s) return nullptr;
  if (length) *length = s->length;
  return s->seq[s->cur];
}

int mi355x_beam_scorer_is_done(mi355x_beam_scorer* s, void* stream, int* done) {
  if (!s || !done) return Fail(MI355X_E_INVALID, "null argument");
  int nd = 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  HIP_TRY(hipMemcpyAsync(&nd, s->st.not_done, sizeof(int), hipMemcpyDeviceToHost, st));
  HIP_TRY(hipStreamSynchronize(st));
  *done = (nd == 0) || (s->length == s->st.max_length);  // BeamSearch_Cpu::IsDone, src/search.cpp:345-352
  return MI355X_OK;
}

int mi355x_beam_scorer_hypothesis(mi355x_beam_scorer* s, void* stream, int batch, int index, int32_t* out, int capacity,
                                  int* length, float* score) {
  if (!s || !out || !length) return Fail(MI355X_E_INVALID, "null argument");
  if (batch < 0 || batch >= s->st.batch) return Fail(MI355X_E_INVALID, "batch index out of range");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!s->finalized) {
    HIP_TRY(ms_launch_scorer_finalize(&s->st, s->seq[s->cur], s->length, st));
    s->finalized = true;
  }
  const int nb = s->st.beams;
  int used = 0;
  HIP_TRY(hipMemcpyAsync(&used, s->st.hyp_used + batch, sizeof(int), hipMemcpyDeviceToHost, st));
  HIP_TRY(hipStreamSynchronize(st));
  if (index < 0 || index >= used) return Fail(MI355X_E_INVALID, "GetHypothesis index out of bounds");
  int len = 0, slot = 0;
  float sc = 0.0f;
  HIP_TRY(hipMemcpy(&len, s->st.hyp_len + batch * nb + index, sizeof(int), hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(&slot, s->st.hyp_slot + batch * (nb + 1) + index, sizeof(int), hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(&sc, s->st.hyp_score + batch * nb + index, sizeof(float), hipMemcpyDeviceToHost));
  const int n = len < capacity ? len : capacity;
  HIP_TRY(hipMemcpy(out, s->st.hyp_tokens + (static_cast<size_t>(batch) * (nb + 1) + slot) * s->st.max_length,
                    sizeof(int32_t) * n, hipMemcpyDeviceToHost));
  *length = len;
  if (score) *score = sc;
  return MI355X_OK;
}

}  // extern "C"
