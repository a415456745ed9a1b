// mi355x_argmax_static: the greedy argmax of mi355x_argmax for callers that cannot allocate (code
// under HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It needs no context:
// the per-row partial results of the chunked kernel (running best key and arrival counter of every
// row) live in a file-scope device array that each GPU holds from library load until the process ends.
#include <mutex>
#include "api_internal.h"

namespace {

constexpr int kStaticMaxRows = MI355X_ARGMAX_STATIC_MAX_ROWS;
constexpr int kMaxDevices = 64;

// [0, kStaticMaxRows) 64-bit words: a row's best key so far; the 32-bit arrival counters follow.
static __device__ __align__(256) unsigned long long scratch[kStaticMaxRows + kStaticMaxRows / 2];

// In host code `scratch` only names the symbol; each device's copy has its own address, looked up once.
std::mutex g_mu;
void* g_scratch_ptr[kMaxDevices];

int FailHere(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  ms_vfail(code, fmt, ap);
  va_end(ap);
  return code;
}

// The array's address on the calling thread's current device; looked up on first use unless `lookup_allowed` is
// false (then an unknown address reports hipErrorNotReady).
hipError_t ScratchOfCurrentDevice(void** out, bool lookup_allowed = true) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_scratch_ptr[device]) {
    if (!lookup_allowed) return hipErrorNotReady;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_scratch_ptr[device] = p;
  }
  if (out) *out = g_scratch_ptr[device];
  return hipSuccess;
}

// The chunked kernel expects zeroed slots and leaves them zeroed, but the array outlives every call,
// including one whose launch failed half-way: the rows about to be used are cleared first (a kernel
// rather than a memset node, so the call can sit in a captured graph).
__global__ void static_clear_kernel(ms::u64* row_best, uint32_t* row_arrive, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) {
    row_best[i] = 0;
    row_arrive[i] = 0u;
  }
}

}  // namespace

extern "C" hipError_t ms_static_scratch_setup() { return ScratchOfCurrentDevice(nullptr); }

extern "C" int mi355x_argmax_static(void* stream, const void* logits, int dtype, int64_t row_stride, int rows,
                                    int vocab, const mi355x_logits_xform* xf, int32_t* out_tokens) {
  if (rows <= 0 || vocab <= 0) return FailHere(MI355X_E_INVALID, "rows (%d) and vocab (%d) must be positive", rows, vocab);
  if (rows > kStaticMaxRows)
    return FailHere(MI355X_E_CAPACITY, "rows (%d) exceed the %d rows the static scratch holds; use mi355x_argmax", rows,
                    kStaticMaxRows);
  if (!logits || !out_tokens) return FailHere(MI355X_E_INVALID, "null logits or output");
  if (dtype != MI355X_F32 && dtype != MI355X_F16 && dtype != MI355X_BF16)
    return FailHere(MI355X_E_UNSUPPORTED, "dtype %d not supported", dtype);
  if (row_stride < vocab) return FailHere(MI355X_E_INVALID, "row_stride smaller than vocab");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // every GPU has its own copy of the array: the stream must belong to the device whose copy is used
  int current = 0, of_stream = 0;
  if (s != nullptr && hipGetDevice(&current) == hipSuccess && hipStreamGetDevice(s, &of_stream) == hipSuccess &&
      of_stream != current)
    return FailHere(MI355X_E_INVALID, "the stream belongs to device %d, the calling thread's current device is %d", of_stream,
                    current);
  ms::ArgmaxArgs a{};
  if (int r = ms_make_xform(nullptr, xf, rows, vocab, s, &a.xf)) return r;
  // the first use on a device looks the array's address up, which is no work for a stream that records a graph
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  const bool capturing = hipStreamIsCapturing(s, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
  void* base = nullptr;
  hipError_t e = ScratchOfCurrentDevice(&base, !capturing);
  if (e == hipErrorNotReady)
    return FailHere(MI355X_E_UNSUPPORTED, "the first call on a device cannot be captured into a graph: call once outside "
                    "the capture (or create a context on the device) first");
  if (e != hipSuccess) return FailHere(MI355X_E_HIP, "static scratch lookup failed: %s", hipGetErrorString(e));
  a.logits = logits;
  a.row_stride = row_stride;
  a.rows = rows;
  a.vocab = vocab;
  a.chunks = (vocab + ms::kChunk - 1) / ms::kChunk;
  a.out_tokens = out_tokens;
  a.row_best = static_cast<ms::u64*>(base);
  a.row_arrive = reinterpret_cast<uint32_t*>(static_cast<ms::u64*>(base) + kStaticMaxRows);
  hipLaunchKernelGGL(static_clear_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, a.row_best, a.row_arrive, rows);
  e = hipGetLastError();
  if (e == hipSuccess) e = ms_launch_argmax(&a, dtype, s);
  if (e != hipSuccess) return FailHere(MI355X_E_HIP, "argmax launch failed: %s", hipGetErrorString(e));
  return MI355X_OK;
}
