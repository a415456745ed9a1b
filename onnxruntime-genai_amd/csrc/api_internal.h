// Pieces of the host side of the C ABI that more than one source file uses.
#pragma once
#include <cstdarg>
#include "kernels.h"
#include "mi355x_search.h"

// Stores the formatted message as the calling thread's last error and returns `code`.
int ms_vfail(int code, const char* fmt, va_list ap);
// Validates a caller's logits-processing request and turns it into the kernels' form (launches the
// n-gram bitmap kernel into the context's workspace when that rule is on; ctx may be null otherwise).
int ms_make_xform(mi355x_search_ctx* ctx, const mi355x_logits_xform* in, int rows, int vocab, hipStream_t stream,
                  ms::Xform* out);
// Resolves, for the current device, the address of the static scratch behind mi355x_argmax_static.
extern "C" hipError_t ms_static_scratch_setup();
