// The streaming kernels of the sampling path for bfloat16 logits (widened in registers as the reference's
// BFloat16ToFloat32 does, src/models/utils.cpp:84-86).
#include "sample_stream.h"

MS_STREAM_KERNELS(_bf16, ms::bf16_t)
