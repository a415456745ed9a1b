// The streaming kernels of the sampling path for fp16 logits (widened in registers as the reference's
// FastFloat16ToFloat32 does, src/models/utils.cpp:103-109).
#include "sample_stream.h"

MS_STREAM_KERNELS(_f16, uint16_t)
