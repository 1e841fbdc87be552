// placeholder until the MFMA kernels land
#include "dispatch.hip.h"
extern "C" int fa_matmul(fa_stream_t, fa_dtype, const void *, const void *, float *, int64_t, int64_t, int64_t, int64_t) { return FA_ENOTSUP; }
