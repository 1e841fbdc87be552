// temporary
#include "dispatch.hip.h"
extern "C" size_t fa_seghist_scratch_bytes(fa_dtype, int64_t) { return 4; }
extern "C" int fa_seghist(fa_stream_t, fa_dtype, fa_op, const void *, int, const void *, int64_t, void *, int64_t, void *, size_t) { return FA_ENOTSUP; }
extern "C" size_t fa_radix_sort_scratch_bytes(int64_t) { return 4; }
extern "C" int fa_radix_sort(fa_stream_t, int, int, const void *, void *, void *, const void *, void *, void *, int64_t, int, int, void *, size_t) { return FA_ENOTSUP; }
extern "C" int fa_matmul(fa_stream_t, fa_dtype, const void *, const void *, float *, int64_t, int64_t, int64_t, int64_t) { return FA_ENOTSUP; }
