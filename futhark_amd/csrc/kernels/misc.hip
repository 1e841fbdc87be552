// Builtin data-movement kernels: replicate, iota, copy and the batched 2-D
// copy.  They stand where the reference keeps builtin#replicate_* /
// builtin#iota_* (src/Futhark/CodeGen/ImpGen/GPU/Base.hs:1274-1436).
#include "dispatch.hip.h"

namespace fa {

template <class T>
__global__ __launch_bounds__(256) void replicate_kernel(T *dst, int64_t n, T v) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = v;
}

template <class T>
__global__ __launch_bounds__(256) void iota_kernel(T *dst, int64_t n, T start, T step) {
  using U = typename std::make_unsigned<T>::type;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
    dst[i] = (T)((U)start + (U)i * (U)step);
}

// 16 bytes per lane per access, four accesses in flight.
__global__ __launch_bounds__(256) void copy_kernel(uint4 *__restrict__ dst,
                                                   const uint4 *__restrict__ src, int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 3 * stride < nvec; i += 4 * stride) {
    uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    dst[i] = a;
    dst[i + stride] = b;
    dst[i + 2 * stride] = c;
    dst[i + 3 * stride] = d;
  }
  for (; i < nvec; i += stride) dst[i] = src[i];
}

__global__ void copy_tail_kernel(uint8_t *dst, const uint8_t *src, int64_t from, int64_t n) {
  const int64_t i = from + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

static int grid_for(int64_t n, int per_block) {
  int64_t g = ceil_div(n, per_block);
  if (g < 1) g = 1;
  if (g > 256 * 16) g = 256 * 16;
  return (int)g;
}

}  // namespace fa

extern "C" int fa_replicate(fa_stream_t stream, int elem_bytes, void *dst, int64_t n,
                            uint64_t pattern) {
  if (n < 0 || (n > 0 && dst == nullptr)) return FA_EINVAL;
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int g = grid_for(n, 256 * 4);
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL((replicate_kernel<uint8_t>), dim3(g), dim3(256), 0, s, (uint8_t *)dst, n, (uint8_t)pattern); break;
    case 2: hipLaunchKernelGGL((replicate_kernel<uint16_t>), dim3(g), dim3(256), 0, s, (uint16_t *)dst, n, (uint16_t)pattern); break;
    case 4: hipLaunchKernelGGL((replicate_kernel<uint32_t>), dim3(g), dim3(256), 0, s, (uint32_t *)dst, n, (uint32_t)pattern); break;
    case 8: hipLaunchKernelGGL((replicate_kernel<uint64_t>), dim3(g), dim3(256), 0, s, (uint64_t *)dst, n, (uint64_t)pattern); break;
    default: return FA_ENOTSUP;
  }
  return launch_status();
}

extern "C" int fa_iota(fa_stream_t stream, fa_dtype t, void *dst, int64_t n, int64_t start,
                       int64_t step) {
  if (n < 0 || (n > 0 && dst == nullptr)) return FA_EINVAL;
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int g = grid_for(n, 256 * 4);
  switch (t) {
    case FA_I32: case FA_U32:
      hipLaunchKernelGGL((iota_kernel<int32_t>), dim3(g), dim3(256), 0, s, (int32_t *)dst, n, (int32_t)start, (int32_t)step);
      break;
    case FA_I64: case FA_U64:
      hipLaunchKernelGGL((iota_kernel<int64_t>), dim3(g), dim3(256), 0, s, (int64_t *)dst, n, start, step);
      break;
    default: return FA_ENOTSUP;
  }
  return launch_status();
}

extern "C" int fa_copy(fa_stream_t stream, void *dst, const void *src, size_t bytes) {
  if (bytes > 0 && (dst == nullptr || src == nullptr)) return FA_EINVAL;
  if (bytes == 0) return 0;
  if (!is_aligned(dst, 16) || !is_aligned(src, 16)) return FA_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  const int64_t nvec = (int64_t)(bytes / 16);
  if (nvec > 0) {
    hipLaunchKernelGGL(copy_kernel, dim3(grid_for(nvec, 256 * 4)), dim3(256), 0, s, (uint4 *)dst,
                       (const uint4 *)src, nvec);
  }
  if (bytes % 16) {
    hipLaunchKernelGGL(copy_tail_kernel, dim3(1), dim3(16), 0, s, (uint8_t *)dst,
                       (const uint8_t *)src, nvec * 16, (int64_t)bytes);
  }
  return launch_status();
}

// 1.2: fa_tuning has grown by scan_tickets_by_block (1.1) and sort_wide_positions (1.2).
extern "C" int fa_version(void) { return 1002; }

extern "C" const char *fa_strerror(int code) {
  if (code == 0) return "success";
  if (code > 0) return hipGetErrorString((hipError_t)code);
  switch (code) {
    case FA_EINVAL: return "invalid argument";
    case FA_ENOTSUP: return "element type / operator combination not supported";
    case FA_ESCRATCH: return "scratch buffer too small";
    case FA_EALIGN: return "pointer not sufficiently aligned";
    default: return "unknown error";
  }
}

// ------------------------------------------------------------------ tuning
// One set per calling thread: the launchers read it on the thread that calls
// them, so callers that hold different values (contexts with different tuning
// parameters) can run side by side without touching each other's.
static thread_local fa_tuning g_tuning = {0, 0, 0, 0, 0};

extern "C" void fa_set_tuning(const fa_tuning *t) {
  if (t == nullptr) {
    g_tuning = fa_tuning{0, 0, 0, 0, 0};
    return;
  }
  g_tuning = *t;
  if (g_tuning.segred_small_threshold < 0) g_tuning.segred_small_threshold = 0;
  if (g_tuning.hist_lds_bins_max < 0) g_tuning.hist_lds_bins_max = 0;
  if (g_tuning.matmul_pad_min_work < 0) g_tuning.matmul_pad_min_work = 0;
}

extern "C" void fa_get_tuning(fa_tuning *out) {
  if (out == nullptr) return;
  out->segred_small_threshold = g_tuning.segred_small_threshold > 0 ? g_tuning.segred_small_threshold : 8192;
  int64_t bins = g_tuning.hist_lds_bins_max > 0 ? g_tuning.hist_lds_bins_max : 32768;
  if (bins > 32768) bins = 32768;
  if (bins < 64) bins = 64;
  out->hist_lds_bins_max = bins;
  out->matmul_pad_min_work = g_tuning.matmul_pad_min_work > 0 ? g_tuning.matmul_pad_min_work : (int64_t)1 << 24;
  out->scan_tickets_by_block = g_tuning.scan_tickets_by_block != 0;
  out->sort_wide_positions = g_tuning.sort_wide_positions != 0;
}
