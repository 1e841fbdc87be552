// SegRed for gfx950: non-segmented reduction and regular segmented reduction.
//
// Result-wise this follows the reference's SegRed code generator
// (src/Futhark/CodeGen/ImpGen/GPU/SegRed.hs): a commutative stage one in which
// thread t folds elements t, t+T, t+2T, ... (SegRed.hs:802-832), per-block
// partials, and a stage two run by whichever block finishes last, detected
// with an atomic counter (SegRed.hs:923-1047).  The schedule is new: 128-bit
// loads, four loads in flight per thread, a wave64 DPP reduction and a single
// LDS exchange per block.
#include "common.hip.h"

namespace fa {

// Blocks per launch: enough resident waves on every CU to cover HBM latency
// without making stage two long.
static int segred_grid_limit() {
  static int limit = 0;
  if (limit == 0) {
    int dev = 0, cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess) {
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    }
    limit = cus * 8;
  }
  return limit;
}

constexpr int SEGRED_BLOCK = 256;
constexpr int SEGRED_UNROLL = 4;
constexpr int SEGRED_MAX_GRID = 4096;  // bounds the partials array

template <class T, class Op, int BLOCK>
__device__ __forceinline__ T block_reduce(T v, T *lds /* BLOCK/64 slots */) {
  v = wave_reduce<T, Op>(v);
  const int wave = threadIdx.x / WAVE;
  if (lane_id() == 0) lds[wave] = v;
  __syncthreads();
  T r = Op::identity();
#pragma unroll
  for (int w = 0; w < BLOCK / WAVE; w++) r = Op::apply(r, lds[w]);
  __syncthreads();
  return r;
}

template <class T, class Op>
__global__ __launch_bounds__(SEGRED_BLOCK) void segred_nonseg_kernel(
    const T *__restrict__ xs, int64_t n, T *__restrict__ out, T *partials, uint32_t *counter) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ T lds[SEGRED_BLOCK / WAVE];
  __shared__ uint32_t is_last;

  const int64_t nvec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * SEGRED_BLOCK;
  int64_t i = (int64_t)blockIdx.x * SEGRED_BLOCK + threadIdx.x;

  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();

  for (; i + (SEGRED_UNROLL - 1) * stride < nvec; i += SEGRED_UNROLL * stride) {
    Vec16<T> v[SEGRED_UNROLL];
#pragma unroll
    for (int u = 0; u < SEGRED_UNROLL; u++) v[u] = load_vec16_nt(xs + (i + u * stride) * VEC);
#pragma unroll
    for (int u = 0; u < SEGRED_UNROLL; u++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
  }
  for (; i < nvec; i += stride) {
    Vec16<T> v = load_vec16_nt(xs + i * VEC);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v.e[e]);
  }
  // The last n % VEC elements.
  {
    const int64_t g = (int64_t)blockIdx.x * SEGRED_BLOCK + threadIdx.x;
    const int64_t tail = nvec * VEC + g;
    if (g < VEC && tail < n) acc[0] = Op::apply(acc[0], xs[tail]);
  }

  T v = acc[0];
#pragma unroll
  for (int e = 1; e < VEC; e++) v = Op::apply(v, acc[e]);
  v = block_reduce<T, Op, SEGRED_BLOCK>(v, lds);

  if (gridDim.x == 1) {
    if (threadIdx.x == 0) *out = v;
    return;
  }

  if (threadIdx.x == 0) {
    using U = typename std::conditional<sizeof(T) == 4, uint32_t, uint64_t>::type;
    __hip_atomic_store(reinterpret_cast<U *>(partials) + blockIdx.x, bit_cast<U>(v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();
    uint32_t old = atomicAdd(counter, 1u);
    is_last = (old == gridDim.x - 1) ? 1u : 0u;
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();

  // Stage two: this block arrived last, so every partial is visible.
  T r = Op::identity();
  for (int p = threadIdx.x; p < (int)gridDim.x; p += SEGRED_BLOCK) {
    using U = typename std::conditional<sizeof(T) == 4, uint32_t, uint64_t>::type;
    U bits = __hip_atomic_load(reinterpret_cast<U *>(partials) + p, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    r = Op::apply(r, bit_cast<T>(bits));
  }
  r = block_reduce<T, Op, SEGRED_BLOCK>(r, lds);
  if (threadIdx.x == 0) {
    *out = r;
    __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ------------------------------------------------- regular segments [m][k]

// k small: a group of G lanes (power of two, <= 64) per segment.
template <class T, class Op, int G>
__global__ __launch_bounds__(256) void segred_small_kernel(const T *__restrict__ xss, int64_t m,
                                                           int64_t k, T *__restrict__ out) {
  const int64_t gthread = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t seg = gthread / G;
  const int sub = (int)(gthread % G);
  T acc = Op::identity();
  if (seg < m) {
    const T *row = xss + seg * k;
    for (int64_t j = sub; j < k; j += G) acc = Op::apply(acc, row[j]);
  }
  // Tree over the G lanes of the group; groups never straddle a wave.
#pragma unroll
  for (int d = G / 2; d >= 1; d /= 2) {
    T other;
    if constexpr (sizeof(T) == 4) {
      other = bit_cast<T>(__shfl_down(bit_cast<int>(acc), d, WAVE));
    } else {
      other = bit_cast<T>((unsigned long long)__shfl_down(
          (unsigned long long)bit_cast<uint64_t>(acc), d, WAVE));
    }
    acc = Op::apply(acc, other);
  }
  if (seg < m && sub == 0) out[seg] = acc;
}

// k large: one block per segment (grid-stride over segments).
template <class T, class Op>
__global__ __launch_bounds__(1024) void segred_large_kernel(const T *__restrict__ xss, int64_t m,
                                                            int64_t k, T *__restrict__ out) {
  __shared__ T lds[1024 / WAVE];
  for (int64_t seg = blockIdx.x; seg < m; seg += gridDim.x) {
    const T *row = xss + seg * k;
    T acc0 = Op::identity(), acc1 = Op::identity(), acc2 = Op::identity(),
      acc3 = Op::identity();
    int64_t j = threadIdx.x;
    for (; j + 3 * 1024 < k; j += 4 * 1024) {
      T a = row[j], b = row[j + 1024], c = row[j + 2048], d = row[j + 3072];
      acc0 = Op::apply(acc0, a);
      acc1 = Op::apply(acc1, b);
      acc2 = Op::apply(acc2, c);
      acc3 = Op::apply(acc3, d);
    }
    for (; j < k; j += 1024) acc0 = Op::apply(acc0, row[j]);
    T v = Op::apply(Op::apply(acc0, acc1), Op::apply(acc2, acc3));
    v = block_reduce<T, Op, 1024>(v, lds);
    if (threadIdx.x == 0) out[seg] = v;
  }
}

template <class T, class Op>
static int launch_nonseg(hipStream_t s, const void *xs, int64_t n, void *out, void *scratch,
                         size_t scratch_bytes) {
  constexpr int VEC = Vec16<T>::N;
  if (scratch_bytes < 64 + (size_t)SEGRED_MAX_GRID * sizeof(T)) return FA_ESCRATCH;
  if (!is_aligned(xs, 16) || !is_aligned(scratch, 16)) return FA_EALIGN;
  int64_t want = ceil_div(n / VEC, (int64_t)SEGRED_BLOCK * SEGRED_UNROLL);
  int limit = segred_grid_limit();
  if (limit > SEGRED_MAX_GRID) limit = SEGRED_MAX_GRID;
  int grid = (int)(want < 1 ? 1 : (want > limit ? limit : want));
  uint32_t *counter = (uint32_t *)scratch;
  T *partials = (T *)((char *)scratch + 64);
  hipLaunchKernelGGL((segred_nonseg_kernel<T, Op>), dim3(grid), dim3(SEGRED_BLOCK), 0, s,
                     (const T *)xs, n, (T *)out, partials, counter);
  return launch_status();
}

template <class T, class Op>
static int launch_regular(hipStream_t s, const void *xss, int64_t m, int64_t k, void *out) {
  if (m == 0) return 0;
  const T *in = (const T *)xss;
  T *o = (T *)out;
#define FA_SMALL(G)                                                                          \
  do {                                                                                       \
    int64_t threads = m * (G);                                                               \
    int64_t grid = ceil_div(threads, 256);                                                   \
    if (grid > INT32_MAX) return FA_EINVAL;                                                  \
    hipLaunchKernelGGL((segred_small_kernel<T, Op, G>), dim3((unsigned)grid), dim3(256), 0, \
                       s, in, m, k, o);                                                      \
  } while (0)
  if (k <= 2) FA_SMALL(1);
  else if (k <= 8) FA_SMALL(4);
  else if (k <= 64) FA_SMALL(16);
  else if (k <= 8192) FA_SMALL(64);
  else {
    int64_t grid = m < 65536 ? m : 65536;
    hipLaunchKernelGGL((segred_large_kernel<T, Op>), dim3((unsigned)grid), dim3(1024), 0, s, in,
                       m, k, o);
  }
#undef FA_SMALL
  return launch_status();
}

}  // namespace fa

#include "dispatch.hip.h"

extern "C" size_t fa_segred_scratch_bytes(fa_dtype t) {
  size_t s = dtype_size(t);
  if (s < 4) s = 8;
  return 64 + (size_t)SEGRED_MAX_GRID * s;
}

extern "C" int fa_segred_nonseg(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                                int64_t n, void *out, void *scratch, size_t scratch_bytes) {
  if (n < 0 || out == nullptr || scratch == nullptr || (n > 0 && xs == nullptr))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_nonseg, t, op, s, xs, n, out, scratch, scratch_bytes);
}

extern "C" int fa_segred_regular(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                                 int64_t m, int64_t k, void *out) {
  if (m < 0 || k < 0 || (m > 0 && out == nullptr) || (m * k > 0 && xss == nullptr))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_regular, t, op, s, xss, m, k, out);
}
