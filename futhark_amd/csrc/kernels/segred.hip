// SegRed for gfx950: non-segmented reduction and regular segmented reduction.
//
// Result-wise this follows the reference's SegRed code generator
// (src/Futhark/CodeGen/ImpGen/GPU/SegRed.hs): a commutative stage one in which
// thread t folds elements t, t+T, t+2T, ... (SegRed.hs:802-832), per-block
// partials, and a stage two run by one block of the same launch
// (SegRed.hs:923-1047 picks the block that arrives last with an atomic counter;
// here the block that starts last waits for the others); short rows are folded
// by groups of lanes (SegRed.hs:396-505), long rows by whole blocks, a few very
// long rows by several blocks each (SegRed.hs:507-636).  The schedule is new:
// 128-bit non-temporal loads, four loads in flight per thread, wave64 DPP
// reductions and a single LDS exchange per block.
#include "common.hip.h"

namespace fa {

// Stage two without fences or a last-arrival counter: every block draws a
// ticket when it STARTS (off the critical path; same-address device atomics
// complete at about one per 12 ns on MI355X), publishes its partial as a
// single 64-bit {value, epoch} word (two words for 8-byte types), and the
// block holding the last ticket waits for all partials and folds them.  Every
// other block has started before the finisher drew its ticket and depends on
// nothing, so the wait terminates.
// One block of 1024 threads per CU: measured faster than more, smaller blocks
// (fewer partials for the finisher to collect), 64 bytes in flight per thread.
constexpr int SEGRED_BLOCK = 1024;
// 16-byte loads a thread of the non-segmented kernel keeps in flight.  Measured
// at 2^26 f32: 1 -> 48.1 us, 2 -> 43.9 us, 3 -> 45.5 us, 4 -> 46.5 us, 8 and 16 -> 46 us
// (2^24 elements: 15.7 us for 2 and more).
constexpr int SEGRED_UNROLL = 2;
constexpr int SEGRED_MAX_GRID = 1024;
// The header is shared with the scan kernel (its ticket counters live in the
// first 8 KiB of the same scratch buffer); partials follow it.
constexpr size_t SEGRED_HEADER_BYTES = 8192;

static int segred_grid_limit() {
  static int limit = 0;
  if (limit == 0) {
    int dev = 0, cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess) {
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    }
    limit = cus > SEGRED_MAX_GRID ? SEGRED_MAX_GRID : cus;
  }
  return limit;
}

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

// The scratch buffer and its epochs are shared with the single-pass scan, whose
// descriptor words end in (epoch << 3 | flag << 2 | status) with status 1 or
// 2.  A partial ends in (epoch << 3 | 3): no word a scan has ever left behind
// can be taken for the partial of a later reduction, whatever the two epochs.
__device__ __forceinline__ uint32_t partial_meta(uint32_t epoch) { return (epoch << 3) | 3u; }

template <class T>
__device__ __forceinline__ void partial_publish(uint64_t *desc, int slot, uint32_t epoch, T v) {
  epoch = partial_meta(epoch);
  if constexpr (sizeof(T) == 4) {
    st_relaxed_u64(desc + 2 * slot, ((uint64_t)bit_cast<uint32_t>(v) << 32) | epoch);
  } else {
    const uint64_t b = bit_cast<uint64_t>(v);
    st_relaxed_u64(desc + 2 * slot, ((b & 0xffffffffull) << 32) | epoch);
    st_relaxed_u64(desc + 2 * slot + 1, ((b >> 32) << 32) | epoch);
  }
}

template <class T>
__device__ __forceinline__ T partial_wait(const uint64_t *desc, int slot, uint32_t epoch) {
  epoch = partial_meta(epoch);
  uint64_t w0;
  while ((uint32_t)(w0 = ld_relaxed_u64(desc + 2 * slot)) != epoch) __builtin_amdgcn_s_sleep(1);
  if constexpr (sizeof(T) == 4) {
    return bit_cast<T>((uint32_t)(w0 >> 32));
  } else {
    uint64_t w1;
    while ((uint32_t)(w1 = ld_relaxed_u64(desc + 2 * slot + 1)) != epoch)
      __builtin_amdgcn_s_sleep(1);
    return bit_cast<T>((w0 >> 32) | ((w1 >> 32) << 32));
  }
}

template <class T, class Op>
__global__ __launch_bounds__(SEGRED_BLOCK) void segred_nonseg_kernel(
    const T *__restrict__ xs, int64_t n, T *__restrict__ out, uint32_t *ticket, uint64_t *desc,
    uint32_t epoch) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ T lds[SEGRED_BLOCK / WAVE];
  __shared__ uint32_t s_ticket;

  uint32_t my_ticket = 0;
  if (gridDim.x > 1 && threadIdx.x == 0) my_ticket = atomicAdd(ticket, 1u);

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
    partial_publish<T>(desc, (int)blockIdx.x, epoch, v);
    s_ticket = my_ticket;
    // Last ticket of this launch: rearm the counter for the next one.
    if (my_ticket == gridDim.x - 1) st_relaxed_u32(ticket, 0u);
  }
  __syncthreads();
  if (s_ticket != gridDim.x - 1) return;

  // Stage two, in slot order, so the result does not depend on timing.
  T r = Op::identity();
  for (int p = threadIdx.x; p < (int)gridDim.x; p += SEGRED_BLOCK)
    r = Op::apply(r, partial_wait<T>(desc, p, epoch));
  r = block_reduce<T, Op, SEGRED_BLOCK>(r, lds);
  if (threadIdx.x == 0) *out = r;
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

// The same with 128-bit loads, for rows that are whole vectors (k a multiple of
// VEC, 16-byte aligned base): lane `sub` of a group folds vectors sub, sub + G,
// ... of its row, four loads in flight.  G = 1 is a row per lane.
template <class T, class Op, int G>
__global__ __launch_bounds__(256) void segred_small_vec_kernel(const T *__restrict__ xss, int64_t m,
                                                               int64_t k, T *__restrict__ out) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t gthread = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t seg = gthread / G;
  const int sub = (int)(gthread % G);
  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  if (seg < m) {
    const T *row = xss + seg * k;
    const int64_t kv = k / VEC;
    int64_t j = sub;
    for (; j + 3 * G < kv; j += 4 * G) {
      Vec16<T> v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) v[u] = load_vec16_nt(row + (j + u * G) * VEC);
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
    }
    for (; j < kv; j += G) {
      const Vec16<T> v = load_vec16_nt(row + j * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v.e[e]);
    }
  }
  T a = acc[0];
#pragma unroll
  for (int e = 1; e < VEC; e++) a = Op::apply(a, acc[e]);
#pragma unroll
  for (int d = G / 2; d >= 1; d /= 2) {
    T other;
    if constexpr (sizeof(T) == 4) {
      other = bit_cast<T>(__shfl_down(bit_cast<int>(a), d, WAVE));
    } else {
      other = bit_cast<T>((unsigned long long)__shfl_down(
          (unsigned long long)bit_cast<uint64_t>(a), d, WAVE));
    }
    a = Op::apply(a, other);
  }
  if (seg < m && sub == 0) out[seg] = a;
}

// Rows so short that a lane holds at most two 16-byte vectors of one: a group
// of G lanes takes R rows at a time (rows g, g + groups, g + 2 groups, ..., so
// that the lanes of a wave still read consecutive memory) and requests all
// their vectors before folding any, which keeps 2 R loads in flight per lane
// instead of 2.
template <class T, class Op, int G, int R>
__global__ __launch_bounds__(256) void segred_short_vec_kernel(const T *__restrict__ xss, int64_t m,
                                                               int64_t k, T *__restrict__ out,
                                                               int64_t groups) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t gthread = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t g = gthread / G;
  const int sub = (int)(gthread % G);
  const int64_t kv = k / VEC;  // at most 2 G
  Vec16<T> v[R][2];
  bool have[R][2];
#pragma unroll
  for (int u = 0; u < R; u++) {
    const int64_t seg = g + u * groups;
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int64_t j = sub + q * G;
      have[u][q] = g < groups && seg < m && j < kv;
      if (have[u][q]) v[u][q] = load_vec16_nt(xss + seg * k + j * VEC);
    }
  }
#pragma unroll
  for (int u = 0; u < R; u++) {
    T a = Op::identity();
#pragma unroll
    for (int q = 0; q < 2; q++)
      if (have[u][q]) {
#pragma unroll
        for (int e = 0; e < VEC; e++) a = Op::apply(a, v[u][q].e[e]);
      }
#pragma unroll
    for (int d = G / 2; d >= 1; d /= 2) {
      T other;
      if constexpr (sizeof(T) == 4) {
        other = bit_cast<T>(__shfl_down(bit_cast<int>(a), d, WAVE));
      } else {
        other = bit_cast<T>((unsigned long long)__shfl_down(
            (unsigned long long)bit_cast<uint64_t>(a), d, WAVE));
      }
      a = Op::apply(a, other);
    }
    const int64_t seg = g + u * groups;
    if (g < groups && seg < m && sub == 0) __builtin_nontemporal_store(a, &out[seg]);
  }
}

// k large: one block per segment (grid-stride over segments).  With `pieces`
// > 1 every row is cut into that many pieces of `piece_len` elements (the last
// one shorter) and out[seg * pieces + p] receives the fold of piece p: the
// first of two stages for a few very long rows.
template <class T, class Op>
__global__ __launch_bounds__(1024) void segred_large_kernel(const T *__restrict__ xss, int64_t m,
                                                            int64_t row_len, T *__restrict__ out,
                                                            int64_t pieces, int64_t piece_len) {
  __shared__ T lds[1024 / WAVE];
  for (int64_t seg = blockIdx.x; seg < m * pieces; seg += gridDim.x) {
    const int64_t first = (seg % pieces) * piece_len;
    const int64_t k = row_len - first < piece_len ? row_len - first : piece_len;
    const T *row = xss + (seg / pieces) * row_len + first;
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
                         size_t scratch_bytes, uint32_t epoch) {
  constexpr int VEC = Vec16<T>::N;
  if (scratch_bytes < SEGRED_HEADER_BYTES + (size_t)SEGRED_MAX_GRID * 16) return FA_ESCRATCH;
  if (!is_aligned(xs, 16) || !is_aligned(scratch, 16)) return FA_EALIGN;
  const int64_t want = ceil_div(n / VEC, (int64_t)SEGRED_BLOCK * SEGRED_UNROLL);
  const int limit = segred_grid_limit();
  const int grid = (int)(want < 1 ? 1 : (want > limit ? limit : want));
  uint32_t *ticket = (uint32_t *)scratch;
  uint64_t *desc = (uint64_t *)((char *)scratch + SEGRED_HEADER_BYTES);
  hipLaunchKernelGGL((segred_nonseg_kernel<T, Op>), dim3(grid), dim3(SEGRED_BLOCK), 0, s,
                     (const T *)xs, n, (T *)out, ticket, desc, epoch);
  return launch_status();
}

// Rows longer than this are folded by whole blocks (fa_tuning).
static int64_t segred_large_k() {
  fa_tuning t;
  fa_get_tuning(&t);
  return t.segred_small_threshold;
}

// How many pieces a row is cut into so that a few long rows still fill the
// chip (the reference's large-segments case spreads a segment over several
// blocks too, SegRed.hs:507-636).
static int64_t segred_pieces(int64_t m, int64_t k) {
  const int64_t blocks_wanted = (int64_t)segred_grid_limit() * 4;
  const int64_t large_k = segred_large_k();
  if (k <= large_k || m >= blocks_wanted) return 1;
  const int64_t by_fill = ceil_div(blocks_wanted, m);
  const int64_t by_size = ceil_div(k, (int64_t)16384);  // pieces stay at least this long
  const int64_t p = by_fill < by_size ? by_fill : by_size;
  return p < 1 ? 1 : p;
}

template <class T, class Op>
static int launch_small(hipStream_t s, const T *in, int64_t m, int64_t k, T *o) {
  constexpr int VEC = Vec16<T>::N;
  const bool vec = k % VEC == 0 && is_aligned(in, 16);
  const int64_t units = vec ? k / VEC : k;  // what one lane takes per step
#define FA_SMALL(KERNEL, G)                                                                  \
  do {                                                                                       \
    int64_t threads = m * (G);                                                               \
    int64_t grid = ceil_div(threads, 256);                                                   \
    if (grid > INT32_MAX) return FA_EINVAL;                                                  \
    hipLaunchKernelGGL((KERNEL<T, Op, G>), dim3((unsigned)grid), dim3(256), 0, s, in, m, k, o); \
  } while (0)
#define FA_SMALL_BY_UNITS(KERNEL)            \
  do {                                       \
    if (units <= 2) FA_SMALL(KERNEL, 1);     \
    else if (units <= 8) FA_SMALL(KERNEL, 4);   \
    else if (units <= 64) FA_SMALL(KERNEL, 16); \
    else FA_SMALL(KERNEL, 64);               \
  } while (0)
#define FA_SHORT(G)                                                                           \
  do {                                                                                        \
    constexpr int R = 4;                                                                      \
    const int64_t groups = ceil_div(m, (int64_t)R);                                           \
    const int64_t grid = ceil_div(groups * (G), (int64_t)256);                                \
    if (grid > INT32_MAX) return FA_EINVAL;                                                   \
    hipLaunchKernelGGL((segred_short_vec_kernel<T, Op, G, R>), dim3((unsigned)grid), dim3(256), 0, \
                       s, in, m, k, o, groups);                                               \
  } while (0)
  if (vec && units <= 2) FA_SHORT(1);
  else if (vec && units <= 8) FA_SHORT(4);
  else if (vec && units <= 32) FA_SHORT(16);
  else if (vec) FA_SMALL_BY_UNITS(segred_small_vec_kernel);
  else FA_SMALL_BY_UNITS(segred_small_kernel);
#undef FA_SHORT
#undef FA_SMALL_BY_UNITS
#undef FA_SMALL
  return launch_status();
}

template <class T, class Op>
static int launch_regular(hipStream_t s, const void *xss, int64_t m, int64_t k, void *out,
                          void *workspace, size_t workspace_bytes) {
  if (m == 0) return 0;
  const T *in = (const T *)xss;
  T *o = (T *)out;
  if (k <= segred_large_k()) return launch_small<T, Op>(s, in, m, k, o);
  int64_t pieces = segred_pieces(m, k);
  if (pieces > 1 && (workspace == nullptr || workspace_bytes < (size_t)(m * pieces) * sizeof(T) ||
                     !is_aligned(workspace, 16)))
    pieces = 1;
  const int64_t piece_len = pieces == 1 ? k : ceil_div(ceil_div(k, pieces), (int64_t)4096) * 4096;
  const int64_t blocks = m * pieces;
  const int64_t grid = blocks < 65536 ? blocks : 65536;
  hipLaunchKernelGGL((segred_large_kernel<T, Op>), dim3((unsigned)grid), dim3(1024), 0, s, in, m, k,
                     pieces == 1 ? o : (T *)workspace, pieces, piece_len);
  const int rc = launch_status();
  if (rc != 0 || pieces == 1) return rc;
  return launch_small<T, Op>(s, (const T *)workspace, m, pieces, o);
}

// ------------------------------------------- vectorised operator: columns
// `reduce (map2 op) (replicate k ne) xss` with xss : [n][k] -- a reduction
// whose operator works on whole rows, which the reference turns into one
// reduction per column by interchanging the loops (SegRed.hs:274-290).  Here a
// lane owns VEC consecutive columns (one 16-byte vector per row) and a wave a
// contiguous span of 64 * VEC elements: a strip of columns when rows are longer
// than that, several whole rows when they are shorter (lanes that start in
// different rows of the span own the same columns and are folded at the end).
// The 16 waves of a block take spans in turn within the block's chunk of rows;
// every chunk leaves k partial results and a second launch folds the chunks.
// Measured at 2^26 f32 elements: 1024 threads with 4 rows in flight and two
// blocks per CU (all of them resident at once) did best; 8 rows in flight,
// smaller blocks and more blocks per CU were 5 to 40 % slower.
constexpr int COLRED_BLOCK = 1024;
constexpr int COLRED_UNROLL = 4;
constexpr int COLRED_BLOCKS_PER_CU = 2;
constexpr int COLRED_WAVES = COLRED_BLOCK / WAVE;

struct ColredShape {
  int64_t strips;          // column strips (1 when a span holds whole rows)
  int64_t rows_per_span;   // whole rows in one wave span (1 when a row is longer than a span)
  int64_t chunks;          // blocks along the rows
  int64_t rows_per_chunk;  // multiple of rows_per_span * COLRED_WAVES
};

static ColredShape colred_shape(int64_t n, int64_t k, int vec) {
  ColredShape sh;
  const int64_t span = (int64_t)WAVE * vec;
  sh.strips = k >= span ? ceil_div(k, span) : 1;
  sh.rows_per_span = k >= span ? 1 : span / k;
  const int64_t step = sh.rows_per_span * COLRED_WAVES;  // rows one block takes per turn
  if (n <= 0) {
    sh.chunks = 1;
    sh.rows_per_chunk = step;
    return sh;
  }
  const int64_t want = ceil_div((int64_t)segred_grid_limit() * COLRED_BLOCKS_PER_CU, sh.strips);
  const int64_t most = ceil_div(n, step * 4);  // at least four turns per block
  sh.chunks = want < most ? want : most;
  if (sh.chunks < 1) sh.chunks = 1;
  sh.rows_per_chunk = ceil_div(ceil_div(n, sh.chunks), step) * step;
  sh.chunks = ceil_div(n, sh.rows_per_chunk);
  if (sh.chunks < 1) sh.chunks = 1;
  return sh;
}

template <class T, class Op, int VEC>
__global__ __launch_bounds__(COLRED_BLOCK) void colred_kernel(const T *__restrict__ xss, int64_t n,
                                                              int64_t k, T *__restrict__ out,
                                                              int64_t rows_per_span,
                                                              int64_t rows_per_chunk) {
  extern __shared__ __align__(16) unsigned char s_raw[];
  T *lds = reinterpret_cast<T *>(s_raw);  // [COLRED_WAVES][WAVE * VEC]
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / WAVE));
  const int64_t span = (int64_t)WAVE * VEC;
  const int64_t in_span = (int64_t)lane * VEC;  // first element of this lane inside its span
  // column of this lane's first element, and the row of the span it lies in
  const int64_t sub_row = rows_per_span > 1 ? in_span / k : 0;
  const int64_t col = rows_per_span > 1 ? in_span % k : (int64_t)blockIdx.x * span + in_span;
  const bool owns = rows_per_span > 1 ? sub_row < rows_per_span : col < k;
  const int64_t row0 = (int64_t)blockIdx.y * rows_per_chunk;
  int64_t row1 = row0 + rows_per_chunk;
  if (row1 > n) row1 = n;
  const int64_t step = rows_per_span * COLRED_WAVES;

  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  auto fold = [&](int64_t r) {
    if constexpr (VEC > 1) {
      const Vec16<T> v = load_vec16_nt(xss + r * k + col);
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v.e[e]);
    } else {
      acc[0] = Op::apply(acc[0], xss[r * k + col]);
    }
  };
  if (owns) {
    int64_t r = row0 + (int64_t)wave * rows_per_span + sub_row;
    for (; r + (COLRED_UNROLL - 1) * step < row1; r += COLRED_UNROLL * step) {  // rows in flight
      if constexpr (VEC > 1) {
        Vec16<T> v[COLRED_UNROLL];
#pragma unroll
        for (int u = 0; u < COLRED_UNROLL; u++) v[u] = load_vec16_nt(xss + (r + u * step) * k + col);
#pragma unroll
        for (int u = 0; u < COLRED_UNROLL; u++)
#pragma unroll
          for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
      } else {
        T v[COLRED_UNROLL];
#pragma unroll
        for (int u = 0; u < COLRED_UNROLL; u++) v[u] = xss[(r + u * step) * k + col];
#pragma unroll
        for (int u = 0; u < COLRED_UNROLL; u++) acc[0] = Op::apply(acc[0], v[u]);
      }
    }
    for (; r < row1; r += step) fold(r);
  }
#pragma unroll
  for (int e = 0; e < VEC; e++) lds[(int64_t)wave * span + in_span + e] = acc[e];
  __syncthreads();
  // fold over the waves: thread i takes element i of the span
  const int tid = (int)threadIdx.x;
  T r = Op::identity();
  if (tid < span)
    for (int w = 0; w < COLRED_WAVES; w++) r = Op::apply(r, lds[(int64_t)w * span + tid]);
  __syncthreads();
  if (tid < span) lds[tid] = r;
  __syncthreads();
  if (rows_per_span > 1) {
    // the span holds rows_per_span partial rows of k columns each: halve them
    for (int64_t cnt = rows_per_span; cnt > 1;) {
      const int64_t half = (cnt + 1) / 2;
      if (tid < (cnt - half) * k) lds[tid] = Op::apply(lds[tid], lds[tid + half * k]);
      __syncthreads();
      cnt = half;
    }
    if (tid < k) out[(int64_t)blockIdx.y * k + tid] = lds[tid];
  } else {
    const int64_t c = (int64_t)blockIdx.x * span + tid;
    if (tid < span && c < k) out[(int64_t)blockIdx.y * k + c] = lds[tid];
  }
}

template <class T, class Op, int VEC>
static void colred_launch(hipStream_t s, const T *in, int64_t n, int64_t k, T *out,
                          const ColredShape &sh) {
  const size_t lds = (size_t)COLRED_WAVES * WAVE * VEC * sizeof(T);
  hipLaunchKernelGGL((colred_kernel<T, Op, VEC>), dim3((unsigned)sh.strips, (unsigned)sh.chunks),
                     dim3(COLRED_BLOCK), lds, s, in, n, k, out, sh.rows_per_span, sh.rows_per_chunk);
}

template <class T, class Op>
static int launch_columns(hipStream_t s, const void *xss, int64_t n, int64_t k, void *out,
                          void *workspace, size_t workspace_bytes) {
  if (k == 0) return 0;
  constexpr int V = Vec16<T>::N;
  const T *in = (const T *)xss;
  T *o = (T *)out;
  for (int stage = 0; stage < 2; stage++) {
    const bool vec = k % V == 0 && is_aligned(in, 16);
    ColredShape sh = colred_shape(n, k, vec ? V : 1);
    if (stage == 1 || workspace == nullptr || workspace_bytes < (size_t)(sh.chunks * k) * sizeof(T) ||
        !is_aligned(workspace, 16)) {
      // the last stage: one chunk, straight into out
      sh.chunks = 1;
      const int64_t step = sh.rows_per_span * COLRED_WAVES;
      sh.rows_per_chunk = ceil_div(n > 0 ? n : 1, step) * step;
    }
    if (sh.strips > INT32_MAX || sh.chunks > 65535) return FA_EINVAL;
    T *dst = sh.chunks == 1 ? o : (T *)workspace;
    if (vec) colred_launch<T, Op, V>(s, in, n, k, dst, sh);
    else colred_launch<T, Op, 1>(s, in, n, k, dst, sh);
    const int rc = launch_status();
    if (rc != 0 || sh.chunks == 1) return rc;
    in = (const T *)workspace;  // fold the chunks: [chunks][k]
    n = sh.chunks;
  }
  return 0;
}

}  // namespace fa

#include "dispatch.hip.h"

extern "C" size_t fa_segred_scratch_bytes(fa_dtype t) {
  (void)t;
  return SEGRED_HEADER_BYTES + (size_t)SEGRED_MAX_GRID * 16;
}

extern "C" int fa_segred_nonseg(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                                int64_t n, void *out, void *scratch, size_t scratch_bytes,
                                uint32_t epoch) {
  if (n < 0 || out == nullptr || scratch == nullptr || (n > 0 && xs == nullptr))
    return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_nonseg, t, op, s, xs, n, out, scratch, scratch_bytes, epoch);
}

extern "C" size_t fa_segred_regular_workspace_bytes(fa_dtype t, int64_t m, int64_t k) {
  if (m <= 0 || k <= 0) return 0;
  const int64_t pieces = segred_pieces(m, k);
  const size_t es = (t == FA_I64 || t == FA_U64 || t == FA_F64) ? 8 : 4;
  return pieces > 1 ? (size_t)(m * pieces) * es : 0;
}

extern "C" int fa_segred_regular_ws(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                                    int64_t m, int64_t k, void *out, void *workspace,
                                    size_t workspace_bytes) {
  if (m < 0 || k < 0 || (m > 0 && out == nullptr) || (m * k > 0 && xss == nullptr))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_regular, t, op, s, xss, m, k, out, workspace, workspace_bytes);
}

extern "C" int fa_segred_regular(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                                 int64_t m, int64_t k, void *out) {
  return fa_segred_regular_ws(stream, t, op, xss, m, k, out, nullptr, 0);
}

extern "C" size_t fa_segred_columns_workspace_bytes(fa_dtype t, int64_t n, int64_t k) {
  if (n <= 0 || k <= 0) return 0;
  const size_t es = (t == FA_I64 || t == FA_U64 || t == FA_F64) ? 8 : 4;
  // the larger of the two chunk counts (vector and element-wise spans)
  const ColredShape a = colred_shape(n, k, (int)(16 / es)), b = colred_shape(n, k, 1);
  const int64_t chunks = a.chunks > b.chunks ? a.chunks : b.chunks;
  return chunks > 1 ? (size_t)(chunks * k) * es : 0;
}

extern "C" int fa_segred_columns(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                                 int64_t n, int64_t k, void *out, void *workspace,
                                 size_t workspace_bytes) {
  if (n < 0 || k < 0 || (k > 0 && out == nullptr) || (n * k > 0 && xss == nullptr))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_columns, t, op, s, xss, n, k, out, workspace, workspace_bytes);
}
