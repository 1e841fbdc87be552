// Copies between index-function (LMAD) layouts on gfx950: the step either side
// of any layout-changing program.  An LMAD is an offset plus one stride per
// dimension, in elements; `shape` is shared by source and destination.
//
// The reference decides per copy what it really is (rts/c/copy.h:55-190,
// dispatch in rts/c/gpu.h:484-586): a flat copy when both sides describe the
// same contiguous layout, a batched 2-D transpose when one side is row-major
// and the other a collapsed column-major view, and an element-by-element copy
// otherwise.  The same three answers are given here (tests compare them case
// by case); what runs for each is native:
//   flat       hipMemcpyAsync device to device;
//   transpose  64x64 tiles through LDS, or, when one extent is at most 32,
//              strips of 256 long lines through LDS
//              (the reference has five kernels per element size for this:
//              rts/opencl/transpose.cl, rts/c/gpu.h:333-461);
//   general    one thread per element, index arithmetic in 64 bits (negative
//              strides allowed), rank up to 8.
#include "dispatch.hip.h"

namespace fa {

constexpr int LMAD_MAX_RANK = 8;

struct LmadArgs {
  int64_t shape[LMAD_MAX_RANK];
  int64_t dst_strides[LMAD_MAX_RANK];
  int64_t src_strides[LMAD_MAX_RANK];
  int rank;
};

template <class T>
__global__ __launch_bounds__(256) void lmad_copy_kernel(T *__restrict__ dst,
                                                        const T *__restrict__ src, LmadArgs a,
                                                        int64_t count) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < count; g += stride) {
    int64_t rem = g, d = 0, s = 0;
#pragma unroll
    for (int k = LMAD_MAX_RANK - 1; k >= 0; k--) {
      if (k < a.rank) {
        const int64_t i = rem % a.shape[k];
        rem /= a.shape[k];
        d += i * a.dst_strides[k];
        s += i * a.src_strides[k];
      }
    }
    dst[d] = src[s];
  }
}

// dst[b][j][i] = src[b][i][j] with a short extent S <= 32.  A block moves a
// strip of W long lines through LDS so that both its global reads and its
// global writes are runs of consecutive elements: with SHORT_ROWS (rows = S)
// the strip is W columns, read row by row and written as one contiguous run of
// W * S elements; otherwise (cols = S) it is W rows, read as one contiguous run
// and written column by column.
template <class T> constexpr int skinny_width() { return sizeof(T) == 8 ? 128 : 256; }

template <class T, bool SHORT_ROWS>
__global__ __launch_bounds__(256) void transpose_skinny_kernel(T *__restrict__ dst,
                                                               const T *__restrict__ src,
                                                               int64_t rows, int64_t cols,
                                                               int64_t first_block) {
  constexpr int W = skinny_width<T>();
  constexpr int LD = W + 1;  // padded: the strided side of each phase walks distinct banks
  __shared__ T tile[32 * LD];
  const int64_t b = blockIdx.y;
  const T *s = src + b * rows * cols;
  T *d = dst + b * rows * cols;
  const int tid = threadIdx.x;
  const int64_t x0 = (first_block + blockIdx.x) * W;  // first long-axis index of the strip
  if (SHORT_ROWS) {
    const int S = (int)rows;
    const int w = (int)(cols - x0 < W ? cols - x0 : W);
    for (int r = 0; r < S; r++)
      for (int x = tid; x < w; x += 256) tile[r * LD + x] = s[(int64_t)r * cols + x0 + x];
    __syncthreads();
    T *out = d + x0 * S;
    for (int e = tid; e < w * S; e += 256)
      __builtin_nontemporal_store(tile[(e % S) * LD + e / S], &out[e]);
  } else {
    const int S = (int)cols;
    const int w = (int)(rows - x0 < W ? rows - x0 : W);
    const T *in = s + x0 * S;
    for (int e = tid; e < w * S; e += 256) tile[(e % S) * LD + e / S] = in[e];
    __syncthreads();
    for (int c = 0; c < S; c++)
      for (int x = tid; x < w; x += 256)
        __builtin_nontemporal_store(tile[c * LD + x], &d[(int64_t)c * rows + x0 + x]);
  }
}

template <class T>
__global__ __launch_bounds__(256) void transpose_tile_kernel(T *__restrict__ dst,
                                                             const T *__restrict__ src,
                                                             int64_t rows, int64_t cols,
                                                             int64_t first_block) {
  constexpr int TS = 64;
  __shared__ T tile[TS][TS + 1];
  // grid.x enumerates the tiles of one matrix row by row, from `first_block` on
  // (the second and third grid dimensions hold 65535 at most), grid.y the
  // matrices of the batch.
  const int64_t b = blockIdx.y;
  const int64_t tiles_x = (cols + TS - 1) / TS;
  const int64_t tile_id = first_block + blockIdx.x;
  const int64_t r0 = (tile_id / tiles_x) * TS, c0 = (tile_id % tiles_x) * TS;
  const T *s = src + b * rows * cols;
  T *d = dst + b * rows * cols;
  const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;  // 64 x 4
#pragma unroll 4
  for (int i = ty; i < TS; i += 4) {
    const int64_t r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[i][tx] = s[r * cols + c];
  }
  __syncthreads();
#pragma unroll 4
  for (int i = ty; i < TS; i += 4) {
    const int64_t c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols) __builtin_nontemporal_store(tile[tx][i], &d[c * rows + r]);
  }
}

// The same tile with 16 bytes per lane on both global sides (V = 16 / sizeof(T)
// elements): a lane loads V consecutive elements of a source row, and stores V
// consecutive elements of a destination row, which it gathers from V source
// rows of the LDS tile.  Needs rows and cols that are multiples of V and
// 16-byte aligned bases.
// Stores are non-temporal in all transposes: the destination is written once
// and not read again by the kernel, and on MI355X that alone takes the 8192^2
// f32 case from 127 us to 95 us (a 128 x 128 tile measured no better).
template <class T>
__global__ __launch_bounds__(256) void transpose_tile_vec_kernel(T *__restrict__ dst,
                                                                 const T *__restrict__ src,
                                                                 int64_t rows, int64_t cols,
                                                                 int64_t first_block) {
  constexpr int TS = 64;
  constexpr int V = 16 / sizeof(T);
  constexpr int LANES = TS / V;         // lanes across one tile row
  constexpr int STEP = 256 / LANES;     // tile rows covered per pass
  __shared__ T tile[TS][TS + 1];
  // grid.x enumerates the tiles of one matrix row by row, from `first_block` on
  // (the second and third grid dimensions hold 65535 at most), grid.y the
  // matrices of the batch.
  const int64_t b = blockIdx.y;
  const int64_t tiles_x = (cols + TS - 1) / TS;
  const int64_t tile_id = first_block + blockIdx.x;
  const int64_t r0 = (tile_id / tiles_x) * TS, c0 = (tile_id % tiles_x) * TS;
  const T *s = src + b * rows * cols;
  T *d = dst + b * rows * cols;
  const int tx = threadIdx.x % LANES, ty = threadIdx.x / LANES;
#pragma unroll
  for (int i = ty; i < TS; i += STEP) {
    const int64_t r = r0 + i, c = c0 + tx * V;
    if (r < rows && c < cols) {
      const Vec16<T> v = load_vec16(s + r * cols + c);
#pragma unroll
      for (int e = 0; e < V; e++) tile[i][tx * V + e] = v.e[e];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = ty; i < TS; i += STEP) {
    const int64_t c = c0 + i, r = r0 + tx * V;  // destination row c, columns r..r+V-1
    if (r < rows && c < cols) {
      Vec16<T> v;
#pragma unroll
      for (int e = 0; e < V; e++) v.e[e] = tile[tx * V + e][i];
      store_vec16_nt(d + c * rows + r, v);
    }
  }
}

template <class T>
static int launch_map_transpose(hipStream_t st, T *dst, const T *src, int64_t batch, int64_t rows,
                                int64_t cols) {
  if (batch == 0 || rows == 0 || cols == 0) return 0;
  if (batch > 65535) {  // the grid's second dimension holds 65535: take the batch in pieces
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
      const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
      const int rc = launch_map_transpose<T>(st, dst + b0 * rows * cols, src + b0 * rows * cols, nb, rows, cols);
      if (rc != 0) return rc;
    }
    return 0;
  }
  // A launch holds fewer than 2^32 threads along x: with 256 per block that is
  // 16777215 blocks; longer grids go out in pieces.
  constexpr int64_t MAX_BLOCKS_X = ((int64_t(1) << 32) - 1) / 256;
  if (rows <= 32 || cols <= 32) {
    const bool short_rows = rows <= cols;
    const int64_t longest = short_rows ? cols : rows;
    const int64_t gx = ceil_div(longest, (int64_t)skinny_width<T>());
    for (int64_t b0 = 0; b0 < gx; b0 += MAX_BLOCKS_X) {
      const dim3 grid((unsigned)(gx - b0 < MAX_BLOCKS_X ? gx - b0 : MAX_BLOCKS_X), (unsigned)batch);
      if (short_rows)
        hipLaunchKernelGGL((transpose_skinny_kernel<T, true>), grid, dim3(256), 0, st, dst, src,
                           rows, cols, b0);
      else
        hipLaunchKernelGGL((transpose_skinny_kernel<T, false>), grid, dim3(256), 0, st, dst, src,
                           rows, cols, b0);
      const int rc = launch_status();
      if (rc != 0) return rc;
    }
    return 0;
  }
  const int64_t gx = ceil_div(cols, (int64_t)64), gy = ceil_div(rows, (int64_t)64);
  if (gx > INT64_MAX / gy) return FA_EINVAL;
  const int64_t tiles = gx * gy;
  constexpr int V = 16 / (int)sizeof(T);
  const bool vec = sizeof(T) >= 4 && rows % V == 0 && cols % V == 0 && is_aligned(dst, 16) &&
                   is_aligned(src, 16);
  for (int64_t b0 = 0; b0 < tiles; b0 += MAX_BLOCKS_X) {
    const dim3 grid((unsigned)(tiles - b0 < MAX_BLOCKS_X ? tiles - b0 : MAX_BLOCKS_X), (unsigned)batch);
    if (vec)
      hipLaunchKernelGGL((transpose_tile_vec_kernel<T>), grid, dim3(256), 0, st, dst, src, rows,
                         cols, b0);
    else
      hipLaunchKernelGGL((transpose_tile_kernel<T>), grid, dim3(256), 0, st, dst, src, rows, cols, b0);
    const int rc = launch_status();
    if (rc != 0) return rc;
  }
  return 0;
}

// ------------------------------------------------------------ classification
// Row-major strides of `shape`.
static void row_major(int r, const int64_t *shape, int64_t *out) {
  int64_t acc = 1;
  for (int i = r - 1; i >= 0; i--) {
    out[i] = acc;
    acc *= shape[i];
  }
}

// Is (strides, shape) a row-major [n][m] array read as its transpose, for
// some split of the dimensions into a leading group (extent n, the fast one in
// memory) and a trailing group (extent m)?  (rts/c/copy.h:55-85)
static bool is_transposed_2d(int r, const int64_t *strides, const int64_t *shape, int64_t *n_out,
                             int64_t *m_out) {
  for (int split = 1; split < r; split++) {
    int64_t expect = 1, n = 1, m = 1;
    bool ok = true;
    for (int j = split - 1; j >= 0; j--) {
      ok = ok && strides[j] == expect;
      expect *= shape[j];
      n *= shape[j];
    }
    for (int j = r - 1; j >= split; j--) {
      ok = ok && strides[j] == expect;
      expect *= shape[j];
      m *= shape[j];
    }
    if (ok) {
      *n_out = n;
      *m_out = m;
      return true;
    }
  }
  return false;
}

// A copy is a batched transpose when, below some leading dimensions on which
// both sides are row-major, one side is row-major and the other a transposed
// 2-D view (rts/c/copy.h:101-143).  On success the copy is
// dst[b][j][i] = src[b][i][j] with src : [batch][rows][cols].
static bool is_map_transpose(int r, const int64_t *dst_strides, const int64_t *src_strides,
                             const int64_t *shape, int64_t *batch, int64_t *rows, int64_t *cols) {
  int64_t rm[LMAD_MAX_RANK];
  row_major(r, shape, rm);
  int lead = 0;
  int64_t arrays = 1;
  while (lead < r && dst_strides[lead] == rm[lead] && src_strides[lead] == rm[lead]) {
    arrays *= shape[lead];
    lead++;
  }
  *batch = arrays;
  if (lead == r) return false;
  const int rest = r - lead;
  bool dst_rm = true, src_rm = true;
  for (int i = lead; i < r; i++) {
    dst_rm = dst_rm && dst_strides[i] == rm[i];
    src_rm = src_rm && src_strides[i] == rm[i];
  }
  int64_t n, m;
  if (dst_rm && is_transposed_2d(rest, src_strides + lead, shape + lead, &n, &m)) {
    // src memory is [m][n] row-major, dst memory is [n][m]: rows = m, cols = n.
    *rows = m;
    *cols = n;
    return true;
  }
  if (src_rm && is_transposed_2d(rest, dst_strides + lead, shape + lead, &n, &m)) {
    // src memory is [n][m] row-major, dst memory is [m][n].
    *rows = n;
    *cols = m;
    return true;
  }
  return false;
}

// Do the strides enumerate, for some order of the dimensions, a dense block
// with positive strides?  (rts/c/copy.h:145-176)
static bool dense_search(int placed, int64_t expect, int r, const int64_t *strides,
                         const int64_t *shape, bool *used) {
  for (int j = 0; j < r; j++) {
    if (used[j] || strides[j] != expect || strides[j] < 0) continue;
    used[j] = true;
    if (placed + 1 == r || dense_search(placed + 1, expect * shape[j], r, strides, shape, used))
      return true;
    used[j] = false;
  }
  return false;
}

static bool is_flat_copy(int r, const int64_t *dst_strides, const int64_t *src_strides,
                         const int64_t *shape) {
  bool used[LMAD_MAX_RANK] = {false};
  if (!dense_search(0, 1, r, dst_strides, shape, used)) return false;
  for (int i = 0; i < r; i++)
    if (dst_strides[i] != src_strides[i] && shape[i] != 1) return false;
  return true;
}

template <class T>
static int lmad_copy_typed(hipStream_t st, T *dst, int64_t dst_offset, const int64_t *dst_strides,
                           const T *src, int64_t src_offset, const int64_t *src_strides,
                           const int64_t *shape, int rank, int *path) {
  int64_t count = 1;
  for (int i = 0; i < rank; i++) count *= shape[i];
  if (path) *path = FA_LMAD_NOTHING;
  if (count == 0) return 0;
  int64_t batch, rows, cols;
  if (is_map_transpose(rank, dst_strides, src_strides, shape, &batch, &rows, &cols)) {
    if (path) *path = FA_LMAD_TRANSPOSE;
    return launch_map_transpose<T>(st, dst + dst_offset, src + src_offset, batch, rows, cols);
  }
  if (is_flat_copy(rank, dst_strides, src_strides, shape)) {
    if (path) *path = FA_LMAD_FLAT;
    hipError_t e = hipMemcpyAsync(dst + dst_offset, src + src_offset, (size_t)count * sizeof(T),
                                  hipMemcpyDeviceToDevice, st);
    return e == hipSuccess ? 0 : (int)e;
  }
  if (path) *path = FA_LMAD_GENERAL;
  LmadArgs a;
  a.rank = rank;
  for (int i = 0; i < LMAD_MAX_RANK; i++) {
    a.shape[i] = i < rank ? shape[i] : 1;
    a.dst_strides[i] = i < rank ? dst_strides[i] : 0;
    a.src_strides[i] = i < rank ? src_strides[i] : 0;
  }
  int64_t g = ceil_div(count, (int64_t)256);
  if (g > 256 * 64) g = 256 * 64;
  hipLaunchKernelGGL((lmad_copy_kernel<T>), dim3((unsigned)g), dim3(256), 0, st, dst + dst_offset,
                     src + src_offset, a, count);
  return launch_status();
}

}  // namespace fa

extern "C" int fa_lmad_copy(fa_stream_t stream, int elem_bytes, void *dst, int64_t dst_offset,
                            const int64_t *dst_strides, const void *src, int64_t src_offset,
                            const int64_t *src_strides, const int64_t *shape, int rank,
                            int *path) {
  if (rank < 0 || rank > fa::LMAD_MAX_RANK) return FA_ENOTSUP;
  if (rank > 0 && (dst_strides == nullptr || src_strides == nullptr || shape == nullptr))
    return FA_EINVAL;
  for (int i = 0; i < rank; i++)
    if (shape[i] < 0) return FA_EINVAL;
  if (dst == nullptr || src == nullptr) {
    int64_t count = 1;
    for (int i = 0; i < rank; i++) count *= shape[i];
    if (path) *path = FA_LMAD_NOTHING;
    return count == 0 ? 0 : FA_EINVAL;
  }
  hipStream_t st = (hipStream_t)stream;
#define FA_LMAD(T)                                                                             \
  return fa::lmad_copy_typed<T>(st, (T *)dst, dst_offset, dst_strides, (const T *)src,         \
                                src_offset, src_strides, shape, rank, path)
  switch (elem_bytes) {
    case 1: FA_LMAD(uint8_t);
    case 2: FA_LMAD(uint16_t);
    case 4: FA_LMAD(uint32_t);
    case 8: FA_LMAD(uint64_t);
    default: return FA_ENOTSUP;
  }
#undef FA_LMAD
}

extern "C" int fa_map_transpose(fa_stream_t stream, int elem_bytes, void *dst, const void *src,
                                int64_t batch, int64_t rows, int64_t cols) {
  if (batch < 0 || rows < 0 || cols < 0) return FA_EINVAL;
  if (batch == 0 || rows == 0 || cols == 0) return 0;
  if (dst == nullptr || src == nullptr) return FA_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  switch (elem_bytes) {
    case 1: return fa::launch_map_transpose<uint8_t>(st, (uint8_t *)dst, (const uint8_t *)src, batch, rows, cols);
    case 2: return fa::launch_map_transpose<uint16_t>(st, (uint16_t *)dst, (const uint16_t *)src, batch, rows, cols);
    case 4: return fa::launch_map_transpose<uint32_t>(st, (uint32_t *)dst, (const uint32_t *)src, batch, rows, cols);
    case 8: return fa::launch_map_transpose<uint64_t>(st, (uint64_t *)dst, (const uint64_t *)src, batch, rows, cols);
    default: return FA_ENOTSUP;
  }
}
