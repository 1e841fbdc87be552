// Tiled SegMap for map-reduce contractions (batched matrix product) on gfx950.
//
// Computes what the reference's block/register tiling computes
// (src/Futhark/Optimise/BlkRegTiling.hs:463-621 for
//  map (\Arow -> map (\Bcol -> reduce (+) 0 (map2 (*) Arow Bcol)) (transpose B)) A,
//  tests/reg-tiling/mmm.fut:17-21): C[b][i][j] = sum_k A[b][i][k] * B[b][k][j]
// with products and sums in f32.  The schedule is CDNA4's, not the
// reference's scalar-FMA 32x32x(2x2) tiling:
//   * a block computes a 256x256 tile of C with four waves, each wave a
//     128x128 sub-tile as 4x4 MFMA tiles of 32x32 (256 accumulator registers);
//   * f16/bf16 use v_mfma_f32_32x32x16, f32 uses v_mfma_f32_32x32x2;
//   * A tiles sit in LDS as [m][k] with a 16-byte XOR swizzle so that the
//     128-bit fragment reads of 8 consecutive rows hit distinct banks;
//   * B stays row-major [k][n] all the way into LDS; the f16/bf16 fragments
//     (8 consecutive k for one n) come out of LDS through the transposing read
//     ds_read_b64_tr_b16, so B is never transposed in memory (the reference
//     may materialise `transpose B` with map_transpose);
//   * global loads for tile k+1 are in flight while tile k is multiplied; LDS
//     is double buffered, one barrier per k-step.
// Shapes that are not multiples of the tile go to a plain LDS-tiled kernel.
#include "dispatch.hip.h"

namespace fa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

constexpr int MM_BM = 256, MM_BN = 256;
constexpr int MM_XCDS = 8;
constexpr int MM_GROUP_M = 4;

// Block -> C tile.  Consecutive block ids land on different XCDs (id mod 8),
// each with its own L2.  The ids of one XCD are therefore made consecutive
// first (id' = xcd * per_xcd + id / 8) and then walked in groups of
// MM_GROUP_M tile rows, so that the 32 tiles an XCD works on at a time form a
// compact 4 x 8 patch: it streams 4 row panels of A and 8 column panels of B
// through its L2 instead of 16 + 2.
__device__ __forceinline__ void mm_tile_of_block(int &tile_m, int &tile_n) {
  const int tiles_n = gridDim.x, tiles_m = gridDim.y;
  const int total = tiles_m * tiles_n;
  int id = blockIdx.y * tiles_n + blockIdx.x;
  if (total % MM_XCDS == 0) id = (id % MM_XCDS) * (total / MM_XCDS) + id / MM_XCDS;
  const int width = MM_GROUP_M * tiles_n;
  const int group = id / width;
  const int first_m = group * MM_GROUP_M;
  const int rows = tiles_m - first_m < MM_GROUP_M ? tiles_m - first_m : MM_GROUP_M;
  tile_m = first_m + (id % width) % rows;
  tile_n = (id % width) / rows;
}
constexpr int MM_THREADS = 256;
constexpr int MM_A_ROW_BYTES = 64;                     // one k-step of a row of A
constexpr int MM_A_TILE_BYTES = MM_BM * MM_A_ROW_BYTES;  // 16 KiB

// ---------------------------------------------------------------- 16-bit inputs
// k-step: 64 elements, i.e. 128-byte rows of A (eight 16-byte units, XOR
// swizzled with the low three bits of the row) and 64 rows of B of 256
// elements, row stride padded by 32 bytes so that the four rows touched by one
// transposing read fall on different banks.  A step is 64 MFMAs per wave,
// long enough to hide the HBM/L2 latency of the loads for the next step.
constexpr int MM16_BK = 64;
constexpr int MM16_A_ROW_BYTES = MM16_BK * 2;
constexpr int MM16_A_TILE_BYTES = MM_BM * MM16_A_ROW_BYTES;  // 32 KiB
constexpr int MM16_B_STRIDE = MM_BN * 2 + 32;                // bytes
constexpr int MM16_B_TILE_BYTES = MM16_BK * MM16_B_STRIDE;
constexpr int MM16_STAGE_BYTES = MM16_A_TILE_BYTES + MM16_B_TILE_BYTES;
constexpr int MM16_UNITS = 8;  // 16-byte units per thread per operand per step

__device__ __forceinline__ int a16_swizzled_offset(int m, int unit) {
  return m * MM16_A_ROW_BYTES + ((unit ^ (m & 7)) << 4);
}

template <bool BF16>
__global__ __launch_bounds__(MM_THREADS) void matmul16_kernel(const uint16_t *__restrict__ A,
                                                              const uint16_t *__restrict__ B,
                                                              float *__restrict__ C, int M, int N,
                                                              int K) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t batch = blockIdx.z;
  int tile_m, tile_n;
  mm_tile_of_block(tile_m, tile_n);
  const int bm = tile_m * MM_BM, bn = tile_n * MM_BN;
  const uint16_t *Ab = A + batch * (int64_t)M * K;
  const uint16_t *Bb = B + batch * (int64_t)K * N;
  float *Cb = C + batch * (int64_t)M * N;

  // This thread's 16-byte units of the A tile and of the B tile: unit i is
  // 32 rows of A (8 rows of B) below unit 0, so one base address each and
  // constant strides describe all of them.
  const int am0 = tid >> 3, au = tid & 7;
  const int bk0 = tid >> 5, bu = tid & 31;
  // Addresses are a block-uniform base (scalar registers) plus one 32-bit
  // per-thread byte offset, which keeps the 16 loads of a step off the vector
  // register budget.
  const char *a_base = reinterpret_cast<const char *>(Ab + (int64_t)bm * K);
  const char *b_base = reinterpret_cast<const char *>(Bb + bn);
  const uint32_t a_toff = (uint32_t)(am0 * K + au * 8) * 2u;
  const uint32_t b_toff = (uint32_t)(bk0 * N + bu * 8) * 2u;
  const int64_t a_src_step = (int64_t)32 * K * 2;  // bytes between units
  const int64_t b_src_step = (int64_t)8 * N * 2;
  const int a_dst0 = a16_swizzled_offset(am0, au);  // (am0 + 32 i) & 7 == am0 & 7
  const int b_dst0 = MM16_A_TILE_BYTES + bk0 * MM16_B_STRIDE + bu * 16;
  constexpr int a_dst_step = 32 * MM16_A_ROW_BYTES;
  constexpr int b_dst_step = 8 * MM16_B_STRIDE;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  const int KT = K / MM16_BK;
#pragma unroll
  for (int i = 0; i < MM16_UNITS; i++) {
    *reinterpret_cast<uint4 *>(lds + a_dst0 + i * a_dst_step) =
        *reinterpret_cast<const uint4 *>(a_base + i * a_src_step + a_toff);
    *reinterpret_cast<uint4 *>(lds + b_dst0 + i * b_dst_step) =
        *reinterpret_cast<const uint4 *>(b_base + i * b_src_step + b_toff);
  }
  __syncthreads();

  // Fragment addresses inside a stage (k16 step 0; later steps add constants).
  const int a_row = wm * 128 + (lane & 31);  // + mt * 32
  const int a_half = lane >> 5;              // which 8 of the 16 k of a step
  int b_frag[4];                             // [n-tile], first of the two transposing reads
  {
    const int r = lane & 15;
    const int kbase = (lane >> 5) * 8 + (r >> 2);
#pragma unroll
    for (int nt = 0; nt < 4; nt++) {
      const int n0 = wn * 128 + nt * 32 + ((lane >> 4) & 1) * 16 + 4 * (r & 3);
      b_frag[nt] = MM16_A_TILE_BYTES + kbase * MM16_B_STRIDE + n0 * 2;
    }
  }

  auto multiply = [&](const unsigned char *stage) {
#pragma unroll
    for (int ks = 0; ks < MM16_BK / 16; ks++) {
      uint4 af[4], bf[4];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
        af[mt] = *reinterpret_cast<const uint4 *>(
            stage + a16_swizzled_offset(a_row + mt * 32, ks * 2 + a_half));
#pragma unroll
      for (int nt = 0; nt < 4; nt++) {
        const unsigned char *p = stage + b_frag[nt] + ks * 16 * MM16_B_STRIDE;
        const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (i16x4 __attribute__((address_space(3))) *)(p));
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (i16x4 __attribute__((address_space(3))) *)(p + 4 * MM16_B_STRIDE));
        uint2 l2 = bit_cast<uint2>(lo), h2 = bit_cast<uint2>(hi);
        bf[nt] = make_uint4(l2.x, l2.y, h2.x, h2.y);
      }
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
          if constexpr (BF16) {
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                bit_cast<bf16x8>(af[mt]), bit_cast<bf16x8>(bf[nt]), acc[mt][nt], 0, 0, 0);
          } else {
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                bit_cast<f16x8>(af[mt]), bit_cast<f16x8>(bf[nt]), acc[mt][nt], 0, 0, 0);
          }
        }
    }
  };

  // Steady state.  Two register sets hold the tiles that are in flight from
  // HBM/L2: while tile kt is multiplied out of LDS, tile kt+1 (requested one
  // step earlier) is parked in the other LDS stage and tile kt+2 is requested.
  // A load therefore has two multiply steps (128 MFMAs per wave) to arrive.
  // The staged tiles are individual registers on purpose: as arrays carried
  // around the loop they were kept in scratch memory by the compiler.
  static_assert(MM16_UNITS == 8, "the staging code below is written out for 8 units");
  uint4 pa0, pa1, pa2, pa3, pa4, pa5, pa6, pa7, pb0, pb1, pb2, pb3, pb4, pb5, pb6, pb7, qa0, qa1, qa2, qa3, qa4, qa5, qa6, qa7, qb0, qb1, qb2, qb3, qb4, qb5, qb6, qb7;
#define MM16_KOFF(T) const int64_t koff_ = (int64_t)((T) > KT - 1 ? KT - 1 : (T)) * MM16_BK * 2
#define MM16_FETCH_P(T) \
  do { \
    MM16_KOFF(T); \
    pa0 = *reinterpret_cast<const uint4 *>(a_base + (0 * a_src_step + koff_) + a_toff); \
    pb0 = *reinterpret_cast<const uint4 *>(b_base + (0 * b_src_step + koff_ * N) + b_toff); \
    pa1 = *reinterpret_cast<const uint4 *>(a_base + (1 * a_src_step + koff_) + a_toff); \
    pb1 = *reinterpret_cast<const uint4 *>(b_base + (1 * b_src_step + koff_ * N) + b_toff); \
    pa2 = *reinterpret_cast<const uint4 *>(a_base + (2 * a_src_step + koff_) + a_toff); \
    pb2 = *reinterpret_cast<const uint4 *>(b_base + (2 * b_src_step + koff_ * N) + b_toff); \
    pa3 = *reinterpret_cast<const uint4 *>(a_base + (3 * a_src_step + koff_) + a_toff); \
    pb3 = *reinterpret_cast<const uint4 *>(b_base + (3 * b_src_step + koff_ * N) + b_toff); \
    pa4 = *reinterpret_cast<const uint4 *>(a_base + (4 * a_src_step + koff_) + a_toff); \
    pb4 = *reinterpret_cast<const uint4 *>(b_base + (4 * b_src_step + koff_ * N) + b_toff); \
    pa5 = *reinterpret_cast<const uint4 *>(a_base + (5 * a_src_step + koff_) + a_toff); \
    pb5 = *reinterpret_cast<const uint4 *>(b_base + (5 * b_src_step + koff_ * N) + b_toff); \
    pa6 = *reinterpret_cast<const uint4 *>(a_base + (6 * a_src_step + koff_) + a_toff); \
    pb6 = *reinterpret_cast<const uint4 *>(b_base + (6 * b_src_step + koff_ * N) + b_toff); \
    pa7 = *reinterpret_cast<const uint4 *>(a_base + (7 * a_src_step + koff_) + a_toff); \
    pb7 = *reinterpret_cast<const uint4 *>(b_base + (7 * b_src_step + koff_ * N) + b_toff); \
  } while (0)
#define MM16_FETCH_Q(T) \
  do { \
    MM16_KOFF(T); \
    qa0 = *reinterpret_cast<const uint4 *>(a_base + (0 * a_src_step + koff_) + a_toff); \
    qb0 = *reinterpret_cast<const uint4 *>(b_base + (0 * b_src_step + koff_ * N) + b_toff); \
    qa1 = *reinterpret_cast<const uint4 *>(a_base + (1 * a_src_step + koff_) + a_toff); \
    qb1 = *reinterpret_cast<const uint4 *>(b_base + (1 * b_src_step + koff_ * N) + b_toff); \
    qa2 = *reinterpret_cast<const uint4 *>(a_base + (2 * a_src_step + koff_) + a_toff); \
    qb2 = *reinterpret_cast<const uint4 *>(b_base + (2 * b_src_step + koff_ * N) + b_toff); \
    qa3 = *reinterpret_cast<const uint4 *>(a_base + (3 * a_src_step + koff_) + a_toff); \
    qb3 = *reinterpret_cast<const uint4 *>(b_base + (3 * b_src_step + koff_ * N) + b_toff); \
    qa4 = *reinterpret_cast<const uint4 *>(a_base + (4 * a_src_step + koff_) + a_toff); \
    qb4 = *reinterpret_cast<const uint4 *>(b_base + (4 * b_src_step + koff_ * N) + b_toff); \
    qa5 = *reinterpret_cast<const uint4 *>(a_base + (5 * a_src_step + koff_) + a_toff); \
    qb5 = *reinterpret_cast<const uint4 *>(b_base + (5 * b_src_step + koff_ * N) + b_toff); \
    qa6 = *reinterpret_cast<const uint4 *>(a_base + (6 * a_src_step + koff_) + a_toff); \
    qb6 = *reinterpret_cast<const uint4 *>(b_base + (6 * b_src_step + koff_ * N) + b_toff); \
    qa7 = *reinterpret_cast<const uint4 *>(a_base + (7 * a_src_step + koff_) + a_toff); \
    qb7 = *reinterpret_cast<const uint4 *>(b_base + (7 * b_src_step + koff_ * N) + b_toff); \
  } while (0)
#define MM16_PARK_P(STAGE) \
  do { \
    unsigned char *dst_ = lds + (STAGE)*MM16_STAGE_BYTES; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 0 * a_dst_step) = pa0; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 0 * b_dst_step) = pb0; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 1 * a_dst_step) = pa1; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 1 * b_dst_step) = pb1; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 2 * a_dst_step) = pa2; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 2 * b_dst_step) = pb2; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 3 * a_dst_step) = pa3; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 3 * b_dst_step) = pb3; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 4 * a_dst_step) = pa4; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 4 * b_dst_step) = pb4; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 5 * a_dst_step) = pa5; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 5 * b_dst_step) = pb5; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 6 * a_dst_step) = pa6; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 6 * b_dst_step) = pb6; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 7 * a_dst_step) = pa7; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 7 * b_dst_step) = pb7; \
  } while (0)
#define MM16_PARK_Q(STAGE) \
  do { \
    unsigned char *dst_ = lds + (STAGE)*MM16_STAGE_BYTES; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 0 * a_dst_step) = qa0; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 0 * b_dst_step) = qb0; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 1 * a_dst_step) = qa1; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 1 * b_dst_step) = qb1; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 2 * a_dst_step) = qa2; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 2 * b_dst_step) = qb2; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 3 * a_dst_step) = qa3; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 3 * b_dst_step) = qb3; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 4 * a_dst_step) = qa4; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 4 * b_dst_step) = qb4; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 5 * a_dst_step) = qa5; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 5 * b_dst_step) = qb5; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 6 * a_dst_step) = qa6; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 6 * b_dst_step) = qb6; \
    *reinterpret_cast<uint4 *>(dst_ + a_dst0 + 7 * a_dst_step) = qa7; \
    *reinterpret_cast<uint4 *>(dst_ + b_dst0 + 7 * b_dst_step) = qb7; \
  } while (0)
  MM16_FETCH_P(1);
  for (int kt = 0; kt + 1 < KT; kt += 2) {
    MM16_FETCH_Q(kt + 2);
    __builtin_amdgcn_sched_barrier(0);
    multiply(lds);  // tile kt sits in stage 0
    __builtin_amdgcn_sched_barrier(0);
    MM16_PARK_P(1);
    __syncthreads();
    MM16_FETCH_P(kt + 3);
    __builtin_amdgcn_sched_barrier(0);
    multiply(lds + MM16_STAGE_BYTES);  // tile kt+1
    __builtin_amdgcn_sched_barrier(0);
    if (kt + 2 < KT) MM16_PARK_Q(0);
    __syncthreads();
  }
#undef MM16_KOFF
#undef MM16_FETCH_P
#undef MM16_FETCH_Q
#undef MM16_PARK_P
#undef MM16_PARK_Q
  if (KT & 1) multiply(lds);  // odd count: the last tile was parked in stage 0

  // C fragment: element e of lane l is row (e/4)*8 + (l/32)*4 + e%4, column l%32.
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int row = bm + wm * 128 + mt * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        const int col = bn + wn * 128 + nt * 32 + (lane & 31);
        Cb[(int64_t)row * N + col] = acc[mt][nt][e];
      }
}

// ---------------------------------------------------------------- f32 inputs
// k-step: 16 elements.  A tile rows are again 64 bytes (same swizzle); B tile is
// 16 rows of 256 floats.
__device__ __forceinline__ int a_swizzled_offset(int m, int unit) {
  return m * MM_A_ROW_BYTES + ((unit ^ ((m >> 1) & 3)) << 4);
}

constexpr int MM32_BK = 16;
constexpr int MM32_B_STRIDE = MM_BN * 4;  // bytes
constexpr int MM32_B_TILE_BYTES = MM32_BK * MM32_B_STRIDE;
constexpr int MM32_STAGE_BYTES = MM_A_TILE_BYTES + MM32_B_TILE_BYTES;

__global__ __launch_bounds__(MM_THREADS) void matmul32_kernel(const float *__restrict__ A,
                                                              const float *__restrict__ B,
                                                              float *__restrict__ C, int M, int N,
                                                              int K) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t batch = blockIdx.z;
  int tile_m, tile_n;
  mm_tile_of_block(tile_m, tile_n);
  const int bm = tile_m * MM_BM, bn = tile_n * MM_BN;
  const float *Ab = A + batch * (int64_t)M * K;
  const float *Bb = B + batch * (int64_t)K * N;
  float *Cb = C + batch * (int64_t)M * N;

  const float *a_src[4];
  const float *b_src[4];
  int a_dst[4], b_dst[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int q = tid + MM_THREADS * i;
    const int am = q >> 2, au = q & 3;
    a_src[i] = Ab + (int64_t)(bm + am) * K + au * 4;
    a_dst[i] = a_swizzled_offset(am, au);
    const int bk = q >> 6, bu = q & 63;
    b_src[i] = Bb + (int64_t)bk * N + bn + bu * 4;
    b_dst[i] = MM_A_TILE_BYTES + bk * MM32_B_STRIDE + bu * 16;
  }

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  const int KT = K / MM32_BK;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    *reinterpret_cast<uint4 *>(lds + a_dst[i]) = *reinterpret_cast<const uint4 *>(a_src[i]);
    *reinterpret_cast<uint4 *>(lds + b_dst[i]) = *reinterpret_cast<const uint4 *>(b_src[i]);
  }
  __syncthreads();

  // Lane group g = lane/32 owns k = g*4 + s (s = 0..3) of each group of 8 k.
  int a_frag[4][2];  // [m-tile][group of 8 k]
#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int kg = 0; kg < 2; kg++) {
      const int m = wm * 128 + mt * 32 + (lane & 31);
      a_frag[mt][kg] = a_swizzled_offset(m, kg * 2 + (lane >> 5));
    }
  const int b_frag = MM_A_TILE_BYTES + (lane >> 5) * 4 * MM32_B_STRIDE +
                     (wn * 128 + (lane & 31)) * 4;

  auto multiply = [&](const unsigned char *stage) {
#pragma unroll
    for (int kg = 0; kg < 2; kg++) {
      float4 af[4];
#pragma unroll
      for (int mt = 0; mt < 4; mt++)
        af[mt] = *reinterpret_cast<const float4 *>(stage + a_frag[mt][kg]);
#pragma unroll
      for (int s = 0; s < 4; s++) {
        float bf[4];
#pragma unroll
        for (int nt = 0; nt < 4; nt++)
          bf[nt] = *reinterpret_cast<const float *>(stage + b_frag +
                                                    (kg * 8 + s) * MM32_B_STRIDE + nt * 32 * 4);
#pragma unroll
        for (int mt = 0; mt < 4; mt++) {
          const float a = s == 0 ? af[mt].x : (s == 1 ? af[mt].y : (s == 2 ? af[mt].z : af[mt].w));
#pragma unroll
          for (int nt = 0; nt < 4; nt++)
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bf[nt], acc[mt][nt], 0, 0, 0);
        }
      }
    }
  };

  for (int kt = 0; kt + 1 < KT; kt++) {
    uint4 ra0 = *reinterpret_cast<const uint4 *>(a_src[0] + (int64_t)(kt + 1) * MM32_BK);
    uint4 ra1 = *reinterpret_cast<const uint4 *>(a_src[1] + (int64_t)(kt + 1) * MM32_BK);
    uint4 ra2 = *reinterpret_cast<const uint4 *>(a_src[2] + (int64_t)(kt + 1) * MM32_BK);
    uint4 ra3 = *reinterpret_cast<const uint4 *>(a_src[3] + (int64_t)(kt + 1) * MM32_BK);
    uint4 rb0 = *reinterpret_cast<const uint4 *>(b_src[0] + (int64_t)(kt + 1) * MM32_BK * N);
    uint4 rb1 = *reinterpret_cast<const uint4 *>(b_src[1] + (int64_t)(kt + 1) * MM32_BK * N);
    uint4 rb2 = *reinterpret_cast<const uint4 *>(b_src[2] + (int64_t)(kt + 1) * MM32_BK * N);
    uint4 rb3 = *reinterpret_cast<const uint4 *>(b_src[3] + (int64_t)(kt + 1) * MM32_BK * N);
    __builtin_amdgcn_sched_barrier(0);
    multiply(lds + (kt & 1) * MM32_STAGE_BYTES);
    __builtin_amdgcn_sched_barrier(0);
    unsigned char *next = lds + ((kt + 1) & 1) * MM32_STAGE_BYTES;
    *reinterpret_cast<uint4 *>(next + a_dst[0]) = ra0;
    *reinterpret_cast<uint4 *>(next + a_dst[1]) = ra1;
    *reinterpret_cast<uint4 *>(next + a_dst[2]) = ra2;
    *reinterpret_cast<uint4 *>(next + a_dst[3]) = ra3;
    *reinterpret_cast<uint4 *>(next + b_dst[0]) = rb0;
    *reinterpret_cast<uint4 *>(next + b_dst[1]) = rb1;
    *reinterpret_cast<uint4 *>(next + b_dst[2]) = rb2;
    *reinterpret_cast<uint4 *>(next + b_dst[3]) = rb3;
    __syncthreads();
  }
  multiply(lds + ((KT - 1) & 1) * MM32_STAGE_BYTES);

#pragma unroll
  for (int mt = 0; mt < 4; mt++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int row = bm + wm * 128 + mt * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        const int col = bn + wn * 128 + nt * 32 + (lane & 31);
        Cb[(int64_t)row * N + col] = acc[mt][nt][e];
      }
}

// ------------------------------------------------------------- any shape
// 64x64 tile of C per block, 16 k per step, 4x4 outputs per thread, scalar FMA
// in k order.  Serves shapes the MFMA kernels do not cover.
__device__ __forceinline__ float widen(float x) { return x; }
template <bool BF16> __device__ __forceinline__ float widen16(uint16_t x) {
  if (BF16) return bit_cast<float>((uint32_t)x << 16);
  return (float)bit_cast<_Float16>(x);
}

template <class InT, int KIND /*0 f32, 1 f16, 2 bf16*/>
__global__ __launch_bounds__(256) void matmul_generic_kernel(const InT *__restrict__ A,
                                                             const InT *__restrict__ B,
                                                             float *__restrict__ C, int64_t M,
                                                             int64_t N, int64_t K) {
  __shared__ float As[16][64 + 1];
  __shared__ float Bs[16][64 + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int64_t batch = blockIdx.z;
  const int64_t bm = (int64_t)blockIdx.y * 64, bn = (int64_t)blockIdx.x * 64;
  const InT *Ab = A + batch * M * K;
  const InT *Bb = B + batch * K * N;
  float *Cb = C + batch * M * N;
  auto cvt = [](InT x) -> float {
    if constexpr (KIND == 0) return x;
    else return widen16<KIND == 2>(x);
  };
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < K; k0 += 16) {
    for (int i = tid; i < 64 * 16; i += 256) {
      const int m = i >> 4, k = i & 15;
      As[k][m] = (bm + m < M && k0 + k < K) ? cvt(Ab[(bm + m) * K + k0 + k]) : 0.0f;
      const int kk = i >> 6, n = i & 63;
      Bs[kk][n] = (k0 + kk < K && bn + n < N) ? cvt(Bb[(k0 + kk) * N + bn + n]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int64_t r = bm + ty * 4 + i, c = bn + tx * 4 + j;
      if (r < M && c < N) Cb[r * N + c] = acc[i][j];
    }
}

template <class Kern> static int raise_lds(Kern k, int bytes) {
  hipError_t e = hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  return e == hipSuccess ? 0 : (int)e;
}

}  // namespace fa

extern "C" int fa_matmul(fa_stream_t stream, fa_dtype in_t, const void *A, const void *B, float *C,
                         int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch < 0 || M < 0 || N < 0 || K < 0) return FA_EINVAL;
  if (in_t != FA_F32 && in_t != FA_F16 && in_t != FA_BF16) return FA_ENOTSUP;
  if (batch * M * N == 0) return 0;
  if (C == nullptr || (K > 0 && (A == nullptr || B == nullptr))) return FA_EINVAL;
  if (batch > 65535 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return FA_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const int bk = in_t == FA_F32 ? MM32_BK : MM16_BK;
  const bool tiled = M % MM_BM == 0 && N % MM_BN == 0 && K % bk == 0 && K > 0 &&
                     is_aligned(A, 16) && is_aligned(B, 16) && is_aligned(C, 16);
  if (tiled) {
    const dim3 grid((unsigned)(N / MM_BN), (unsigned)(M / MM_BM), (unsigned)batch);
    int rc = 0;
    if (in_t == FA_F32) {
      static bool raised = false;
      if (!raised) { rc = raise_lds(matmul32_kernel, 2 * MM32_STAGE_BYTES); raised = rc == 0; }
      if (rc) return rc;
      hipLaunchKernelGGL(matmul32_kernel, grid, dim3(MM_THREADS), 2 * MM32_STAGE_BYTES, st,
                         (const float *)A, (const float *)B, C, (int)M, (int)N, (int)K);
    } else if (in_t == FA_F16) {
      static bool raised = false;
      if (!raised) { rc = raise_lds(matmul16_kernel<false>, 2 * MM16_STAGE_BYTES); raised = rc == 0; }
      if (rc) return rc;
      hipLaunchKernelGGL((matmul16_kernel<false>), grid, dim3(MM_THREADS), 2 * MM16_STAGE_BYTES, st,
                         (const uint16_t *)A, (const uint16_t *)B, C, (int)M, (int)N, (int)K);
    } else {
      static bool raised = false;
      if (!raised) { rc = raise_lds(matmul16_kernel<true>, 2 * MM16_STAGE_BYTES); raised = rc == 0; }
      if (rc) return rc;
      hipLaunchKernelGGL((matmul16_kernel<true>), grid, dim3(MM_THREADS), 2 * MM16_STAGE_BYTES, st,
                         (const uint16_t *)A, (const uint16_t *)B, C, (int)M, (int)N, (int)K);
    }
    return launch_status();
  }
  const dim3 grid((unsigned)ceil_div(N, 64), (unsigned)ceil_div(M, 64), (unsigned)batch);
  if (grid.y > 65535) return FA_EINVAL;
  if (in_t == FA_F32)
    hipLaunchKernelGGL((matmul_generic_kernel<float, 0>), grid, dim3(256), 0, st, (const float *)A,
                       (const float *)B, C, M, N, K);
  else if (in_t == FA_F16)
    hipLaunchKernelGGL((matmul_generic_kernel<uint16_t, 1>), grid, dim3(256), 0, st,
                       (const uint16_t *)A, (const uint16_t *)B, C, M, N, K);
  else
    hipLaunchKernelGGL((matmul_generic_kernel<uint16_t, 2>), grid, dim3(256), 0, st,
                       (const uint16_t *)A, (const uint16_t *)B, C, M, N, K);
  return launch_status();
}
