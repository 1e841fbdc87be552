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
//     128-bit fragment reads hit distinct banks;
//   * B stays row-major [k][n] all the way into LDS; the f16/bf16 fragments
//     (8 consecutive k for one n) come out of LDS through the transposing read
//     ds_read_b64_tr_b16, so B is never transposed in memory (the reference
//     may materialise `transpose B` with map_transpose);
//   * LDS is double buffered, one barrier per k-step; f16/bf16 tiles go from
//     global memory straight into LDS (no register staging) while the previous
//     tile is multiplied, with the MFMA / LDS-read / load order fixed by hand.
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

// Block -> (matrix of the batch, C tile).  Blocks are dispatched in the order
// of their linear id (x fastest, then y, then z) and consecutive ids land on
// different XCDs (id mod 8), each with its own L2.  The ids of one XCD are
// therefore made consecutive first (id' = xcd * per_xcd + id / 8), over the
// whole batch, and then walked matrix by matrix and, inside a matrix, in groups
// of MM_GROUP_M tile rows: the 32 tiles of a large matrix that an XCD works on
// at a time form a compact 4 x 8 patch (it streams 4 row panels of A and 8
// column panels of B through its L2 instead of 16 + 2), and the few tiles of a
// small matrix of a batch all run on one XCD, where the second tile that needs
// a panel finds it in L2 (64 products of 512^3 f16, four tiles each: with the
// tiles of a matrix on four XCDs every panel came from memory twice, 134 MB
// fetched instead of 67, and the launch took 33 us).
__device__ __forceinline__ void mm_tile_of_block(int64_t &batch, int &tile_m, int &tile_n) {
  const int tiles_n = gridDim.x, tiles_m = gridDim.y;
  const int64_t per_matrix = (int64_t)tiles_m * tiles_n;
  const int64_t total = per_matrix * gridDim.z;
  int64_t id = ((int64_t)blockIdx.z * tiles_m + blockIdx.y) * tiles_n + blockIdx.x;
  if (total % MM_XCDS == 0) id = (id % MM_XCDS) * (total / MM_XCDS) + id / MM_XCDS;
  batch = id / per_matrix;
  const int in_matrix = (int)(id % per_matrix);
  const int width = MM_GROUP_M * tiles_n;
  const int group = in_matrix / width;
  const int first_m = group * MM_GROUP_M;
  const int rows = tiles_m - first_m < MM_GROUP_M ? tiles_m - first_m : MM_GROUP_M;
  tile_m = first_m + (in_matrix % width) % rows;
  tile_n = (in_matrix % width) / rows;
}
constexpr int MM_THREADS = 256;
constexpr int MM_A_ROW_BYTES = 64;                     // one k-step of a row of A
constexpr int MM_A_TILE_BYTES = MM_BM * MM_A_ROW_BYTES;  // 16 KiB

// ---------------------------------------------------------------- 16-bit inputs
// k-step: 64 elements.  Tiles travel from global memory straight into LDS
// (global_load_lds_dwordx4: lane l of a wave deposits 16 bytes at M0 + 16 l, so
// one instruction fills 1 KiB of LDS and the swizzles below are applied by
// choosing which global unit each lane fetches):
//   A: 256 rows of 128 bytes, eight 16-byte units per row; unit u of row m sits
//      in slot u ^ ((m >> 1) & 7), so the 16 lanes of one phase of a 128-bit
//      fragment read (16 consecutive rows, one unit) cover all 64 banks once;
//   B: 64 rows [k] of 512 bytes (256 n), 32 units per row; unit u of row k sits
//      in slot u ^ ((k & 3) << 2), so the four rows touched by one transposing
//      read (64 bytes each) fall into different 64-byte bank groups.
// Nothing is staged in registers, and LDS is double buffered with one barrier
// per k-step.
constexpr int MM16_BK = 64;
constexpr int MM16_A_ROW_BYTES = MM16_BK * 2;
constexpr int MM16_A_TILE_BYTES = MM_BM * MM16_A_ROW_BYTES;  // 32 KiB
constexpr int MM16_B_ROW_BYTES = MM_BN * 2;
constexpr int MM16_B_TILE_BYTES = MM16_BK * MM16_B_ROW_BYTES;  // 32 KiB
constexpr int MM16_STAGE_BYTES = MM16_A_TILE_BYTES + MM16_B_TILE_BYTES;
// Four waves in a 2 x 2 arrangement, each computing a 128 x 128 sub-tile (4 x 4
// MFMA tiles, 256 accumulator registers): the arrangement with the least LDS
// read traffic per MFMA (8 waves as 2 x 4 measured the same speed).
constexpr int MM16_WAVES_M = 2, MM16_WAVES_N = 2;
constexpr int MM16_WAVES = MM16_WAVES_M * MM16_WAVES_N;
constexpr int MM16_THREADS = 64 * MM16_WAVES;
constexpr int MM16_MT = MM_BM / (MM16_WAVES_M * 32);  // MFMA tiles per wave along m
constexpr int MM16_NT = MM_BN / (MM16_WAVES_N * 32);  // and along n
constexpr int MM16_CHUNKS = MM16_A_TILE_BYTES / 1024 / MM16_WAVES;  // 1 KiB loads per wave, per operand
// The loads of the next tile ride on the first two k16 steps of a tile, which
// leaves them the other two steps to land before the barrier.
constexpr int MM16_LOAD_KSTEPS = 2;

__device__ __forceinline__ int a16_swizzled_offset(int m, int unit) {
  return m * MM16_A_ROW_BYTES + ((unit ^ ((m >> 1) & 7)) << 4);
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order: a
// loop whose index is a compile-time constant in every iteration.
template <int N, class F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// One direct global -> LDS load of 16 bytes per lane.  `lds_addr` (wave
// uniform) goes to M0; the kernel has no other user of M0.  The compiler does
// not track this load: the caller waits for vmcnt before the barrier that
// publishes the tile.
// The source is a wave-uniform base (scalar registers) plus a 32-bit per-lane
// byte offset, so the loads of a tile cost no vector registers for addresses.
__device__ __forceinline__ void load_to_lds_16(const char *uniform_base, uint32_t lane_offset,
                                               uint32_t lds_addr) {
  const uint64_t base = (uint64_t)uniform_base;
  const uint64_t sbase =
      ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(base >> 32)) << 32) |
      (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(
                   __builtin_amdgcn_readfirstlane(lds_addr)),
               "v"(lane_offset), "s"(sbase)
               : "memory", "m0");
}

// BM x BN: the block's tile of C; WAVES_M x WAVES_N: how its waves share it.
// 256 x 256 with 2 x 2 waves is the kernel for large products (one block per
// CU, the least LDS traffic per MFMA); 128 x 128 with 1 x 2 waves takes shapes
// that are multiples of 128 only.
template <bool BF16, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void matmul16_kernel(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, float *__restrict__ C, int M,
    int N, int K) {
  constexpr int MM16_WAVES = WAVES_M * WAVES_N;
  constexpr int MM16_WAVES_N = WAVES_N;
  constexpr int MM_BM = BM, MM_BN = BN;
  constexpr int MM16_A_TILE_BYTES = BM * MM16_A_ROW_BYTES;
  constexpr int MM16_B_ROW_BYTES = BN * 2;
  constexpr int MM16_B_TILE_BYTES = MM16_BK * MM16_B_ROW_BYTES;
  constexpr int MM16_STAGE_BYTES = MM16_A_TILE_BYTES + MM16_B_TILE_BYTES;
  constexpr int MM16_MT = BM / (WAVES_M * 32), MM16_NT = BN / (WAVES_N * 32);
  constexpr int MM16_CHUNKS = MM16_A_TILE_BYTES / 1024 / MM16_WAVES;  // 1 KiB loads per wave, per operand
  static_assert(MM16_B_TILE_BYTES == MM16_A_TILE_BYTES, "as many chunks of B as of A");
  constexpr int B_UNITS = MM16_B_ROW_BYTES / 16;  // 16-byte units per row of the B tile
  constexpr int B_ROWS = 1024 / MM16_B_ROW_BYTES;  // rows of the B tile per 1 KiB chunk
  static_assert((B_ROWS * MM16_WAVES) % 4 == 0, "a lane's swizzle term is the same in all its chunks");
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / MM16_WAVES_N, wn = wave % MM16_WAVES_N;
  int64_t batch;
  int tile_m, tile_n;
  mm_tile_of_block(batch, tile_m, tile_n);
  const int bm = tile_m * MM_BM, bn = tile_n * MM_BN;
  const uint16_t *Ab = A + batch * (int64_t)M * K;
  const uint16_t *Bb = B + batch * (int64_t)K * N;
  float *Cb = C + batch * (int64_t)M * N;

  // Loads.  Chunk c of the A tile is rows 8c..8c+7 (1 KiB of LDS), chunk c of
  // the B tile is rows B_ROWS c .. B_ROWS c + B_ROWS - 1.  Wave w moves chunks w, w + WAVES, ...; since
  // WAVES is even the swizzle term of a lane's row does not depend on the
  // chunk, so a lane's chunks differ by a constant stride in global memory.
  static_assert(MM16_WAVES % 2 == 0, "swizzle terms assume an even chunk stride");
  const int a_r = lane >> 3, a_slot = lane & 7;
  const int a_unit = a_slot ^ (((wave & 1) << 2) | (a_r >> 1));  // ((8 w + a_r) >> 1) & 7
  const int b_r = lane / B_UNITS, b_slot = lane % B_UNITS;
  const int b_unit = b_slot ^ (((B_ROWS * wave + b_r) & 3) << 2);  // row k of the tile: (k & 3) << 2
  const char *a_src = reinterpret_cast<const char *>(Ab + (int64_t)(bm + wave * 8) * K);
  const char *b_src = reinterpret_cast<const char *>(Bb + (int64_t)(wave * B_ROWS) * N + bn);
  const uint32_t a_lane = (uint32_t)(a_r * K * 2 + a_unit * 16);  // K, N < 2^27 elements
  const uint32_t b_lane = (uint32_t)(b_r * N * 2 + b_unit * 16);
  const int64_t a_chunk_step = (int64_t)MM16_WAVES * 8 * K * 2;
  const int64_t b_chunk_step = (int64_t)MM16_WAVES * B_ROWS * N * 2;
  const int64_t b_tile_step = (int64_t)MM16_BK * N * 2;
  const uint32_t lds_base =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
  const uint32_t a_dst = lds_base + wave * 1024;
  const uint32_t b_dst = lds_base + MM16_A_TILE_BYTES + wave * 1024;
  // Load j of a tile: even j moves a chunk of A, odd j a chunk of B.
  auto fetch_one = [&](int kt, int stage, int j) __attribute__((always_inline)) {
    const int i = j >> 1;
    if ((j & 1) == 0)
      load_to_lds_16(a_src + (int64_t)kt * (MM16_BK * 2) + i * a_chunk_step, a_lane,
                     a_dst + stage * MM16_STAGE_BYTES + i * (MM16_WAVES * 1024));
    else
      load_to_lds_16(b_src + (int64_t)kt * b_tile_step + i * b_chunk_step, b_lane,
                     b_dst + stage * MM16_STAGE_BYTES + i * (MM16_WAVES * 1024));
  };

  f32x16 acc[MM16_MT][MM16_NT];
#pragma unroll
  for (int i = 0; i < MM16_MT; i++)
#pragma unroll
    for (int j = 0; j < MM16_NT; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  // Fragment addresses inside a stage (k16 step 0; later steps add constants).
  const int a_row = wm * (MM16_MT * 32) + (lane & 31);  // + mt * 32
  const int a_half = lane >> 5;                         // which 8 of the 16 k of a step
  int b_frag[MM16_NT];  // [n-tile], first of the two transposing reads
  {
    // Lane r of a group of 16 supplies the 8 bytes at row kbase + r/4, columns
    // n0 + 4 (r%4) .. +3; the read hands lane j the k-column it needs.
    const int r = lane & 15;
    const int kbase = (lane >> 5) * 8 + (r >> 2);  // kbase & 3 == r >> 2 in every step
#pragma unroll
    for (int nt = 0; nt < MM16_NT; nt++) {
      const int n0 = wn * (MM16_NT * 32) + nt * 32 + ((lane >> 4) & 1) * 16 + 4 * (r & 3);
      const int unit = (n0 >> 3) ^ ((r >> 2) << 2);
      b_frag[nt] = MM16_A_TILE_BYTES + kbase * MM16_B_ROW_BYTES + unit * 16 + (n0 & 7) * 2;
    }
  }

  // A k16 step is MT*NT MFMAs, walked n-tile by n-tile.  Its instruction order
  // is fixed by hand (a scheduling barrier after every MFMA):
  //   * after each of the first MT + 2 NT MFMAs one LDS read of the next step's
  //     fragments is issued (fragments are double buffered), in the order the
  //     next step consumes them: B0, A0..A(MT-1), B1, B2, ...  The last reads
  //     are needed only late in the next step, so no MFMA waits on a read that
  //     was issued just before it;
  //   * after every second MFMA of the first steps one load of the next tile is
  //     issued.  Loads are spread out because a wave that issues many of them
  //     back to back stalls until the memory pipeline has taken them, with its
  //     SIMD's MFMA unit idle meanwhile.
  constexpr int KSTEPS = MM16_BK / 16;
  constexpr int MFMAS = MM16_MT * MM16_NT, READS = MM16_MT + 2 * MM16_NT;
  static_assert(READS <= MFMAS, "one LDS read follows one MFMA");
  constexpr int LOADS = 2 * MM16_CHUNKS;  // per wave and tile
  static_assert(LOADS % MM16_LOAD_KSTEPS == 0, "loads divide evenly over the steps");
  constexpr int LOADS_PER_STEP = LOADS / MM16_LOAD_KSTEPS;
  static_assert(MFMAS % LOADS_PER_STEP == 0, "loads divide evenly over the MFMAs");
  constexpr int MFMAS_PER_LOAD = MFMAS / LOADS_PER_STEP;
  struct Frags {
    uint4 a[MM16_MT];
    uint4 b[MM16_NT];  // .xy: k 0..3|8..11 of the step, .zw: k 4..7|12..15 (one read each)
  };
  auto read_b_half = [&](const unsigned char *stage, int ks, int nt,
                         int half) __attribute__((always_inline)) -> uint2 {
    const unsigned char *p =
        stage + b_frag[nt] + (ks * 16 + half * 4) * MM16_B_ROW_BYTES;
    return bit_cast<uint2>(__builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (i16x4 __attribute__((address_space(3))) *)(p)));
  };
  // Read number `idx` of a step, in consumption order.
  auto issue_read = [&](const unsigned char *stage, int ks, int idx,
                        Frags &f) __attribute__((always_inline)) {
    if (idx < 2) {
      const uint2 h = read_b_half(stage, ks, 0, idx);
      if (idx == 0) f.b[0].x = h.x, f.b[0].y = h.y;
      else f.b[0].z = h.x, f.b[0].w = h.y;
    } else if (idx < 2 + MM16_MT) {
      const int mt = idx - 2;
      f.a[mt] = *reinterpret_cast<const uint4 *>(
          stage + a16_swizzled_offset(a_row + mt * 32, ks * 2 + a_half));
    } else {
      const int j = idx - 2 - MM16_MT, nt = 1 + (j >> 1);
      const uint2 h = read_b_half(stage, ks, nt, j & 1);
      if ((j & 1) == 0) f.b[nt].x = h.x, f.b[nt].y = h.y;
      else f.b[nt].z = h.x, f.b[nt].w = h.y;
    }
  };
  const int KT = K / MM16_BK;
  // All of this wave's loads have landed and its LDS reads have returned, then
  // all waves': the next tile is public and the current one may be overwritten.
  auto publish = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __syncthreads();
  };
  // With more MFMAs in a step than LDS reads (MM16_EARLY), the barrier that
  // publishes the next tile is taken inside the last k16 step of the current
  // one, after MFMA number PUBLISH_AT, and the first fragments of the next tile
  // are read behind the remaining MFMAs: the next tile starts with an MFMA
  // instead of a barrier and a dozen LDS round trips.  (The current tile's LDS
  // bytes are no longer needed by then: the fragments of its last step were
  // read during the step before.)
  constexpr bool MM16_EARLY = MFMAS > READS;
  constexpr int PUBLISH_AT = MFMAS - READS - 1;
  auto k16_step = [&](const unsigned char *stage, const unsigned char *other, int ks,
                      const Frags &cur, Frags &next, int next_kt, int next_stage,
                      auto fetch) __attribute__((always_inline)) {
    static_for<MFMAS>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      constexpr int nt = i / MM16_MT, mt = i % MM16_MT;
      const uint4 bfrag = cur.b[nt];
      if constexpr (BF16) {
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            bit_cast<bf16x8>(cur.a[mt]), bit_cast<bf16x8>(bfrag), acc[mt][nt], 0, 0, 0);
      } else {
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            bit_cast<f16x8>(cur.a[mt]), bit_cast<f16x8>(bfrag), acc[mt][nt], 0, 0, 0);
      }
      if (ks + 1 < KSTEPS) {
        if (i < READS) issue_read(stage, ks + 1, i, next);
      } else if constexpr (MM16_EARLY) {
        if (i == PUBLISH_AT) publish();
        if (i > PUBLISH_AT) issue_read(other, 0, i - PUBLISH_AT - 1, next);
      }
      if constexpr (decltype(fetch)::value)
        if (ks < MM16_LOAD_KSTEPS && i % MFMAS_PER_LOAD == MFMAS_PER_LOAD - 1)
        fetch_one(next_kt, next_stage, ks * LOADS_PER_STEP + i / MFMAS_PER_LOAD);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  Frags f0, f1;
  auto first_reads = [&](const unsigned char *stage) __attribute__((always_inline)) {
    static_for<READS>([&](auto ic) __attribute__((always_inline)) { issue_read(stage, 0, decltype(ic)::value, f0); });
    __builtin_amdgcn_sched_barrier(0);
  };
  auto multiply = [&](const unsigned char *stage, const unsigned char *other, int next_kt,
                      int next_stage, auto fetch) __attribute__((always_inline)) {
    if constexpr (!MM16_EARLY) first_reads(stage);
    static_assert(KSTEPS % 2 == 0, "the fragment buffers swap an even number of times per tile");
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks += 2) {
      k16_step(stage, other, ks, f0, f1, next_kt, next_stage, fetch);
      k16_step(stage, other, ks + 1, f1, f0, next_kt, next_stage, fetch);
    }
    if constexpr (!MM16_EARLY) publish();
  };

#pragma unroll
  for (int j = 0; j < LOADS; j++) fetch_one(0, 0, j);
  publish();
  if constexpr (MM16_EARLY) first_reads(lds);
  // While tile kt is multiplied out of one stage, tile kt+1 streams into the
  // other, which every wave finished reading before the previous barrier.
  // The tile after the last one is the last one again (loaded, never used),
  // which keeps the loop free of special cases.
  constexpr std::true_type with_fetch{};
  unsigned char *const stage0 = lds, *const stage1 = lds + MM16_STAGE_BYTES;
  for (int kt = 0; kt + 1 < KT; kt += 2) {
    multiply(stage0, stage1, kt + 1, 1, with_fetch);
    multiply(stage1, stage0, kt + 2 < KT ? kt + 2 : KT - 1, 0, with_fetch);
  }
  if (KT & 1) multiply(stage0, stage1, KT - 1, 1, with_fetch);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // no load outlives the wave

  // C fragment: element e of lane l is row (e/4)*8 + (l/32)*4 + e%4, column l%32.
#pragma unroll
  for (int mt = 0; mt < MM16_MT; mt++)
#pragma unroll
    for (int nt = 0; nt < MM16_NT; nt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int row =
            bm + wm * (MM16_MT * 32) + mt * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        const int col = bn + wn * (MM16_NT * 32) + nt * 32 + (lane & 31);
        // C is not read again by this kernel: non-temporal stores (122.7 -> 121.0 us at 4096^3)
        __builtin_nontemporal_store(acc[mt][nt][e], &Cb[(int64_t)row * N + col]);
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
  int64_t batch;
  int tile_m, tile_n;
  mm_tile_of_block(batch, tile_m, tile_n);
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

// ---------------------------------------------------------- padded operands
// Shapes the MFMA kernels do not take (M or N not a multiple of 256, K not a
// multiple of the k-step) run on zero-padded copies of A and B in a workspace
// when that is cheaper than the scalar kernel: dst[b][r][c] = src[b][r][c]
// inside [rows][cols] and 0 outside, and the [M][N] corner of the padded
// product is copied out.  Padding K with zeros adds zeros to every sum; padded
// rows of A and columns of B only produce elements that are not copied.
template <class T>
__global__ __launch_bounds__(256) void mm_pad_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                     int64_t rows, int64_t cols, int64_t rows_p,
                                                     int64_t cols_p) {
  const int64_t b = blockIdx.z;
  // grid.y is capped (65535 at most), so a block walks rows with that stride.
  for (int64_t r = blockIdx.y; r < rows_p; r += gridDim.y) {
    const T *s = src + (b * rows + r) * cols;
    T *d = dst + (b * rows_p + r) * cols_p;
    const bool row_in = r < rows;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols_p; c += (int64_t)gridDim.x * 256)
      __builtin_nontemporal_store((row_in && c < cols) ? s[c] : T(0), &d[c]);
  }
}

__global__ __launch_bounds__(256) void mm_unpad_kernel(const float *__restrict__ src,
                                                       float *__restrict__ dst, int64_t rows,
                                                       int64_t cols, int64_t rows_p, int64_t cols_p) {
  const int64_t b = blockIdx.z;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const float *s = src + (b * rows_p + r) * cols_p;
    float *d = dst + (b * rows + r) * cols;
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += (int64_t)gridDim.x * 256)
      __builtin_nontemporal_store(s[c], &d[c]);
  }
}

struct MmPlan {
  bool direct_tiled;  // the MFMA kernels take the shape as it is
  bool padded;        // run them on padded copies
  int64_t Mp, Np, Kp;
  size_t a_bytes, b_bytes, c_bytes;  // 256-byte multiples
};

static size_t mm_align(size_t x) { return (x + 255) & ~(size_t)255; }

static bool mm16_small_tiles_fit(int64_t M, int64_t N, int64_t K);
static MmPlan mm_plan(fa_dtype in_t, int64_t batch, int64_t M, int64_t N, int64_t K) {
  MmPlan p = {};
  const int bk = in_t == FA_F32 ? MM32_BK : MM16_BK;
  const size_t es = in_t == FA_F32 ? 4 : 2;
  p.direct_tiled = (M % MM_BM == 0 && N % MM_BN == 0 && K % bk == 0 && K > 0) ||
                   (in_t != FA_F32 && mm16_small_tiles_fit(M, N, K));
  if (p.direct_tiled || batch * M * N == 0 || K == 0) return p;
  p.Mp = ceil_div(M, (int64_t)MM_BM) * MM_BM;
  p.Np = ceil_div(N, (int64_t)MM_BN) * MM_BN;
  p.Kp = ceil_div(K, (int64_t)bk) * bk;
  // Worth it when there is enough work to pay for four more launches and the
  // padding does not multiply the work too much: the scalar kernel runs at a
  // few percent of the MFMA rate.
  const double work = (double)batch * M * N * K, padded_work = (double)batch * p.Mp * p.Np * p.Kp;
  fa_tuning tune;
  fa_get_tuning(&tune);
  p.padded = work >= (double)tune.matmul_pad_min_work && padded_work <= 8.0 * work && batch <= 65535;
  p.a_bytes = mm_align((size_t)batch * p.Mp * p.Kp * es);
  p.b_bytes = mm_align((size_t)batch * p.Kp * p.Np * es);
  p.c_bytes = mm_align((size_t)batch * p.Mp * p.Np * 4);
  return p;
}

// Launch of one geometry of the 16-bit kernel.
template <bool BF16, int BM, int BN, int WAVES_M, int WAVES_N>
static int launch_mm16(hipStream_t st, const uint16_t *A, const uint16_t *B, float *C, int64_t batch,
                       int64_t M, int64_t N, int64_t K) {
  constexpr int lds = 2 * (BM * MM16_A_ROW_BYTES + MM16_BK * BN * 2);
  auto kernel = matmul16_kernel<BF16, BM, BN, WAVES_M, WAVES_N>;
  static const int raised = raise_lds(kernel, lds);
  if (raised) return raised;
  // The grid's second dimension holds 65535 tile rows: a single matrix with more
  // goes out in bands of rows (A and C advance, B stays); with a batch the
  // matrices of a band would no longer be M rows apart, so that case is refused.
  constexpr int64_t BAND = (int64_t)65535 * BM;
  if (M > BAND && batch > 1) return FA_EINVAL;
  for (int64_t r0 = 0; r0 < M; r0 += BAND) {
    const int64_t rows = M - r0 < BAND ? M - r0 : BAND;
    const dim3 grid((unsigned)(N / BN), (unsigned)(rows / BM), (unsigned)batch);
    hipLaunchKernelGGL(kernel, grid, dim3(64 * WAVES_M * WAVES_N), lds, st, A + r0 * K, B, C + r0 * N,
                       (int)rows, (int)N, (int)K);
    const int rc = launch_status();
    if (rc != 0) return rc;
  }
  return 0;
}

// 128 x 128 tiles serve shapes that are multiples of 128 but not of 256 without
// padded copies.  They are not faster where both fit, not even for products
// with few k-steps per tile: b = 64, M = N = K = 512 f16 takes 30.5 us with
// them against 28.5 us with 256 x 256 tiles on the same box, and 4096^3 141
// against 118 us (two blocks share a CU and one's C store runs under the
// other's k-loop, but every block moves twice the bytes from L2 into LDS per
// flop, and reads LDS a third more often per MFMA).
static bool mm16_small_tiles_fit(int64_t M, int64_t N, int64_t K) {
  return M % 128 == 0 && N % 128 == 0 && K % MM16_BK == 0 && K > 0;
}

static int matmul_direct(fa_stream_t stream, fa_dtype in_t, const void *A, const void *B, float *C,
                         int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch < 0 || M < 0 || N < 0 || K < 0) return FA_EINVAL;
  if (in_t != FA_F32 && in_t != FA_F16 && in_t != FA_BF16) return FA_ENOTSUP;
  if (batch * M * N == 0) return 0;
  if (C == nullptr || (K > 0 && (A == nullptr || B == nullptr))) return FA_EINVAL;
  if (batch > 65535 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return FA_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const int bk = in_t == FA_F32 ? MM32_BK : MM16_BK;
  const bool aligned = is_aligned(A, 16) && is_aligned(B, 16) && is_aligned(C, 16);
  const bool tiled = M % MM_BM == 0 && N % MM_BN == 0 && K % bk == 0 && K > 0 && aligned;
  if (in_t != FA_F32 && aligned && !tiled && mm16_small_tiles_fit(M, N, K)) {
    const uint16_t *a = (const uint16_t *)A, *b = (const uint16_t *)B;
    return in_t == FA_F16 ? launch_mm16<false, 128, 128, 1, 2>(st, a, b, C, batch, M, N, K)
                          : launch_mm16<true, 128, 128, 1, 2>(st, a, b, C, batch, M, N, K);
  }
  if (tiled) {
    if (in_t == FA_F32) {
      const dim3 grid((unsigned)(N / MM_BN), (unsigned)(M / MM_BM), (unsigned)batch);
      static const int raised = raise_lds(matmul32_kernel, 2 * MM32_STAGE_BYTES);
      if (raised) return raised;
      hipLaunchKernelGGL(matmul32_kernel, grid, dim3(MM_THREADS), 2 * MM32_STAGE_BYTES, st,
                         (const float *)A, (const float *)B, C, (int)M, (int)N, (int)K);
      return launch_status();
    }
    const uint16_t *a = (const uint16_t *)A, *b = (const uint16_t *)B;
    return in_t == FA_F16 ? launch_mm16<false, 256, 256, 2, 2>(st, a, b, C, batch, M, N, K)
                          : launch_mm16<true, 256, 256, 2, 2>(st, a, b, C, batch, M, N, K);
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

extern "C" size_t fa_matmul_workspace_bytes(fa_dtype in_t, int64_t batch, int64_t M, int64_t N,
                                            int64_t K) {
  if (batch < 0 || M < 0 || N < 0 || K < 0) return 0;
  if (in_t != FA_F32 && in_t != FA_F16 && in_t != FA_BF16) return 0;
  const MmPlan p = mm_plan(in_t, batch, M, N, K);
  return p.padded ? p.a_bytes + p.b_bytes + p.c_bytes : 0;
}

template <class T>
static int mm_pad(hipStream_t st, const void *src, void *dst, int64_t batch, int64_t rows,
                  int64_t cols, int64_t rows_p, int64_t cols_p) {
  const dim3 grid((unsigned)std::min<int64_t>(ceil_div(cols_p, (int64_t)256), 64),
                  (unsigned)std::min<int64_t>(rows_p, 65535), (unsigned)batch);
  hipLaunchKernelGGL((mm_pad_kernel<T>), grid, dim3(256), 0, st, (const T *)src, (T *)dst, rows, cols,
                     rows_p, cols_p);
  return launch_status();
}

extern "C" int fa_matmul_ws(fa_stream_t stream, fa_dtype in_t, const void *A, const void *B,
                            float *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                            void *workspace, size_t workspace_bytes) {
  if (batch < 0 || M < 0 || N < 0 || K < 0) return FA_EINVAL;
  if (in_t != FA_F32 && in_t != FA_F16 && in_t != FA_BF16) return FA_ENOTSUP;
  const MmPlan p = mm_plan(in_t, batch, M, N, K);
  if (!p.padded || workspace == nullptr || workspace_bytes < p.a_bytes + p.b_bytes + p.c_bytes ||
      !is_aligned(workspace, 256))
    return matmul_direct(stream, in_t, A, B, C, batch, M, N, K);
  if (C == nullptr || A == nullptr || B == nullptr) return FA_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  char *Ap = (char *)workspace, *Bp = Ap + p.a_bytes, *Cp = Bp + p.b_bytes;
  int rc;
  if (in_t == FA_F32) {
    rc = mm_pad<float>(st, A, Ap, batch, M, K, p.Mp, p.Kp);
    if (rc == 0) rc = mm_pad<float>(st, B, Bp, batch, K, N, p.Kp, p.Np);
  } else {
    rc = mm_pad<uint16_t>(st, A, Ap, batch, M, K, p.Mp, p.Kp);
    if (rc == 0) rc = mm_pad<uint16_t>(st, B, Bp, batch, K, N, p.Kp, p.Np);
  }
  if (rc != 0) return rc;
  rc = matmul_direct(stream, in_t, Ap, Bp, (float *)Cp, batch, p.Mp, p.Np, p.Kp);
  if (rc != 0) return rc;
  const dim3 grid((unsigned)std::min<int64_t>(ceil_div(N, (int64_t)256), 64),
                  (unsigned)std::min<int64_t>(M, 65535), (unsigned)batch);
  hipLaunchKernelGGL(mm_unpad_kernel, grid, dim3(256), 0, st, (const float *)Cp, C, M, N, p.Mp, p.Np);
  return launch_status();
}

// ------------------------------------------------------------ MFMA rate probe
// What the matrix cores sustain on registers alone: every wave loads one A and
// one B fragment (16 bytes each) from `operands` and then issues `iters` rounds
// of 16 independent 32x32x16 MFMAs into 256 accumulator registers, the inner
// tile of matmul16_kernel without its loads and LDS reads.  The figure depends
// on the operand values (power management lowers the clock when the multiplier
// inputs toggle), so the caller supplies operands distributed like its
// matrices.  One 256-thread block per CU and launch.
namespace fa {
template <bool BF16>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const uint16_t *__restrict__ operands,
                                                         int iters, float *sink) {
  using Frag = __attribute__((ext_vector_type(4))) uint32_t;
  const Frag a = reinterpret_cast<const Frag *>(operands)[threadIdx.x];
  const Frag b = reinterpret_cast<const Frag *>(operands)[256 + threadIdx.x];
  f32x16 acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      if constexpr (BF16)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bit_cast<bf16x8>(a), bit_cast<bf16x8>(b), acc[i], 0, 0, 0);
      else
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bit_cast<f16x8>(a), bit_cast<f16x8>(b), acc[i], 0, 0, 0);
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int e = 0; e < 16; e++) s += acc[i][e];
  if (s == 12345.678f) sink[0] = s;  // keeps the loop alive
}
}  // namespace fa

extern "C" int fa_mfma_probe(fa_stream_t stream, fa_dtype in_t, const void *operands, int blocks,
                             int iters, float *sink, double *flop) {
  if (in_t != FA_F16 && in_t != FA_BF16) return FA_ENOTSUP;
  if (operands == nullptr || sink == nullptr || blocks < 1 || iters < 1) return FA_EINVAL;
  if (!is_aligned(operands, 16)) return FA_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  if (in_t == FA_F16)
    hipLaunchKernelGGL((mfma_probe_kernel<false>), dim3(blocks), dim3(256), 0, st,
                       (const uint16_t *)operands, iters, sink);
  else
    hipLaunchKernelGGL((mfma_probe_kernel<true>), dim3(blocks), dim3(256), 0, st,
                       (const uint16_t *)operands, iters, sink);
  if (flop != nullptr) *flop = (double)blocks * 4.0 * iters * 16.0 * (2.0 * 32 * 32 * 16);
  return launch_status();
}

extern "C" int fa_matmul(fa_stream_t stream, fa_dtype in_t, const void *A, const void *B, float *C,
                         int64_t batch, int64_t M, int64_t N, int64_t K) {
  return matmul_direct(stream, in_t, A, B, C, batch, M, N, K);
}
