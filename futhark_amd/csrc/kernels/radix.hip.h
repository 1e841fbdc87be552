// Kernels of the 8-bit radix pass shared by the sort (radix.hip) and by the
// bin-range partition of large histograms (seghist.hip).
//
// A pass is three launches: per-tile digit counts (a read-only stream, the
// cheapest thing this GPU does), an exclusive scan of the digit-major counts
// with the single-pass scan kernel, and a ranked scatter.  A one-kernel pass
// with per-digit decoupled look-back was measured slower here: with one large
// tile per CU in flight the look-back chain is hundreds of tiles deep and each
// hop is a device-scope load of more than a microsecond.
#pragma once

#include "dispatch.hip.h"

namespace fa {

constexpr int RS_BLOCK = 512;
constexpr int RS_WAVES = RS_BLOCK / WAVE;
constexpr int RS_KPT = 16;  // keys per thread
constexpr int RS_TILE = RS_BLOCK * RS_KPT;
constexpr int RS_RADIX = 256;
// Positions in the output (counts, offsets, the scatter's destinations) are of
// type Off: unsigned 32-bit numbers for fewer than RS_WIDE_N keys, 64-bit ones
// from there on.  Everything that scales with the tile count is 64-bit.
constexpr int64_t RS_WIDE_N = ((int64_t)1 << 32) - 1;
constexpr int RS_DIES = 8;  // a block runs on die blockIdx.x % 8

struct RsScratch {
  void *counts;    // [256][tiles] of Off
  void *offsets;   // [256][tiles] exclusive scan of counts, digit-major
  void *lookback;  // scratch of the scan kernel, cleared once per call
  size_t lookback_bytes;
  int64_t tiles;
  bool wide;  // Off is 64-bit
};

static inline int64_t rs_num_tiles(int64_t n) { return ceil_div(n, (int64_t)RS_TILE); }
static inline size_t rs_align(size_t x) { return (x + 255) & ~(size_t)255; }

static inline size_t rs_scratch_bytes(int64_t tiles, bool wide) {
  if (tiles < 1) tiles = 1;
  return 2 * rs_align((size_t)tiles * RS_RADIX * (wide ? 8 : 4)) +
         rs_align(fa_segscan_scratch_bytes(wide ? FA_U64 : FA_U32, tiles * RS_RADIX));
}

static inline RsScratch rs_carve(void *scratch, int64_t tiles, bool wide) {
  RsScratch sc;
  const size_t counts = rs_align((size_t)tiles * RS_RADIX * (wide ? 8 : 4));
  sc.counts = scratch;
  sc.offsets = (char *)scratch + counts;
  sc.lookback = (char *)scratch + 2 * counts;
  sc.lookback_bytes = rs_align(fa_segscan_scratch_bytes(wide ? FA_U64 : FA_U32, tiles * RS_RADIX));
  sc.tiles = tiles;
  sc.wide = wide;
  return sc;
}

// The scan scratch must start zeroed; after that each pass uses its own epoch.
static inline int rs_prepare(hipStream_t st, const RsScratch &sc) {
  return fa_replicate((fa_stream_t)st, 4, sc.lookback, (int64_t)(sc.lookback_bytes / 4), 0);
}

// counts[d][tile] = number of keys of the tile whose digit is d.  A block
// counts RS_HIST_TILES consecutive tiles into one set of LDS counters per
// tile, so that nothing has to be summed or cleared between tiles and the only
// barrier comes after the last key.  What the block writes for a digit is a
// run of RS_HIST_TILES counts (one 32-byte store) instead of single 4-byte
// stores 4*num_tiles bytes apart.
//
// The keys are read with the non-temporal policy (58.8 -> 51.1 us per pass
// over 2^26 4-byte keys, 145 -> 102 us over 8-byte keys), and the keys of the
// next tile are in flight while the current one is counted.  For that the
// loads must not sit under a condition: where two paths meet, one with loads in
// flight and one without, the compiler waits for the memory counter to reach
// what is right for both, which is "everything has arrived".  So every step
// loads a whole tile, from the start of the keys when its own tile is not a
// whole one, and counts it, by one or by zero (with the counting under a
// condition the compiler moves the loads of the first tile there, behind the
// prefetch of the second).  The one ragged tile at the end of the input is read
// element by element.
constexpr int RS_HIST_TILES = 8;

// h[d] += one for every lane.  Sorted or small keys and skewed histogram
// indices give most lanes of a wave the same digit, and 64 atomics on one LDS
// word are taken one after the other (a pass over keys with one digit ran at
// 183 us against 50 us); so the lanes that share the first lane's digit are
// counted with a ballot and added once.
__device__ __forceinline__ void rs_count(uint32_t *h, uint32_t d, uint32_t one) {
  const uint32_t d0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)d);
  const uint64_t same = __ballot(d == d0);
  if (d != d0)
    atomicAdd(&h[d], one);
  else if (lane_id() == 0)
    atomicAdd(&h[d0], one * (uint32_t)__builtin_popcountll(same));
}

template <class K, class DigitFn, class Off>
__global__ __launch_bounds__(RS_BLOCK) void rs_hist_kernel(const K *__restrict__ keys, int64_t n,
                                                           DigitFn fn, int pass, Off *counts,
                                                           int64_t num_tiles) {
  constexpr int VEC = 16 / sizeof(K);
  constexpr int ROWS = RS_KPT / VEC;
  __shared__ __align__(16) uint32_t h[RS_HIST_TILES][RS_RADIX];
  for (int i = threadIdx.x; i < RS_HIST_TILES * RS_RADIX; i += RS_BLOCK) (&h[0][0])[i] = 0u;
  // The scatter kernel that follows takes the tiles die by die (block b: tile
  // (b % 8) * tiles_per_die + b / 8).  Counting the keys in the reverse of that
  // order leaves in the memory-side cache what the scatter reads first; the
  // non-temporal loads bypass L2 only.  Sort of 2^26 4-byte keys: 770 -> 747 us;
  // with 8-byte keys, where a pass reads twice the cache's size, the order
  // costs 1 % instead (3521 -> 3552 us), so those keep the plain order.
  // (gridDim.x is a multiple of RS_DIES.)
  int64_t group = blockIdx.x;
  if constexpr (sizeof(K) == 4) {
    const int64_t rb = (int64_t)gridDim.x - 1 - blockIdx.x;
    group = (rb % RS_DIES) * (gridDim.x / RS_DIES) + rb / RS_DIES;
  }
  const int64_t tile0 = group * RS_HIST_TILES;
  // The tiles of a block are taken in an order rotated by the block's number:
  // blocks run in step, and with every block at the same place of its own run
  // of tiles the reads of one moment would lie 8 tiles apart from each other
  // (a stride that visits few memory channels) instead of covering a stretch
  // of memory evenly.
  const int rot = blockIdx.x % RS_HIST_TILES;
  auto tile_id = [&](int i) { return tile0 + (i + rot) % RS_HIST_TILES; };
  auto exists = [&](int i) { return tile_id(i) < num_tiles; };
  auto full = [&](int i) { return (tile_id(i) + 1) * RS_TILE <= n; };
  const bool pipelined = n >= RS_TILE;  // a whole tile can be loaded from the start of the keys
  Vec16<K> cur[ROWS], nxt[ROWS];
  auto fetch = [&](int i, Vec16<K>(&v)[ROWS]) {
    const int64_t base = full(i) ? tile_id(i) * RS_TILE : 0;
#pragma unroll
    for (int r = 0; r < ROWS; r++)
      v[r] = load_vec16_nt(keys + base + ((int64_t)r * RS_BLOCK + threadIdx.x) * VEC);
  };
  auto count_ragged = [&](int i) {
    const int64_t base = tile_id(i) * RS_TILE;
    for (int j = threadIdx.x; j < RS_TILE && base + j < n; j += RS_BLOCK)
      atomicAdd(&h[i][fn(keys[base + j], pass)], 1u);
  };
  __syncthreads();
  if (pipelined) {
    fetch(0, cur);
    __builtin_amdgcn_sched_barrier(0);  // loads complete in the order of issue: keep it
#pragma unroll
    for (int i = 0; i < RS_HIST_TILES; i++) {
      if (i + 1 < RS_HIST_TILES) fetch(i + 1, nxt);
      __builtin_amdgcn_sched_barrier(0);
      const uint32_t one = full(i) ? 1u : 0u;  // uniform
#pragma unroll
      for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int e = 0; e < VEC; e++) rs_count(&h[i][0], fn(cur[r].e[e], pass), one);
#pragma unroll
      for (int r = 0; r < ROWS; r++) cur[r] = nxt[r];
    }
  }
  for (int i = 0; i < RS_HIST_TILES; i++)
    if (exists(i) && !full(i)) count_ragged(i);
  __syncthreads();
  if (threadIdx.x < RS_RADIX) {
    uint32_t mine[RS_HIST_TILES];
#pragma unroll
    for (int i = 0; i < RS_HIST_TILES; i++) mine[(i + rot) % RS_HIST_TILES] = h[i][threadIdx.x];
    Off *dst = counts + (int64_t)threadIdx.x * num_tiles + tile0;
    const int tiles_here =
        (int)(num_tiles - tile0 < RS_HIST_TILES ? num_tiles - tile0 : RS_HIST_TILES);
    if (sizeof(Off) == 4 && tiles_here == RS_HIST_TILES && (num_tiles & 3) == 0) {
      static_assert(RS_HIST_TILES == 8, "two 16-byte stores per digit");
      reinterpret_cast<uint4 *>(dst)[0] = make_uint4(mine[0], mine[1], mine[2], mine[3]);
      reinterpret_cast<uint4 *>(dst)[1] = make_uint4(mine[4], mine[5], mine[6], mine[7]);
    } else {
#pragma unroll
      for (int t = 0; t < RS_HIST_TILES; t++)
        if (t < tiles_here) dst[t] = mine[t];
    }
  }
}

template <int BYTES> struct ValType;
template <> struct ValType<0> { using T = uint32_t; };
template <> struct ValType<1> { using T = uint8_t; };
template <> struct ValType<2> { using T = uint16_t; };
template <> struct ValType<4> { using T = uint32_t; };
template <> struct ValType<8> { using T = uint64_t; };

// For two digits per lane (two rounds of a wave), the lanes of the wave whose
// digit equals this lane's, as 64-bit masks in halves.  Per digit bit and
// round: the lane's bit spread over a word (v_bfe_i32 gives 0 or ~0), the
// ballot of that bit (v_cmp into a scalar pair), and per half one three-input
// boolean, same &= ~(ballot ^ mine) (truth table 0xf0 & ~(0xcc ^ 0xaa) = 0x90).
// The compiler turns the same source into five to six instructions per bit.
// Here the two rounds are interleaved and bits are taken two at a time: the
// extracts and ballots of the next pair of bits are issued before the
// booleans of the current pair, so that at least eight instructions lie
// between a ballot and the first instruction that reads its scalar pair (with
// two the scatter kernel was no faster than with the compiler's code; the
// scatter of 2^26 4-byte keys takes 139 us with this and 153 us with the
// compiler's).  Must be called with all 64 lanes active.
__device__ __forceinline__ void rs_match2(uint32_t da, uint32_t db, uint32_t &a_lo, uint32_t &a_hi,
                                          uint32_t &b_lo, uint32_t &b_hi) {
  uint32_t t0, t1, t2, t3, t4, t5, t6, t7;
  asm(
      "v_bfe_i32 %4, %12, 0, 1\n"
      "v_bfe_i32 %5, %12, 1, 1\n"
      "v_bfe_i32 %6, %13, 0, 1\n"
      "v_bfe_i32 %7, %13, 1, 1\n"
      "v_cmp_ne_u32_e64 s[84:85], 0, %4\n"
      "v_cmp_ne_u32_e64 s[86:87], 0, %5\n"
      "v_cmp_ne_u32_e64 s[88:89], 0, %6\n"
      "v_cmp_ne_u32_e64 s[90:91], 0, %7\n"
      "v_bfe_i32 %8, %12, 2, 1\n"
      "v_bfe_i32 %9, %12, 3, 1\n"
      "v_bfe_i32 %10, %13, 2, 1\n"
      "v_bfe_i32 %11, %13, 3, 1\n"
      "v_cmp_ne_u32_e64 s[92:93], 0, %8\n"
      "v_cmp_ne_u32_e64 s[94:95], 0, %9\n"
      "v_cmp_ne_u32_e64 s[96:97], 0, %10\n"
      "v_cmp_ne_u32_e64 s[98:99], 0, %11\n"
      "v_xnor_b32 %0, s84, %4\n"
      "v_xnor_b32 %1, s85, %4\n"
      "v_bitop3_b32 %0, %0, s86, %5 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s87, %5 bitop3:0x90\n"
      "v_xnor_b32 %2, s88, %6\n"
      "v_xnor_b32 %3, s89, %6\n"
      "v_bitop3_b32 %2, %2, s90, %7 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s91, %7 bitop3:0x90\n"
      "v_bfe_i32 %4, %12, 4, 1\n"
      "v_bfe_i32 %5, %12, 5, 1\n"
      "v_bfe_i32 %6, %13, 4, 1\n"
      "v_bfe_i32 %7, %13, 5, 1\n"
      "v_cmp_ne_u32_e64 s[84:85], 0, %4\n"
      "v_cmp_ne_u32_e64 s[86:87], 0, %5\n"
      "v_cmp_ne_u32_e64 s[88:89], 0, %6\n"
      "v_cmp_ne_u32_e64 s[90:91], 0, %7\n"
      "v_bitop3_b32 %0, %0, s92, %8 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s93, %8 bitop3:0x90\n"
      "v_bitop3_b32 %0, %0, s94, %9 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s95, %9 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s96, %10 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s97, %10 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s98, %11 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s99, %11 bitop3:0x90\n"
      "v_bfe_i32 %8, %12, 6, 1\n"
      "v_bfe_i32 %9, %12, 7, 1\n"
      "v_bfe_i32 %10, %13, 6, 1\n"
      "v_bfe_i32 %11, %13, 7, 1\n"
      "v_cmp_ne_u32_e64 s[92:93], 0, %8\n"
      "v_cmp_ne_u32_e64 s[94:95], 0, %9\n"
      "v_cmp_ne_u32_e64 s[96:97], 0, %10\n"
      "v_cmp_ne_u32_e64 s[98:99], 0, %11\n"
      "v_bitop3_b32 %0, %0, s84, %4 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s85, %4 bitop3:0x90\n"
      "v_bitop3_b32 %0, %0, s86, %5 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s87, %5 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s88, %6 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s89, %6 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s90, %7 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s91, %7 bitop3:0x90\n"
      "v_bitop3_b32 %0, %0, s92, %8 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s93, %8 bitop3:0x90\n"
      "v_bitop3_b32 %0, %0, s94, %9 bitop3:0x90\n"
      "v_bitop3_b32 %1, %1, s95, %9 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s96, %10 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s97, %10 bitop3:0x90\n"
      "v_bitop3_b32 %2, %2, s98, %11 bitop3:0x90\n"
      "v_bitop3_b32 %3, %3, s99, %11 bitop3:0x90\n"
      : "=&v"(a_lo), "=&v"(a_hi), "=&v"(b_lo), "=&v"(b_hi), "=&v"(t0), "=&v"(t1), "=&v"(t2),
        "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
      : "v"(da), "v"(db)
      : "s84", "s85", "s86", "s87", "s88", "s89", "s90", "s91", "s92", "s93", "s94", "s95", "s96", "s97", "s98", "s99");
}

constexpr size_t RS_LDS_FIXED = RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4 + 64;

// Ranked scatter.  Inside a wave, lanes with equal digits find each other with
// eight ballots; per-wave digit counters in LDS chain the 16 rounds; the tile
// is then reordered in LDS so that the global stores of a wave are contiguous
// runs per digit.  Order is preserved at every level (round, lane, wave, tile).
// The stores stay ordinary ones: the runs are shorter than a cache line, and
// non-temporal stores, which help every streaming kernel here, cost 35 % (L2
// no longer merges the pieces of a line).
//
// Tiles are dealt to blocks so that each of the eight dies of the GPU (a block
// goes to die blockIdx.x % 8) works on one contiguous eighth of the tiles: the
// run of a digit in tile t ends in the cache line where the run of the same
// digit in tile t + 1 begins, and the two halves of that line meet in one L2
// only if both tiles are scattered on the same die.
template <class K, int VB, bool FULL, class DigitFn, class Off>
__device__ __forceinline__ void rs_scatter_tile(const K *__restrict__ kin,
                                                typename DigitFn::Out *__restrict__ kout,
                                                const typename ValType<VB>::T *__restrict__ vin,
                                                typename ValType<VB>::T *__restrict__ vout,
                                                int64_t n, DigitFn fn, int pass,
                                                const Off *__restrict__ offs,
                                                int64_t num_tiles, int64_t tile,
                                                unsigned char *s_raw) {
  using V = typename ValType<VB>::T;
  uint32_t(*cnt)[RS_RADIX] = reinterpret_cast<uint32_t(*)[RS_RADIX]>(s_raw);
  static_assert(sizeof(Off) <= 8, "the table of a tile is 2 * RS_RADIX words");
  Off *s_tab = reinterpret_cast<Off *>(s_raw + RS_WAVES * RS_RADIX * 4);
  uint32_t *s_wsum =
      reinterpret_cast<uint32_t *>(s_raw + RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4);  // 4 used
  unsigned char *buf = s_raw + RS_LDS_FIXED;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int lane = lane_id();
  const int64_t base = tile * RS_TILE;
  const int tile_n = FULL ? RS_TILE : (int)(n - base);

  // Wave-striped arrangement: wave w owns keys [w*64*KPT, (w+1)*64*KPT) of the
  // tile, round r is 64 consecutive keys.
  K key[RS_KPT];
  int pos[RS_KPT];
  const int wbase = wave * WAVE * RS_KPT;
  auto present = [&](int r) { return FULL || wbase + r * WAVE + lane < tile_n; };
  {
    const K *src = kin + base + wbase + lane;
#pragma unroll
    for (int r = 0; r < RS_KPT; r++) key[r] = present(r) ? __builtin_nontemporal_load(src + r * WAVE) : (K)0;
  }
  // Values are asked for now and used after the keys have gone out.
  V val[VB != 0 ? RS_KPT : 1];
  if constexpr (VB != 0) {
    const V *src = vin + base + wbase + lane;
#pragma unroll
    for (int r = 0; r < RS_KPT; r++) val[r] = present(r) ? __builtin_nontemporal_load(src + r * WAVE) : (V)0;
  }
  for (int i = tid; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&cnt[0][0])[i] = 0u;
  // Global offsets of this tile, one digit per thread (strided, L2-resident).
  Off goff = 0;
  if (tid < RS_RADIX) goff = offs[(int64_t)tid * num_tiles + tile];
  __syncthreads();
  // The kernel is bound by vector-ALU issue; rs_match2 finds the lanes with
  // equal digits for two rounds at a time in four instructions per digit bit.
#pragma unroll
  for (int r2 = 0; r2 < RS_KPT; r2 += 2) {
    uint32_t d[2], peers_lo[2], peers_hi[2];
    d[0] = fn(key[r2], pass);
    d[1] = fn(key[r2 + 1], pass);
    rs_match2(d[0], d[1], peers_lo[0], peers_hi[0], peers_lo[1], peers_hi[1]);
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int r = r2 + h;
      const bool valid = present(r);
      if constexpr (!FULL) {
        const uint64_t vm = __ballot(valid);
        peers_lo[h] &= (uint32_t)vm;
        peers_hi[h] &= (uint32_t)(vm >> 32);
      }
      const int rank = (int)__builtin_amdgcn_mbcnt_hi(
          peers_hi[h], __builtin_amdgcn_mbcnt_lo(peers_lo[h], 0u));
      int p = 0;
      if (valid) {
        const uint32_t prev = cnt[wave][d[h]];
        p = (int)prev + rank;
        if (rank == 0)
          cnt[wave][d[h]] = prev + (uint32_t)(__builtin_popcount(peers_lo[h]) +
                                              __builtin_popcount(peers_hi[h]));
      }
      pos[r] = p;
    }
  }
  __syncthreads();

  // Per digit: exclusive prefix over waves, then exclusive prefix over digits.
  uint32_t total = 0, incl = 0;
  uint32_t wrun[RS_WAVES];
  if (tid < RS_RADIX) {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < RS_WAVES; w++) {
      wrun[w] = run;
      run += cnt[w][tid];
    }
    total = run;
    incl = wave_incl_scan<uint32_t, OpAdd<uint32_t>>(total);
    if (lane == 63) s_wsum[wave] = incl;
  }
  __syncthreads();
  if (tid < RS_RADIX) {
    uint32_t wpre = 0;
    for (int w = 0; w < wave; w++) wpre += s_wsum[w];
    const uint32_t dbase = wpre + incl - total;
    // cnt[w][d] becomes the place in the reordered tile of wave w's first key
    // with digit d
#pragma unroll
    for (int w = 0; w < RS_WAVES; w++) cnt[w][tid] = dbase + wrun[w];
    // destination of element i of the reordered tile with digit d: tab[d] + i
    s_tab[tid] = goff - dbase;
  }
  __syncthreads();

  // Reorder keys inside LDS.
  K *kbuf = reinterpret_cast<K *>(buf);
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) pos[r] += (int)cnt[wave][fn(key[r], pass)];
#pragma unroll
  for (int r = 0; r < RS_KPT; r++)
    if (present(r)) kbuf[pos[r]] = key[r];
  __syncthreads();
  // The offsets come from this library's own histogram and scan; should they
  // ever be wrong, a store outside the output would fault the GPU, whereas a
  // dropped key is a wrong result the caller can see.
  Off dst[RS_KPT];
  const Off limit = (Off)n;
#pragma unroll
  for (int j = 0; j < RS_KPT; j++) {
    const int i = j * RS_BLOCK + tid;
    dst[j] = limit;
    if (FULL || i < tile_n) {
      const K k = kbuf[i];
      dst[j] = s_tab[fn(k, pass)] + (Off)i;
      if (dst[j] < limit) kout[dst[j]] = fn.out(k);
    }
  }
  if constexpr (VB != 0) {
    __syncthreads();
    V *vbuf = reinterpret_cast<V *>(buf);
#pragma unroll
    for (int r = 0; r < RS_KPT; r++)
      if (present(r)) vbuf[pos[r]] = val[r];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < RS_KPT; j++) {
      const int i = j * RS_BLOCK + tid;
      if ((FULL || i < tile_n) && dst[j] < limit) vout[dst[j]] = vbuf[i];
    }
  }
}

template <class K, int VB, class DigitFn, class Off>
__global__ __launch_bounds__(RS_BLOCK) void rs_scatter_kernel(
    const K *__restrict__ kin, typename DigitFn::Out *__restrict__ kout,
    const void *__restrict__ vin_, void *__restrict__ vout_, int64_t n, DigitFn fn, int pass,
    const Off *__restrict__ offs,
    int64_t num_tiles) {
  using V = typename ValType<VB>::T;
  extern __shared__ __align__(16) unsigned char s_raw[];
  // gridDim.x = RS_DIES * tiles_per_die
  const int64_t tiles_per_die = gridDim.x / RS_DIES;
  const int64_t tile = (int64_t)(blockIdx.x % RS_DIES) * tiles_per_die + blockIdx.x / RS_DIES;
  if (tile >= num_tiles) return;  // uniform over the block
  if ((tile + 1) * RS_TILE <= n)
    rs_scatter_tile<K, VB, true, DigitFn, Off>(kin, kout, (const V *)vin_, (V *)vout_, n, fn, pass, offs,
                                 num_tiles, tile, s_raw);
  else
    rs_scatter_tile<K, VB, false, DigitFn, Off>(kin, kout, (const V *)vin_, (V *)vout_, n, fn, pass, offs,
                                  num_tiles, tile, s_raw);
}

// One pass: keys (and values) move from *in to *out ordered by digit `pass`,
// equal digits keeping their order.  What is written for a key is fn.out(key),
// of type DigitFn::Out: the key itself for the sort, what is left of a bin
// number inside its range for the partition of a histogram.  `epoch` must grow from call to call on
// the same scratch (1, 2, ...).  Afterwards sc.offsets[d * tiles] is the
// position where digit d starts in the output.
template <class K, int VB, class DigitFn, class Off = uint32_t>
static int rs_pass(hipStream_t st, const K *kin, typename DigitFn::Out *kout, const void *vin,
                   void *vout, int64_t n,
                   DigitFn fn, int pass, uint32_t epoch, const RsScratch &sc) {
  using V = typename ValType<VB>::T;
  constexpr bool WIDE = sizeof(Off) == 8;
  if (sc.wide != WIDE || (!WIDE && n >= RS_WIDE_N)) return FA_EINVAL;
  const size_t lds =
      RS_LDS_FIXED + (size_t)RS_TILE * (sizeof(K) > sizeof(V) ? sizeof(K) : sizeof(V));
  auto scatter = rs_scatter_kernel<K, VB, DigitFn, Off>;
  // Initialised once, under the lock C++ gives function-local statics.
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)scatter, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL((rs_hist_kernel<K, DigitFn, Off>),
                     dim3((unsigned)(ceil_div(sc.tiles, (int64_t)RS_HIST_TILES * RS_DIES) * RS_DIES)),
                     dim3(RS_BLOCK), 0, st,
                     kin, n, fn, pass, (Off *)sc.counts, sc.tiles);
  int rc = launch_status();
  if (rc != 0) return rc;
  rc = fa_segscan((fa_stream_t)st, WIDE ? FA_U64 : FA_U32, FA_ADD, sc.counts, nullptr, sc.tiles * RS_RADIX, 1,
                  sc.offsets, sc.lookback, sc.lookback_bytes, epoch);
  if (rc != 0) return rc;
  const int64_t tiles_per_die = ceil_div(sc.tiles, (int64_t)RS_DIES);
  hipLaunchKernelGGL(scatter, dim3((unsigned)(tiles_per_die * RS_DIES)), dim3(RS_BLOCK), lds, st,
                     kin, kout, vin, vout, n, fn, pass, (const Off *)sc.offsets, sc.tiles);
  return launch_status();
}

}  // namespace fa
