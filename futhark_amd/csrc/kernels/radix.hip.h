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

struct RsScratch {
  uint32_t *counts;   // [256][tiles]
  uint32_t *offsets;  // [256][tiles] exclusive scan of counts, digit-major
  void *lookback;     // scratch of the scan kernel, cleared once per call
  size_t lookback_bytes;
  int64_t tiles;
};

static inline int64_t rs_num_tiles(int64_t n) { return ceil_div(n, (int64_t)RS_TILE); }
static inline size_t rs_align(size_t x) { return (x + 255) & ~(size_t)255; }

static inline size_t rs_scratch_bytes(int64_t tiles) {
  if (tiles < 1) tiles = 1;
  return 2 * rs_align((size_t)tiles * RS_RADIX * 4) +
         rs_align(fa_segscan_scratch_bytes(FA_U32, tiles * RS_RADIX));
}

static inline RsScratch rs_carve(void *scratch, int64_t tiles) {
  RsScratch sc;
  const size_t counts = rs_align((size_t)tiles * RS_RADIX * 4);
  sc.counts = (uint32_t *)scratch;
  sc.offsets = (uint32_t *)((char *)scratch + counts);
  sc.lookback = (char *)scratch + 2 * counts;
  sc.lookback_bytes = rs_align(fa_segscan_scratch_bytes(FA_U32, tiles * RS_RADIX));
  sc.tiles = tiles;
  return sc;
}

// The scan scratch must start zeroed; after that each pass uses its own epoch.
static inline int rs_prepare(hipStream_t st, const RsScratch &sc) {
  return fa_replicate((fa_stream_t)st, 4, sc.lookback, (int64_t)(sc.lookback_bytes / 4), 0);
}

// counts[d][tile] = number of keys of the tile whose digit is d.  The kernel
// runs at the rate of LDS atomics (about one per nanosecond chip-wide, 72 us
// per 2^26 keys); spreading each counter over 32 bank-private columns made no
// difference, so the limit is the atomic unit and not bank conflicts.  A block
// counts RS_HIST_TILES consecutive tiles, so that what it writes for a digit
// is a run of RS_HIST_TILES counts (one 32-byte store) instead of single
// 4-byte stores 4*num_tiles bytes apart, and the keys of the next tile are in
// flight while the current one is counted.
constexpr int RS_HIST_TILES = 8;

template <class K, class DigitFn>
__global__ __launch_bounds__(RS_BLOCK) void rs_hist_kernel(const K *__restrict__ keys, int64_t n,
                                                           DigitFn fn, int pass, uint32_t *counts,
                                                           int64_t num_tiles) {
  constexpr int VEC = 16 / sizeof(K);
  constexpr int ROWS = RS_KPT / VEC;
  __shared__ __align__(16) uint32_t h[RS_WAVES][RS_RADIX];
  for (int i = threadIdx.x; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&h[0][0])[i] = 0u;
  const int wave = threadIdx.x / WAVE;
  const int64_t tile0 = (int64_t)blockIdx.x * RS_HIST_TILES;
  const int tiles_here =
      (int)(num_tiles - tile0 < RS_HIST_TILES ? num_tiles - tile0 : RS_HIST_TILES);
  uint32_t c[RS_HIST_TILES];  // thread d < 256: count of digit d per tile
#pragma unroll
  for (int t = 0; t < RS_HIST_TILES; t++) c[t] = 0u;

  // Full tiles are fetched one tile ahead; the last tile of the input may be
  // ragged and is read element-wise.
  Vec16<K> cur[ROWS], nxt[ROWS];
  auto full = [&](int t) { return t < tiles_here && (tile0 + t + 1) * RS_TILE <= n; };
  auto fetch = [&](int t, Vec16<K>(&v)[ROWS]) {
    const int64_t base = (tile0 + t) * RS_TILE;
#pragma unroll
    for (int r = 0; r < ROWS; r++)
      v[r] = load_vec16(keys + base + ((int64_t)r * RS_BLOCK + threadIdx.x) * VEC);
  };
  // The tiles of a block are taken in an order rotated by the block's number:
  // blocks run in step, and with every block at the same place of its own run
  // of tiles the reads of one moment would lie 8 tiles apart from each other
  // (a stride that visits few memory channels) instead of covering a stretch
  // of memory evenly.
  const int rot = blockIdx.x % RS_HIST_TILES;
  auto tile_at = [&](int i) { return (i + rot) % RS_HIST_TILES; };
  if (full(tile_at(0))) fetch(tile_at(0), cur);
  __syncthreads();
#pragma unroll
  for (int i = 0; i < RS_HIST_TILES; i++) {
    const int t = tile_at(i);
    if (i + 1 < RS_HIST_TILES && full(tile_at(i + 1))) fetch(tile_at(i + 1), nxt);
    if (t < tiles_here) {  // uniform
      if (full(t)) {
#pragma unroll
        for (int r = 0; r < ROWS; r++)
#pragma unroll
          for (int e = 0; e < VEC; e++) atomicAdd(&h[wave][fn(cur[r].e[e], pass)], 1u);
      } else {
        const int64_t base = (tile0 + t) * RS_TILE;
        for (int r = 0; r < ROWS; r++)
          for (int e = 0; e < VEC; e++) {
            const int64_t idx = base + ((int64_t)r * RS_BLOCK + threadIdx.x) * VEC + e;
            if (idx < n) atomicAdd(&h[wave][fn(keys[idx], pass)], 1u);
          }
      }
      __syncthreads();
      if (threadIdx.x < RS_RADIX) {  // sum the waves' counters and clear them
        uint32_t sum = 0;
#pragma unroll
        for (int w = 0; w < RS_WAVES; w++) {
          sum += h[w][threadIdx.x];
          h[w][threadIdx.x] = 0u;
        }
        c[i] = sum;
      }
      __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++) cur[r] = nxt[r];
  }
  if (threadIdx.x < RS_RADIX) {
    // c[i] belongs to tile tile_at(i): put the counts in tile order through
    // this thread's own eight words of LDS (the counters are no longer in use)
    static_assert(RS_WAVES * RS_RADIX >= RS_RADIX * RS_HIST_TILES, "room for the counts");
    uint32_t *mine = &h[0][0] + threadIdx.x * RS_HIST_TILES;
#pragma unroll
    for (int i = 0; i < RS_HIST_TILES; i++) mine[tile_at(i)] = c[i];
    uint32_t *dst = counts + (int64_t)threadIdx.x * num_tiles + tile0;
    if (tiles_here == RS_HIST_TILES && (num_tiles & 3) == 0) {
      static_assert(RS_HIST_TILES == 8, "two 16-byte stores per digit");
      reinterpret_cast<uint4 *>(dst)[0] = reinterpret_cast<const uint4 *>(mine)[0];
      reinterpret_cast<uint4 *>(dst)[1] = reinterpret_cast<const uint4 *>(mine)[1];
    } else {
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

constexpr size_t RS_LDS_FIXED = RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4 + 64;

// Ranked scatter.  Inside a wave, lanes with equal digits find each other with
// eight ballots; per-wave digit counters in LDS chain the 16 rounds; the tile
// is then reordered in LDS so that the global stores of a wave are contiguous
// runs per digit.  Order is preserved at every level (round, lane, wave, tile).
// The stores stay ordinary ones: the runs are shorter than a cache line, and
// non-temporal stores, which help every streaming kernel here, cost 35 % (L2
// no longer merges the pieces of a line).
template <class K, int VB, class DigitFn>
__global__ __launch_bounds__(RS_BLOCK) void rs_scatter_kernel(
    const K *__restrict__ kin, K *__restrict__ kout, const void *__restrict__ vin_,
    void *__restrict__ vout_, int64_t n, DigitFn fn, int pass, const uint32_t *__restrict__ offs,
    int64_t num_tiles) {
  using V = typename ValType<VB>::T;
  const V *vin = reinterpret_cast<const V *>(vin_);
  V *vout = reinterpret_cast<V *>(vout_);

  extern __shared__ __align__(16) unsigned char s_raw[];
  uint32_t(*cnt)[RS_RADIX] = reinterpret_cast<uint32_t(*)[RS_RADIX]>(s_raw);
  uint32_t *s_dbase = reinterpret_cast<uint32_t *>(s_raw + RS_WAVES * RS_RADIX * 4);
  uint32_t *s_tab = s_dbase + RS_RADIX;
  uint32_t *s_wsum = s_tab + RS_RADIX;  // 4 used
  unsigned char *buf = s_raw + RS_LDS_FIXED;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int lane = lane_id();
  const int64_t tile = blockIdx.x;
  const int64_t base = tile * RS_TILE;
  const int64_t rem = n - base;
  const int tile_n = (int)(rem < RS_TILE ? rem : RS_TILE);

  for (int i = tid; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&cnt[0][0])[i] = 0u;
  // Global offsets of this tile, one digit per thread (strided, L2-resident).
  uint32_t goff = 0;
  if (tid < RS_RADIX) goff = offs[(int64_t)tid * num_tiles + tile];
  __syncthreads();

  // Wave-striped arrangement: wave w owns keys [w*64*KPT, (w+1)*64*KPT) of the
  // tile, round r is 64 consecutive keys.
  K key[RS_KPT];
  int pos[RS_KPT];
  const int wbase = wave * WAVE * RS_KPT;
  const bool full = tile_n == RS_TILE;  // uniform over the block
  if (full) {
    const K *src = kin + base + wbase + lane;
#pragma unroll
    for (int r = 0; r < RS_KPT; r++) key[r] = src[r * WAVE];
  } else {
#pragma unroll
    for (int r = 0; r < RS_KPT; r++) {
      const int t = wbase + r * WAVE + lane;
      key[r] = (t < tile_n) ? kin[base + t] : (K)0;
    }
  }
  // The kernel is bound by vector-ALU issue, so the match is written in 32-bit
  // halves: `differ` collects the lanes whose digit differs from this lane's in
  // some bit (ballot of bit b XOR this lane's bit b, broadcast as 0 / ~0).
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const bool valid = full || (wbase + r * WAVE + lane < tile_n);
    const uint32_t d = fn(key[r], pass);
    uint32_t differ_lo = 0u, differ_hi = 0u;
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const uint32_t mine = (uint32_t)(((int32_t)(d << (31 - b))) >> 31);  // 0 or ~0
      const uint64_t m = __ballot(mine != 0u);
      differ_lo |= (uint32_t)m ^ mine;
      differ_hi |= (uint32_t)(m >> 32) ^ mine;
    }
    const uint64_t vm = __ballot(valid);
    const uint32_t peers_lo = ~differ_lo & (uint32_t)vm;
    const uint32_t peers_hi = ~differ_hi & (uint32_t)(vm >> 32);
    const int rank = (int)__builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
    int p = 0;
    if (valid) {
      const uint32_t prev = cnt[wave][d];
      p = (int)prev + rank;
      if (rank == 0)
        cnt[wave][d] = prev + (uint32_t)(__builtin_popcount(peers_lo) + __builtin_popcount(peers_hi));
    }
    pos[r] = p;
  }
  __syncthreads();

  // Per digit: exclusive prefix over waves, then exclusive prefix over digits.
  uint32_t total = 0, incl = 0;
  if (tid < RS_RADIX) {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < RS_WAVES; w++) {
      const uint32_t c = cnt[w][tid];
      cnt[w][tid] = run;
      run += c;
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
    s_dbase[tid] = dbase;
    // destination of element i of the reordered tile with digit d: tab[d] + i
    s_tab[tid] = goff - dbase;
  }
  __syncthreads();

  // Reorder keys inside LDS.
  K *kbuf = reinterpret_cast<K *>(buf);
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const int t = wbase + r * WAVE + lane;
    if (t < tile_n) {
      const uint32_t d = fn(key[r], pass);
      pos[r] += (int)(s_dbase[d] + cnt[wave][d]);
      kbuf[pos[r]] = key[r];
    }
  }
  __syncthreads();
  uint32_t dst[RS_KPT];
#pragma unroll
  for (int j = 0; j < RS_KPT; j++) {
    const int i = j * RS_BLOCK + tid;
    dst[j] = 0;
    if (i < tile_n) {
      const K k = kbuf[i];
      dst[j] = s_tab[fn(k, pass)] + (uint32_t)i;
      // The offsets come from this library's own histogram and scan; should
      // they ever be wrong, a store outside the output would fault the GPU,
      // whereas a dropped key is a wrong result the caller can see.
      if ((int64_t)dst[j] < n) kout[dst[j]] = k;
    }
  }
  if constexpr (VB != 0) {
    __syncthreads();
    V *vbuf = reinterpret_cast<V *>(buf);
#pragma unroll
    for (int r = 0; r < RS_KPT; r++) {
      const int t = wbase + r * WAVE + lane;
      if (t < tile_n) vbuf[pos[r]] = vin[base + t];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < RS_KPT; j++) {
      const int i = j * RS_BLOCK + tid;
      if (i < tile_n && (int64_t)dst[j] < n) vout[dst[j]] = vbuf[i];
    }
  }
}

// One pass: keys (and values) move from *in to *out ordered by digit `pass`,
// equal digits keeping their order.  `epoch` must grow from call to call on
// the same scratch (1, 2, ...).  Afterwards sc.offsets[d * tiles] is the
// position where digit d starts in the output.
template <class K, int VB, class DigitFn>
static int rs_pass(hipStream_t st, const K *kin, K *kout, const void *vin, void *vout, int64_t n,
                   DigitFn fn, int pass, uint32_t epoch, const RsScratch &sc) {
  using V = typename ValType<VB>::T;
  const size_t lds =
      RS_LDS_FIXED + (size_t)RS_TILE * (sizeof(K) > sizeof(V) ? sizeof(K) : sizeof(V));
  auto scatter = rs_scatter_kernel<K, VB, DigitFn>;
  // Initialised once, under the lock C++ gives function-local statics.
  static const hipError_t raised = hipFuncSetAttribute(
      (const void *)scatter, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (raised != hipSuccess) return (int)raised;
  hipLaunchKernelGGL((rs_hist_kernel<K, DigitFn>),
                     dim3((unsigned)ceil_div(sc.tiles, (int64_t)RS_HIST_TILES)), dim3(RS_BLOCK), 0, st,
                     kin, n, fn, pass, sc.counts, sc.tiles);
  int rc = launch_status();
  if (rc != 0) return rc;
  rc = fa_segscan((fa_stream_t)st, FA_U32, FA_ADD, sc.counts, nullptr, sc.tiles * RS_RADIX, 1,
                  sc.offsets, sc.lookback, sc.lookback_bytes, epoch);
  if (rc != 0) return rc;
  hipLaunchKernelGGL(scatter, dim3((unsigned)sc.tiles), dim3(RS_BLOCK), lds, st, kin, kout, vin,
                     vout, n, fn, pass, sc.offsets, sc.tiles);
  return launch_status();
}

}  // namespace fa
