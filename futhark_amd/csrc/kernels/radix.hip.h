// Kernels of the 8-bit radix pass shared by the sort (radix.hip) and by the
// bin-range partition of large histograms (seghist.hip): up-front digit
// histograms, their exclusive scan, and the single-kernel ranked scatter with
// decoupled look-back over the 256 digit counters of each tile.
#pragma once

#include "dispatch.hip.h"

namespace fa {

constexpr int RS_BLOCK = 1024;
constexpr int RS_WAVES = RS_BLOCK / WAVE;
constexpr int RS_KPT = 16;  // keys per thread
constexpr int RS_TILE = RS_BLOCK * RS_KPT;
constexpr int RS_RADIX = 256;
constexpr int RS_MAX_PASSES = 8;

// Same-address device atomics complete at about one per 12 ns, so a tile must
// be large: 16384 keys per ticket keeps the ticket rate above the data rate.

constexpr uint32_t RS_ST_A = 1u << 30;  // count of this tile
constexpr uint32_t RS_ST_P = 2u << 30;  // count of this tile and all before it
constexpr uint32_t RS_COUNT_MASK = (1u << 30) - 1;

struct RsScratch {
  uint32_t *tickets;  // [passes]
  uint32_t *ghist;    // [passes][256]
  uint32_t *gbase;    // [passes][256] exclusive scan of ghist
  uint32_t *desc;     // [passes][tiles][256]
  size_t zero_words;  // words to clear before use, from `tickets`
  int64_t tiles;
};

static inline int64_t rs_num_tiles(int64_t n) { return ceil_div(n, (int64_t)RS_TILE); }

static inline size_t rs_scratch_bytes(int64_t tiles, int passes) {
  if (tiles < 1) tiles = 1;
  return 256 + 2 * (size_t)RS_MAX_PASSES * RS_RADIX * 4 + (size_t)passes * tiles * RS_RADIX * 4;
}

static inline RsScratch rs_carve(void *scratch, int64_t tiles, int passes) {
  RsScratch sc;
  char *p = (char *)scratch;
  sc.tickets = (uint32_t *)p;
  sc.ghist = (uint32_t *)(p + 256);
  sc.gbase = sc.ghist + RS_MAX_PASSES * RS_RADIX;
  sc.desc = sc.gbase + RS_MAX_PASSES * RS_RADIX;
  sc.zero_words = rs_scratch_bytes(tiles, passes) / 4;
  sc.tiles = tiles;
  return sc;
}

static __global__ __launch_bounds__(256) void rs_zero_kernel(uint4 *p, size_t nvec) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride)
    p[i] = make_uint4(0, 0, 0, 0);
}

// Digit histograms of all passes from one read of the keys.
template <class K, class DigitFn>
__global__ __launch_bounds__(RS_BLOCK) void rs_count_kernel(const K *__restrict__ keys, int64_t n,
                                                            DigitFn fn, int passes,
                                                            uint32_t *ghist) {
  constexpr int COPIES = 4;
  constexpr int VEC = 16 / sizeof(K);
  __shared__ uint32_t h[COPIES][RS_MAX_PASSES][RS_RADIX];
  for (int i = threadIdx.x; i < COPIES * RS_MAX_PASSES * RS_RADIX; i += RS_BLOCK)
    (&h[0][0][0])[i] = 0u;
  __syncthreads();
  const int copy = (threadIdx.x / WAVE) % COPIES;
  const int64_t nvec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * RS_BLOCK;
  for (int64_t i = (int64_t)blockIdx.x * RS_BLOCK + threadIdx.x; i < nvec; i += stride) {
    const Vec16<K> v = load_vec16(keys + i * VEC);
#pragma unroll
    for (int e = 0; e < VEC; e++)
      for (int p = 0; p < passes; p++) atomicAdd(&h[copy][p][fn(v.e[e], p)], 1u);
  }
  if (blockIdx.x == 0) {
    const int64_t t = nvec * VEC + threadIdx.x;
    if (threadIdx.x < VEC && t < n)
      for (int p = 0; p < passes; p++) atomicAdd(&h[copy][p][fn(keys[t], p)], 1u);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < passes * RS_RADIX; i += RS_BLOCK) {
    uint32_t c = 0;
#pragma unroll
    for (int q = 0; q < COPIES; q++) c += (&h[q][0][0])[i];
    if (c) atomicAdd(&ghist[i], c);
  }
}

// gbase[p][d] = number of keys whose digit in pass p is below d.
static __global__ __launch_bounds__(RS_RADIX) void rs_base_kernel(const uint32_t *ghist, uint32_t *gbase) {
  __shared__ uint32_t wsum[RS_RADIX / WAVE];
  const int p = blockIdx.x, d = threadIdx.x;
  const uint32_t c = ghist[p * RS_RADIX + d];
  const uint32_t incl = wave_incl_scan<uint32_t, OpAdd<uint32_t>>(c);
  if (lane_id() == 63) wsum[d / WAVE] = incl;
  __syncthreads();
  uint32_t pre = 0;
  for (int w = 0; w < d / WAVE; w++) pre += wsum[w];
  gbase[p * RS_RADIX + d] = pre + incl - c;
}

template <int BYTES> struct ValType;
template <> struct ValType<0> { using T = uint32_t; };
template <> struct ValType<4> { using T = uint32_t; };
template <> struct ValType<8> { using T = uint64_t; };

constexpr size_t RS_LDS_FIXED = RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4 + 128;

template <class K, int VB, class DigitFn>
__global__ __launch_bounds__(RS_BLOCK) void rs_pass_kernel(
    const K *__restrict__ kin, K *__restrict__ kout, const void *__restrict__ vin_,
    void *__restrict__ vout_, int64_t n, DigitFn fn, int pass, uint32_t *ticket,
    const uint32_t *__restrict__ gbase, uint32_t *desc) {
  using V = typename ValType<VB>::T;
  const V *vin = reinterpret_cast<const V *>(vin_);
  V *vout = reinterpret_cast<V *>(vout_);

  extern __shared__ __align__(16) unsigned char s_raw[];
  uint32_t(*cnt)[RS_RADIX] = reinterpret_cast<uint32_t(*)[RS_RADIX]>(s_raw);
  uint32_t *s_dbase = reinterpret_cast<uint32_t *>(s_raw + RS_WAVES * RS_RADIX * 4);
  uint32_t *s_tab = s_dbase + RS_RADIX;
  uint32_t *s_misc = s_tab + RS_RADIX;  // [0..3] wave sums, [8] tile id
  unsigned char *buf = s_raw + RS_LDS_FIXED;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int lane = lane_id();
  if (tid == 0) s_misc[8] = atomicAdd(ticket, 1u);
  for (int i = tid; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&cnt[0][0])[i] = 0u;
  __syncthreads();
  const int64_t tile = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_misc[8]);
  const int64_t base = tile * RS_TILE;
  const int64_t rem = n - base;
  const int tile_n = (int)(rem < RS_TILE ? rem : RS_TILE);
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

  // Wave-striped arrangement: wave w owns keys [w*64*KPT, (w+1)*64*KPT) of the
  // tile, round r is 64 consecutive keys.
  K key[RS_KPT];
  int pos[RS_KPT];
  const int wbase = wave * WAVE * RS_KPT;
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const int t = wbase + r * WAVE + lane;
    key[r] = (t < tile_n) ? kin[base + t] : (K)0;
  }
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const int t = wbase + r * WAVE + lane;
    const bool valid = t < tile_n;
    const uint32_t d = fn(key[r], pass);
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const bool bit = (d >> b) & 1u;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const int rank = __builtin_popcountll(peers & lt_mask);
    const int count = __builtin_popcountll(peers);
    int p = 0;
    if (valid) {
      const uint32_t prev = cnt[wave][d];
      p = (int)prev + rank;
      if (rank == 0) cnt[wave][d] = prev + (uint32_t)count;
    }
    pos[r] = p;
  }
  __syncthreads();

  // Per digit: exclusive prefix over the waves of the tile; publish the count.
  uint32_t total = 0, incl = 0;
  uint32_t *my_desc = desc + tile * RS_RADIX + tid;
  if (tid < RS_RADIX) {
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < RS_WAVES; w++) {
      const uint32_t c = cnt[w][tid];
      cnt[w][tid] = run;
      run += c;
    }
    total = run;
    st_relaxed_u32(my_desc, (tile == 0 ? RS_ST_P : RS_ST_A) | total);
    incl = wave_incl_scan<uint32_t, OpAdd<uint32_t>>(total);
    if (lane == 63) s_misc[wave] = incl;
  }
  __syncthreads();
  if (tid < RS_RADIX) {
    uint32_t wpre = 0;
    for (int w = 0; w < wave; w++) wpre += s_misc[w];
    const uint32_t dbase = wpre + incl - total;
    // Look back: add the counts of earlier tiles until one carries a prefix.
    // Four predecessors are read per round trip.
    uint32_t prefix = 0;
    if (tile > 0) {
      int64_t j = tile - 1;
      bool done = false;
      while (!done) {
        uint32_t v[4];
#pragma unroll
        for (int q = 0; q < 4; q++)
          v[q] = (j - q >= 0) ? ld_relaxed_u32(desc + (j - q) * RS_RADIX + tid) : RS_ST_P;
        int used = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          if (done || used != q) continue;
          const uint32_t st = v[q] >> 30;
          if (st == 0) continue;  // not published yet: read again from here
          prefix += v[q] & RS_COUNT_MASK;
          used = q + 1;
          if (st == 2) done = true;
        }
        j -= used;
        if (used == 0) __builtin_amdgcn_s_sleep(1);
      }
      st_relaxed_u32(my_desc, RS_ST_P | (prefix + total));
    }
    s_dbase[tid] = dbase;
    // destination of element i of the reordered tile with digit d: tab[d] + i
    s_tab[tid] = gbase[tid] + prefix - dbase;
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
      kout[dst[j]] = k;
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
      if (i < tile_n) vout[dst[j]] = vbuf[i];
    }
  }
}

static inline int rs_num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    cus = NUM_CUS_HINT;
    if (hipGetDevice(&dev) == hipSuccess)
      (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  }
  return cus;
}

// Clears the scratch, builds the digit histograms of `passes` passes and their
// exclusive scans.
template <class K, class DigitFn>
static int rs_prepare(hipStream_t st, const K *keys, int64_t n, DigitFn fn, int passes,
                      const RsScratch &sc) {
  const size_t nvec = (sc.zero_words + 3) / 4;
  int zgrid = (int)(ceil_div((int64_t)nvec, 256) < 2048 ? ceil_div((int64_t)nvec, 256) : 2048);
  hipLaunchKernelGGL(rs_zero_kernel, dim3(zgrid), dim3(256), 0, st, (uint4 *)sc.tickets, nvec);
  int64_t want = ceil_div(n, (int64_t)RS_BLOCK * 16);
  const int limit = rs_num_cus() * 2;
  const int grid = (int)(want < 1 ? 1 : (want > limit ? limit : want));
  hipLaunchKernelGGL((rs_count_kernel<K, DigitFn>), dim3(grid), dim3(RS_BLOCK), 0, st, keys, n, fn,
                     passes, sc.ghist);
  hipLaunchKernelGGL(rs_base_kernel, dim3(passes), dim3(RS_RADIX), 0, st, sc.ghist, sc.gbase);
  return launch_status();
}

// One pass: keys (and values) move from *in to *out ordered by digit `pass`,
// equal digits keeping their order.
template <class K, int VB, class DigitFn>
static int rs_pass(hipStream_t st, const K *kin, K *kout, const void *vin, void *vout, int64_t n,
                   DigitFn fn, int pass, const RsScratch &sc) {
  using V = typename ValType<VB>::T;
  const size_t lds =
      RS_LDS_FIXED + (size_t)RS_TILE * (sizeof(K) > sizeof(V) ? sizeof(K) : sizeof(V));
  auto kernel = rs_pass_kernel<K, VB, DigitFn>;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void *)kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    raised = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)sc.tiles), dim3(RS_BLOCK), lds, st, kin, kout, vin, vout,
                     n, fn, pass, sc.tickets + pass, sc.gbase + pass * RS_RADIX,
                     sc.desc + (size_t)pass * sc.tiles * RS_RADIX);
  return launch_status();
}

}  // namespace fa
