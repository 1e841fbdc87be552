// Stable LSD radix sort for gfx950, 8-bit digits.
//
// Each pass is the composition the reference reaches radix sort through
// (tests/issue2234.fut:10-44, tests/ad/custom/radixsort.fut:13-25): a histogram
// of the digit per tile (SegHist), an exclusive scan of the counts laid out
// digit-major (SegScan, the single-pass kernel of segscan.hip) and a scatter
// to the scanned offsets plus the rank of the key inside its tile
// (src/Futhark/Tools.hs:328-363 for scatter).  The rank is computed without any
// n-length intermediate: inside a wave, lanes with equal digits find each other
// with eight ballots; per-wave digit counters in LDS chain the rounds; the tile
// is then reordered in LDS so that the global stores of a wave are contiguous
// runs per digit.  Order is preserved at every level (round, lane, wave, tile),
// which makes the sort stable.
#include "dispatch.hip.h"

namespace fa {

constexpr int RS_BLOCK = 512;
constexpr int RS_WAVES = RS_BLOCK / WAVE;
constexpr int RS_KPT = 16;  // keys per thread
constexpr int RS_TILE = RS_BLOCK * RS_KPT;
constexpr int RS_RADIX = 256;

template <class K>
__global__ __launch_bounds__(RS_BLOCK) void radix_hist_kernel(const K *__restrict__ keys, int64_t n,
                                                              int shift, uint32_t *counts,
                                                              int64_t num_tiles) {
  __shared__ uint32_t h[RS_WAVES][RS_RADIX];
  for (int i = threadIdx.x; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&h[0][0])[i] = 0u;
  __syncthreads();
  const int wave = threadIdx.x / WAVE;
  const int64_t base = (int64_t)blockIdx.x * RS_TILE;
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const int64_t idx = base + r * RS_BLOCK + threadIdx.x;
    if (idx < n) atomicAdd(&h[wave][(uint32_t)(keys[idx] >> shift) & 0xffu], 1u);
  }
  __syncthreads();
  if (threadIdx.x < RS_RADIX) {
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < RS_WAVES; w++) c += h[w][threadIdx.x];
    counts[(int64_t)threadIdx.x * num_tiles + blockIdx.x] = c;
  }
}

template <int BYTES> struct ValType;
template <> struct ValType<0> { using T = uint32_t; };
template <> struct ValType<4> { using T = uint32_t; };
template <> struct ValType<8> { using T = uint64_t; };

template <class K, int VB>
__global__ __launch_bounds__(RS_BLOCK) void radix_scatter_kernel(
    const K *__restrict__ kin, K *__restrict__ kout, const void *__restrict__ vin_,
    void *__restrict__ vout_, int64_t n, int shift, const uint32_t *__restrict__ offs,
    int64_t num_tiles) {
  using V = typename ValType<VB>::T;
  const V *vin = reinterpret_cast<const V *>(vin_);
  V *vout = reinterpret_cast<V *>(vout_);

  extern __shared__ __align__(16) unsigned char s_raw[];
  uint32_t(*cnt)[RS_RADIX] = reinterpret_cast<uint32_t(*)[RS_RADIX]>(s_raw);
  uint32_t *s_dbase = reinterpret_cast<uint32_t *>(s_raw + RS_WAVES * RS_RADIX * 4);
  uint32_t *s_tab = s_dbase + RS_RADIX;
  uint32_t *s_wsum = s_tab + RS_RADIX;  // 4 used, 16 reserved
  unsigned char *buf = s_raw + RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4 + 64;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int lane = lane_id();
  const int64_t tile = blockIdx.x;
  const int64_t base = tile * RS_TILE;
  const int64_t rem = n - base;
  const int tile_n = (int)(rem < RS_TILE ? rem : RS_TILE);
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

  for (int i = tid; i < RS_WAVES * RS_RADIX; i += RS_BLOCK) (&cnt[0][0])[i] = 0u;
  __syncthreads();

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
    const uint32_t d = (uint32_t)(key[r] >> shift) & 0xffu;
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
    s_tab[tid] = offs[(int64_t)tid * num_tiles + tile] - dbase;
  }
  __syncthreads();

  // Reorder keys inside LDS.
  K *kbuf = reinterpret_cast<K *>(buf);
#pragma unroll
  for (int r = 0; r < RS_KPT; r++) {
    const int t = wbase + r * WAVE + lane;
    if (t < tile_n) {
      const uint32_t d = (uint32_t)(key[r] >> shift) & 0xffu;
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
      dst[j] = s_tab[(uint32_t)(k >> shift) & 0xffu] + (uint32_t)i;
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

constexpr size_t RS_LDS_FIXED = RS_WAVES * RS_RADIX * 4 + 2 * RS_RADIX * 4 + 64;

static int64_t rs_num_tiles(int64_t n) { return ceil_div(n, (int64_t)RS_TILE); }

struct RsScratch {
  uint32_t *counts;
  uint32_t *offsets;
  void *lookback;
  size_t lookback_bytes;
};

static size_t rs_align(size_t x) { return (x + 255) & ~(size_t)255; }

template <class K, int VB>
static int sort_passes(hipStream_t st, const K *kin, K *kout, K *ktmp, const void *vin, void *vout,
                       void *vtmp, int64_t n, int begin_bit, int end_bit, const RsScratch &sc) {
  using V = typename ValType<VB>::T;
  const int64_t tiles = rs_num_tiles(n);
  const int passes = (end_bit - begin_bit) / 8;
  const size_t lds = RS_LDS_FIXED + (size_t)RS_TILE * (sizeof(K) > sizeof(V) ? sizeof(K) : sizeof(V));
  auto scatter = radix_scatter_kernel<K, VB>;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void *)scatter,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    raised = true;
  }
  // With an even number of passes the ping-pong ends in `out` if it starts by
  // writing `tmp`; with an odd number it starts by writing `out`.
  const K *src_k = kin;
  const void *src_v = vin;
  for (int p = 0; p < passes; p++) {
    const bool to_out = ((passes - 1 - p) % 2) == 0;
    K *dst_k = to_out ? kout : ktmp;
    void *dst_v = to_out ? vout : vtmp;
    const int shift = begin_bit + 8 * p;
    hipLaunchKernelGGL((radix_hist_kernel<K>), dim3((unsigned)tiles), dim3(RS_BLOCK), 0, st, src_k,
                       n, shift, sc.counts, tiles);
    int rc = launch_status();
    if (rc != 0) return rc;
    rc = fa_segscan((fa_stream_t)st, FA_U32, FA_ADD, sc.counts, nullptr, tiles * RS_RADIX, 1,
                    sc.offsets, sc.lookback, sc.lookback_bytes, (uint32_t)(p + 1));
    if (rc != 0) return rc;
    hipLaunchKernelGGL(scatter, dim3((unsigned)tiles), dim3(RS_BLOCK), lds, st, src_k, dst_k, src_v,
                       dst_v, n, shift, sc.offsets, tiles);
    rc = launch_status();
    if (rc != 0) return rc;
    src_k = dst_k;
    src_v = dst_v;
  }
  return 0;
}

}  // namespace fa

extern "C" size_t fa_radix_sort_scratch_bytes(int64_t n) {
  if (n < 0) n = 0;
  const int64_t tiles = rs_num_tiles(n) < 1 ? 1 : rs_num_tiles(n);
  const size_t counts = rs_align((size_t)tiles * RS_RADIX * 4);
  return 2 * counts + rs_align(fa_segscan_scratch_bytes(FA_U32, tiles * RS_RADIX));
}

extern "C" int fa_radix_sort(fa_stream_t stream, int key_bytes, int val_bytes, const void *keys_in,
                             void *keys_out, void *keys_tmp, const void *vals_in, void *vals_out,
                             void *vals_tmp, int64_t n, int begin_bit, int end_bit, void *scratch,
                             size_t scratch_bytes) {
  if (n < 0 || n >= ((int64_t)1 << 31)) return FA_EINVAL;
  if (key_bytes != 4 && key_bytes != 8) return FA_ENOTSUP;
  if (val_bytes != 0 && val_bytes != 4 && val_bytes != 8) return FA_ENOTSUP;
  if (begin_bit < 0 || end_bit > key_bytes * 8 || end_bit < begin_bit ||
      (end_bit - begin_bit) % 8 != 0)
    return FA_EINVAL;
  if (n == 0) return 0;
  if (!keys_in || !keys_out || !keys_tmp || !scratch) return FA_EINVAL;
  if (val_bytes && (!vals_in || !vals_out || !vals_tmp)) return FA_EINVAL;
  if (scratch_bytes < fa_radix_sort_scratch_bytes(n)) return FA_ESCRATCH;
  if (!is_aligned(scratch, 256)) return FA_EALIGN;
  hipStream_t st = (hipStream_t)stream;

  if (end_bit == begin_bit) {  // nothing to sort by: the identity permutation
    hipError_t e = hipMemcpyAsync(keys_out, keys_in, (size_t)n * key_bytes,
                                  hipMemcpyDeviceToDevice, st);
    if (e == hipSuccess && val_bytes)
      e = hipMemcpyAsync(vals_out, vals_in, (size_t)n * val_bytes, hipMemcpyDeviceToDevice, st);
    return e == hipSuccess ? 0 : (int)e;
  }

  const int64_t tiles = rs_num_tiles(n);
  const size_t counts = rs_align((size_t)tiles * RS_RADIX * 4);
  RsScratch sc;
  sc.counts = (uint32_t *)scratch;
  sc.offsets = (uint32_t *)((char *)scratch + counts);
  sc.lookback = (char *)scratch + 2 * counts;
  sc.lookback_bytes = scratch_bytes - 2 * counts;
  // The look-back region starts zeroed; each pass then uses its own epoch.
  int rc = fa_replicate(stream, 4, sc.lookback,
                        (int64_t)(fa_segscan_scratch_bytes(FA_U32, tiles * RS_RADIX) / 4), 0);
  if (rc != 0) return rc;

#define FA_SORT(K, VB)                                                                         \
  return sort_passes<K, VB>(st, (const K *)keys_in, (K *)keys_out, (K *)keys_tmp, vals_in,    \
                            vals_out, vals_tmp, n, begin_bit, end_bit, sc)
  if (key_bytes == 4) {
    if (val_bytes == 0) FA_SORT(uint32_t, 0);
    if (val_bytes == 4) FA_SORT(uint32_t, 4);
    FA_SORT(uint32_t, 8);
  } else {
    if (val_bytes == 0) FA_SORT(uint64_t, 0);
    if (val_bytes == 4) FA_SORT(uint64_t, 4);
    FA_SORT(uint64_t, 8);
  }
#undef FA_SORT
}
