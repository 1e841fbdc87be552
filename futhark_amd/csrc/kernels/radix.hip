// Stable LSD radix sort for gfx950, 8-bit digits.
//
// Each pass is the composition the reference reaches radix sort through
// (tests/issue2234.fut:10-44, tests/ad/custom/radixsort.fut:13-25): a histogram
// of the digit per tile (SegHist), an exclusive scan of the counts laid out
// digit-major (SegScan, the single-pass kernel of segscan.hip) and a scatter
// to the scanned offset plus the rank of the key inside its tile
// (src/Futhark/Tools.hs:328-363 for scatter).  The rank is computed without any
// n-length intermediate (radix.hip.h).  The sort is stable.
#include "radix.hip.h"

namespace fa {

// Digits of pass p are bits [begin + 8p, begin + 8p + 8) of the key.
template <class K> struct DigitBits {
  using Out = K;
  int begin_bit;
  __device__ __forceinline__ K out(K key) const { return key; }
  __device__ __forceinline__ uint32_t operator()(K key, int pass) const {
    return (uint32_t)(key >> (begin_bit + 8 * pass)) & 0xffu;
  }
};

// 64-bit positions: needed from RS_WIDE_N keys on, or asked for.
static bool sort_wide(int64_t n) {
  fa_tuning t;
  fa_get_tuning(&t);
  return n >= RS_WIDE_N || t.sort_wide_positions != 0;
}

template <class K, int VB>
static int sort_passes(hipStream_t st, const K *kin, K *kout, K *ktmp, const void *vin, void *vout,
                       void *vtmp, int64_t n, int begin_bit, int end_bit, void *scratch) {
  const int passes = (end_bit - begin_bit) / 8;
  const bool wide = sort_wide(n);
  RsScratch sc = rs_carve(scratch, rs_num_tiles(n), wide);
  DigitBits<K> fn{begin_bit};
  int rc = rs_prepare(st, sc);
  if (rc != 0) return rc;
  // With an even number of passes the ping-pong ends in `out` if it starts by
  // writing `tmp`; with an odd number it starts by writing `out`.
  const K *src_k = kin;
  const void *src_v = vin;
  for (int p = 0; p < passes; p++) {
    const bool to_out = ((passes - 1 - p) % 2) == 0;
    K *dst_k = to_out ? kout : ktmp;
    void *dst_v = to_out ? vout : vtmp;
    rc = wide ? rs_pass<K, VB, DigitBits<K>, uint64_t>(st, src_k, dst_k, src_v, dst_v, n, fn, p,
                                                       (uint32_t)(p + 1), sc)
              : rs_pass<K, VB, DigitBits<K>, uint32_t>(st, src_k, dst_k, src_v, dst_v, n, fn, p,
                                                       (uint32_t)(p + 1), sc);
    if (rc != 0) return rc;
    src_k = dst_k;
    src_v = dst_v;
  }
  return 0;
}

}  // namespace fa

extern "C" size_t fa_radix_sort_scratch_bytes(int64_t n) {
  if (n < 0) n = 0;
  return rs_scratch_bytes(rs_num_tiles(n), sort_wide(n));
}

extern "C" int fa_radix_sort(fa_stream_t stream, int key_bytes, int val_bytes, const void *keys_in,
                             void *keys_out, void *keys_tmp, const void *vals_in, void *vals_out,
                             void *vals_tmp, int64_t n, int begin_bit, int end_bit, void *scratch,
                             size_t scratch_bytes) {
  if (n < 0) return FA_EINVAL;
  if (key_bytes != 4 && key_bytes != 8) return FA_ENOTSUP;
  if (val_bytes != 0 && val_bytes != 4 && val_bytes != 8) return FA_ENOTSUP;
  if (begin_bit < 0 || end_bit > key_bytes * 8 || end_bit < begin_bit ||
      (end_bit - begin_bit) % 8 != 0)
    return FA_EINVAL;
  if (n == 0) return 0;
  if (!keys_in || !keys_out || !keys_tmp || !scratch) return FA_EINVAL;
  if (val_bytes && (!vals_in || !vals_out || !vals_tmp)) return FA_EINVAL;
  if (scratch_bytes < fa_radix_sort_scratch_bytes(n)) return FA_ESCRATCH;
  if (!is_aligned(scratch, 256) || !is_aligned(keys_in, 16)) return FA_EALIGN;
  hipStream_t st = (hipStream_t)stream;

  if (end_bit == begin_bit) {  // nothing to sort by: the identity permutation
    hipError_t e = hipMemcpyAsync(keys_out, keys_in, (size_t)n * key_bytes,
                                  hipMemcpyDeviceToDevice, st);
    if (e == hipSuccess && val_bytes)
      e = hipMemcpyAsync(vals_out, vals_in, (size_t)n * val_bytes, hipMemcpyDeviceToDevice, st);
    return e == hipSuccess ? 0 : (int)e;
  }

#define FA_SORT(K, VB)                                                                         \
  return sort_passes<K, VB>(st, (const K *)keys_in, (K *)keys_out, (K *)keys_tmp, vals_in,    \
                            vals_out, vals_tmp, n, begin_bit, end_bit, scratch)
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
