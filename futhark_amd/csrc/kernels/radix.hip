// Stable LSD radix sort for gfx950, 8-bit digits, one read and one write of the
// data per pass.
//
// Result-wise each pass is the composition the reference reaches radix sort
// through (tests/issue2234.fut:10-44, tests/ad/custom/radixsort.fut:13-25): a
// histogram of the digit (SegHist), an exclusive scan of the counts (SegScan)
// and a scatter to offset + rank (src/Futhark/Tools.hs:328-363).  The schedule
// fuses them so that no n-length intermediate ever exists:
//   * one up-front kernel builds the digit histograms of ALL passes from a
//     single read of the keys (LDS sub-histograms per wave, one flush);
//   * a pass is ONE kernel.  A tile (1024 threads x 16 keys) ranks its keys:
//     inside a wave, lanes with equal digits find each other with eight
//     ballots; per-wave digit counters in LDS chain the 16 rounds.  The tile's
//     256 digit counts are published and the counts of all earlier tiles are
//     gathered by decoupled look-back, one thread per digit (the chained-scan
//     protocol of SegScan/SinglePass.hs:625-777 applied to 256 counters at
//     once), which replaces the separate count-scan kernel;
//   * the tile is reordered in LDS so that global stores are contiguous runs
//     per digit.
// Order is preserved at every level (round, lane, wave, tile): the sort is
// stable.  The same pass, with a digit function that maps a histogram bin to
// its LDS-sized bin range, partitions (index, value) pairs for large
// histograms (seghist.hip).
#include "radix.hip.h"

namespace fa {

// Digits of pass p are bits [begin + 8p, begin + 8p + 8) of the key.
template <class K> struct DigitBits {
  int begin_bit;
  __device__ __forceinline__ uint32_t operator()(K key, int pass) const {
    return (uint32_t)(key >> (begin_bit + 8 * pass)) & 0xffu;
  }
};

template <class K, int VB>
static int sort_passes(hipStream_t st, const K *kin, K *kout, K *ktmp, const void *vin, void *vout,
                       void *vtmp, int64_t n, int begin_bit, int end_bit, void *scratch) {
  const int passes = (end_bit - begin_bit) / 8;
  const int64_t tiles = rs_num_tiles(n);
  RsScratch sc = rs_carve(scratch, tiles, passes);
  DigitBits<K> fn{begin_bit};
  int rc = rs_prepare<K>(st, kin, n, fn, passes, sc);
  if (rc != 0) return rc;
  // With an even number of passes the ping-pong ends in `out` if it starts by
  // writing `tmp`; with an odd number it starts by writing `out`.
  const K *src_k = kin;
  const void *src_v = vin;
  for (int p = 0; p < passes; p++) {
    const bool to_out = ((passes - 1 - p) % 2) == 0;
    K *dst_k = to_out ? kout : ktmp;
    void *dst_v = to_out ? vout : vtmp;
    rc = rs_pass<K, VB>(st, src_k, dst_k, src_v, dst_v, n, fn, p, sc);
    if (rc != 0) return rc;
    src_k = dst_k;
    src_v = dst_v;
  }
  return 0;
}

}  // namespace fa

extern "C" size_t fa_radix_sort_scratch_bytes(int64_t n) {
  if (n < 0) n = 0;
  return rs_scratch_bytes(rs_num_tiles(n), 8);
}

extern "C" int fa_radix_sort(fa_stream_t stream, int key_bytes, int val_bytes, const void *keys_in,
                             void *keys_out, void *keys_tmp, const void *vals_in, void *vals_out,
                             void *vals_tmp, int64_t n, int begin_bit, int end_bit, void *scratch,
                             size_t scratch_bytes) {
  if (n < 0 || n >= ((int64_t)1 << 30)) return FA_EINVAL;
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
