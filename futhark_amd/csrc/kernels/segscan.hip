// SegScan for gfx950: single-pass scan with decoupled look-back.
//
// What is computed follows src/Futhark/CodeGen/ImpGen/GPU/SegScan/SinglePass.hs
// (dynamic tile ids :443-461, tile aggregate/prefix publication with status
// X/A/P :128-131,625-777) and, for segments, the flag-tuple operator of
// src/Futhark/Pass/Flatten/Builtins.hs:374-393.  How it is computed is native
// to CDNA4:
//   * blocks stay on their CU and take tiles by ticket; tiles travel from HBM
//     straight into LDS two rounds ahead (global_load_lds_dwordx4);
//   * a thread scans 128 consecutive bytes one element after the other, so a
//     wave needs one DPP scan per tile; the LDS layout that makes this possible
//     costs no barrier, because every wave keeps to its own 8 KiB;
//   * a tile descriptor is a 64-bit word {value bits, epoch, segment flag,
//     status} written and read with single relaxed agent-scope accesses, so no
//     fence separates value and status.  8-byte element types use two such
//     words (low and high half), accepted only when both carry the same status;
//   * descriptors carry a launch epoch, so no kernel clears them between calls;
//   * a wave of its own looks back, one round behind the scan and one round
//     ahead of the stores, so nobody waits for a round trip between CUs;
//   * the waves of a block do not meet at barriers: they pass wave totals,
//     prefixes and tickets through small rings in LDS with progress counters,
//     so their load, compute and store phases drift apart and the CU's memory
//     pipeline always has work.
#include <stdlib.h>

#include <mutex>

#include "futhark_amd_segops.hpp"
#include "dispatch.hip.h"

namespace fa {

// How blocks pick their ticket counter: what the calling thread's tuning says.
static ScanTickets scan_tickets() {
  fa_tuning t;
  fa_get_tuning(&t);
  return t.scan_tickets_by_block ? ScanTickets::BY_BLOCK : ScanTickets::BY_ARRIVAL;
}

// ---- scratch for the entry point that allocates nothing
// The header and 256 KiB of tile descriptors (16384 tiles).
constexpr size_t SCAN_STATIC_BYTES = SCAN_HEADER_BYTES + 256 * 1024;
constexpr int SCAN_STATIC_EPOCH_WORD = 16;  // 32-bit word of the header that holds the epoch

}  // namespace fa

// Look-back scratch of fa_segscan_static: ticket counter, epoch word and tile
// descriptors.  Every GPU the library runs on holds its own copy, zero at
// load time, until the process ends.
static __device__ __align__(256) unsigned char static_scratch[fa::SCAN_STATIC_BYTES];

namespace fa {

// Advances the epoch word; before it would wrap, clears the descriptors.  One block.
__global__ __launch_bounds__(256) void scan_static_epoch_kernel(uint32_t *header, uint64_t *desc,
                                                                int words) {
  const uint32_t next = header[SCAN_STATIC_EPOCH_WORD] + 1u;
  const bool wrap = next >= (1u << 28);
  if (wrap)
    for (int i = threadIdx.x; i < words; i += blockDim.x) desc[i] = 0ull;
  __syncthreads();
  if (threadIdx.x == 0) header[SCAN_STATIC_EPOCH_WORD] = wrap ? 1u : next;
}

// Device address of `static_scratch` on the current device (in host code the array's
// name is only a handle for this query).
static int scan_static_scratch(void **out) {
  constexpr int MAX_DEVICES = 64;
  static std::mutex mu;
  static void *ptrs[MAX_DEVICES];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return FA_EINVAL;
  std::lock_guard<std::mutex> guard(mu);
  if (ptrs[dev] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return FA_EINVAL;
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return 0;
}

template <class T, class Op>
static int launch_scan_static(hipStream_t s, const void *xs, const uint8_t *flags, int64_t n,
                              int exclusive, void *out, void *base) {
  uint32_t *header = (uint32_t *)base;
  uint64_t *desc = (uint64_t *)((char *)base + SCAN_HEADER_BYTES);
  hipLaunchKernelGGL(scan_static_epoch_kernel, dim3(1), dim3(256), 0, s, header, desc,
                     (int)((SCAN_STATIC_BYTES - SCAN_HEADER_BYTES) / 8));
  const int rc = launch_status();
  if (rc != 0) return rc;
  return launch_scan<T, Op>(s, xs, flags, (int64_t)0, n, exclusive, out, base, SCAN_STATIC_BYTES, 1u,
                            header + SCAN_STATIC_EPOCH_WORD, scan_tickets());
}

}  // namespace fa

extern "C" int64_t fa_segscan_static_max_n(fa_dtype t) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  const int64_t tile = (es == 4) ? ss_tile_elems<int32_t>() : ss_tile_elems<int64_t>();
  return (int64_t)((SCAN_STATIC_BYTES - SCAN_HEADER_BYTES) / SCAN_DESC_BYTES) * tile;
}

extern "C" int fa_segscan_static_init(void) {
  void *base = nullptr;
  return scan_static_scratch(&base);
}

extern "C" int fa_segscan_static(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                                 const uint8_t *flags, int64_t n, int exclusive, void *out) {
  if (n < 0 || (n > 0 && (xs == nullptr || out == nullptr))) return FA_EINVAL;
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return FA_ENOTSUP;
  if (n > fa_segscan_static_max_n(t)) return FA_ESCRATCH;  // beyond what the fixed scratch holds
  if (n == 0) return 0;
  void *base = nullptr;
  const int rc = scan_static_scratch(&base);
  if (rc != 0) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE
               ? launch_scan_static<AffineI32, OpCompose>(s, xs, flags, n, exclusive, out, base)
               : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan_static, t, op, s, xs, flags, n, exclusive, out, base);
}

extern "C" int64_t fa_segscan_tile_elems(fa_dtype t) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  return (es == 4) ? ss_tile_elems<int32_t>() : ss_tile_elems<int64_t>();
}

extern "C" size_t fa_segscan_scratch_bytes(fa_dtype t, int64_t n) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  if (n < 0) n = 0;
  const int64_t tile = (es == 4) ? ss_tile_elems<int32_t>() : ss_tile_elems<int64_t>();
  const int64_t tiles = ceil_div(n, tile);
  return SCAN_HEADER_BYTES + (size_t)(tiles < 1 ? 1 : tiles) * SCAN_DESC_BYTES;
}

extern "C" int fa_segscan(fa_stream_t stream, fa_dtype t, fa_op op, const void *xs,
                          const uint8_t *flags, int64_t n, int exclusive, void *out,
                          void *scratch, size_t scratch_bytes, uint32_t epoch) {
  if (n < 0 || (n > 0 && (xs == nullptr || out == nullptr || scratch == nullptr)))
    return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE ? launch_scan<AffineI32, OpCompose>(s, xs, flags, (int64_t)0, n, exclusive,
                                                                out, scratch, scratch_bytes, epoch,
                                                                nullptr, scan_tickets())
                            : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xs, flags, (int64_t)0, n, exclusive, out, scratch,
                      scratch_bytes, epoch, (const uint32_t *)nullptr, scan_tickets());
}

extern "C" int fa_segscan_rows(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss,
                               int64_t m, int64_t k, int exclusive, void *out, void *scratch,
                               size_t scratch_bytes, uint32_t epoch) {
  if (m < 0 || k < 0 || (m > 0 && k > INT64_MAX / m)) return FA_EINVAL;
  const int64_t n = m * k;
  if (n > 0 && (xss == nullptr || out == nullptr || scratch == nullptr)) return FA_EINVAL;
  if (epoch == 0 || epoch >= (1u << 28)) return FA_EINVAL;
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (t == FA_I32X2)
    return op == FA_COMPOSE
               ? launch_scan<AffineI32, OpCompose>(s, xss, (const uint8_t *)nullptr, k, n, exclusive,
                                                   out, scratch, scratch_bytes, epoch, nullptr,
                                                   scan_tickets())
               : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xss, (const uint8_t *)nullptr, k, n, exclusive, out,
                      scratch, scratch_bytes, epoch, (const uint32_t *)nullptr, scan_tickets());
}
