// SegScan for gfx950: single-pass scan with decoupled look-back.
//
// What is computed follows src/Futhark/CodeGen/ImpGen/GPU/SegScan/SinglePass.hs
// (dynamic tile ids :443-461, tile aggregate/prefix publication with status
// X/A/P :128-131,625-777) and, for segments, the flag-tuple operator of
// src/Futhark/Pass/Flatten/Builtins.hs:374-393.  How it is computed is native
// to CDNA4:
//   * every wave owns a contiguous chunk; each load/store instruction of a wave
//     covers 1 KiB of consecutive bytes (128 bits per lane), so no LDS
//     transpose is needed to coalesce;
//   * scans inside a wave use DPP row shifts and broadcasts over all 64 lanes;
//   * a tile descriptor is a 64-bit word {value bits, epoch, segment flag,
//     status} written and read with single relaxed agent-scope accesses, so no
//     fence separates value and status.  8-byte element types use two such
//     words (low and high half), accepted only when both carry the same status;
//   * descriptors carry a launch epoch, so no kernel clears them between calls;
//   * the look-back window is a full 64-lane wave with several descriptors per
//     lane.
#include <mutex>

#include "dispatch.hip.h"

namespace fa {

// Tile shape.  Every tile costs one atomic on the shared ticket counter, and
// same-address device atomics complete at roughly one per 12 ns on MI355X, so
// tiles are made large (16 waves x 8 rows x 16 bytes x 64 lanes = 128 KiB of
// 4-byte elements) to keep the ticket rate far below that limit.
#ifndef FA_SCAN_ROWS4
#define FA_SCAN_ROWS4 8 /* 4-byte elements: 32 per thread */
#endif
#ifndef FA_SCAN_ROWS8
#define FA_SCAN_ROWS8 8 /* 8-byte elements: 16 per thread */
#endif
#ifndef FA_SCAN_WAVES
#define FA_SCAN_WAVES 16
#endif
// 8-byte elements: 16 per thread need more than the 128 registers a thread of a
// 1024-thread block may have (8 per thread in such a block: 296 us for a
// segmented i64 scan of 2^26 elements; 16 per thread there spill: 326 us), so
// these scans run in 512-thread blocks, two to a CU, with tiles of 64 KiB:
// 237 us.
#ifndef FA_SCAN_WAVES8
#define FA_SCAN_WAVES8 8
#endif
// Cache policy, measured: plain data loads, non-temporal flag loads and
// non-temporal stores give the best rate (a copy kernel gains 25 % from
// non-temporal stores alone).
#ifndef FA_SCAN_LOAD
#define FA_SCAN_LOAD load_vec16
#endif
#ifndef FA_SCAN_FLAG_LOAD
#define FA_SCAN_FLAG_LOAD __builtin_nontemporal_load
#endif
#ifndef FA_SCAN_STORE
#define FA_SCAN_STORE store_vec16_nt
#endif
template <class T> constexpr int scan_rows() { return sizeof(T) == 4 ? FA_SCAN_ROWS4 : FA_SCAN_ROWS8; }
template <class T> constexpr int scan_waves() { return sizeof(T) == 4 ? FA_SCAN_WAVES : FA_SCAN_WAVES8; }
template <class T> constexpr int scan_block() { return scan_waves<T>() * WAVE; }

// Descriptors per lane in a look-back window.  Measured on 2^26 f32: 1 -> 99 us,
// 2 -> 103 us, 4 -> 109 us; the nearest published prefix is normally within 64
// tiles, and a wider window only adds loads to the round trip.
constexpr int SCAN_LB = 1;

constexpr uint32_t ST_X = 0;  // nothing published
constexpr uint32_t ST_A = 1;  // aggregate of the tile
constexpr uint32_t ST_P = 2;  // inclusive prefix up to the end of the tile

constexpr size_t SCAN_HEADER_BYTES = 256;  // ticket counter, padded
constexpr size_t SCAN_DESC_BYTES = 16;     // per tile

template <class T> constexpr int scan_tile_elems() {
  return scan_block<T>() * scan_rows<T>() * Vec16<T>::N;
}

__device__ __forceinline__ uint32_t desc_meta(uint32_t epoch, uint32_t flag, uint32_t status) {
  return (epoch << 3) | ((flag & 1u) << 2) | status;
}

template <class T>
__device__ __forceinline__ void desc_publish(uint64_t *desc, int64_t tile, uint32_t epoch,
                                             uint32_t status, uint32_t flag, T v) {
  const uint32_t meta = desc_meta(epoch, flag, status);
  if constexpr (sizeof(T) == 4) {
    st_relaxed_u64(desc + 2 * tile, ((uint64_t)bit_cast<uint32_t>(v) << 32) | meta);
  } else {
    const uint64_t b = bit_cast<uint64_t>(v);
    st_relaxed_u64(desc + 2 * tile, ((b & 0xffffffffull) << 32) | meta);
    st_relaxed_u64(desc + 2 * tile + 1, ((b >> 32) << 32) | meta);
  }
}

// Returns false while the tile has published nothing (for this epoch), or
// while the two halves of an 8-byte value belong to different publications.
template <class T>
__device__ __forceinline__ bool desc_read(const uint64_t *desc, int64_t tile, uint32_t epoch,
                                          uint32_t &status, uint32_t &flag, T &v) {
  const uint64_t w0 = ld_relaxed_u64(desc + 2 * tile);
  const uint32_t m0 = (uint32_t)w0;
  if ((m0 >> 3) != epoch || (m0 & 3u) == ST_X) return false;
  if constexpr (sizeof(T) == 4) {
    v = bit_cast<T>((uint32_t)(w0 >> 32));
  } else {
    const uint64_t w1 = ld_relaxed_u64(desc + 2 * tile + 1);
    if ((uint32_t)w1 != m0) return false;
    v = bit_cast<T>((w0 >> 32) | ((w1 >> 32) << 32));
  }
  status = m0 & 3u;
  flag = (m0 >> 2) & 1u;
  return true;
}

// Segment starts among the VEC elements that begin at position `pos` of a row
// of `seg_len` elements: bit e is set when element e opens a row.
template <int VEC>
__device__ __forceinline__ uint32_t regular_start_mask(int64_t pos, int64_t seg_len) {
  uint32_t m = 0u;
#pragma unroll
  for (int e = 0; e < VEC; e++) {
    if (pos == 0) m |= 1u << e;
    pos++;
    if (pos == seg_len) pos = 0;
  }
  return m;
}

// Where segments come from: nowhere, a flag byte per element, or rows of equal
// length (`map (scan op ne) xss`: SegScan with segment dimensions,
// SegScan/SinglePass.hs:327-361 -- the reference tests whether two positions
// lie in the same row; here the row starts are computed from the element
// index, so there is no flag array to read).
enum { SEG_NONE = 0, SEG_FLAGS = 1, SEG_ROWS = 2 };

// out[n]; EXCL selects the exclusive form.
template <class T, class Op, int SEGKIND, bool EXCL>
__global__ __launch_bounds__(scan_block<T>()) void segscan_kernel(
    const T *__restrict__ xs, const uint8_t *__restrict__ flags, int64_t n, T *__restrict__ out,
    uint32_t *ticket, uint64_t *desc, uint32_t epoch, const uint32_t *epoch_dev, int64_t num_tiles,
    int64_t seg_len) {
  // The epoch of this launch: an argument, or (for callers whose launches may
  // be replayed with the same arguments) a word a preceding kernel advanced.
  if (epoch_dev != nullptr) epoch = *epoch_dev;
  constexpr bool SEG = SEGKIND != SEG_NONE;
  constexpr bool FLAGS = SEGKIND == SEG_FLAGS;
  constexpr int VEC = Vec16<T>::N;
  constexpr int SCAN_ROWS = scan_rows<T>();
  constexpr int WCHUNK = SCAN_ROWS * WAVE * VEC;
  constexpr int SCAN_WAVES = scan_waves<T>();
  constexpr int TILE = SCAN_WAVES * WCHUNK;
  using Pair = SegPair<T>;

  __shared__ int64_t s_tile;
  __shared__ T s_wv[SCAN_WAVES];
  __shared__ uint32_t s_wf[SCAN_WAVES];
  __shared__ T s_pv;
  __shared__ uint32_t s_pf;
  // Flag bytes of the tile, one contiguous chunk per wave (segmented scans).
  __shared__ __align__(16) uint32_t s_flags[FLAGS ? TILE / 4 : 4];

  if (threadIdx.x == 0) {
    const uint32_t t = atomicAdd(ticket, 1u);
    s_tile = (int64_t)t;
    // The last ticket of this launch has been drawn: rearm for the next one.
    if ((int64_t)t == num_tiles - 1) st_relaxed_u32(ticket, 0u);
  }
  __syncthreads();
  // Tile and wave numbers are the same in all lanes; say so to the compiler.
  const int64_t tile = (int64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)s_tile);
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / WAVE));
  const int64_t t0 = tile * TILE;
  const int64_t wbase = t0 + (int64_t)wave * WCHUNK;

  // ---- flags: a wave's chunk has WCHUNK consecutive flag bytes.  They are
  //      fetched with 16 bytes per lane (a few wide loads instead of one narrow
  //      load per row) and handed to the lanes that own them through LDS.
  bool flags_staged = false;
  if constexpr (FLAGS) {
    constexpr int FB = WCHUNK / WAVE;  // flag bytes per lane
    static_assert(FB == 8 || FB % 16 == 0, "flag bytes per lane: one 8-byte or whole 16-byte loads");
    flags_staged = wbase + WCHUNK <= n && ((uintptr_t)flags & 15u) == 0;
    if (flags_staged) {
      unsigned char *wf = reinterpret_cast<unsigned char *>(s_flags) + wave * WCHUNK;
      const uint8_t *src = flags + wbase;
      if constexpr (FB == 8) {
        using V2 = __attribute__((ext_vector_type(2))) uint32_t;
        *reinterpret_cast<V2 *>(wf + lane * 8) =
            __builtin_nontemporal_load(reinterpret_cast<const V2 *>(src + lane * 8));
      } else {
        using V4 = __attribute__((ext_vector_type(4))) uint32_t;
#pragma unroll
        for (int j = 0; j < FB / 16; j++)
          *reinterpret_cast<V4 *>(wf + j * (WAVE * 16) + lane * 16) = __builtin_nontemporal_load(
              reinterpret_cast<const V4 *>(src + j * (WAVE * 16) + lane * 16));
      }
    }
  }

  // ---- load: row r of a wave is 64 lanes x 16 bytes of consecutive memory.
  T x[SCAN_ROWS][VEC];
  uint32_t fm[SCAN_ROWS];
#pragma unroll
  for (int r = 0; r < SCAN_ROWS; r++) {
    const int64_t idx = wbase + (int64_t)(r * WAVE + lane) * VEC;
    fm[r] = 0u;
    if (idx + VEC <= n) {
      Vec16<T> v = FA_SCAN_LOAD(xs + idx);
#pragma unroll
      for (int e = 0; e < VEC; e++) x[r][e] = v.e[e];
      if constexpr (FLAGS) {
        if (!flags_staged) {
          if constexpr (VEC == 4) {
            const uint32_t w = FA_SCAN_FLAG_LOAD(reinterpret_cast<const uint32_t *>(flags + idx));
#pragma unroll
            for (int e = 0; e < 4; e++) fm[r] |= ((w >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
          } else {
            const uint32_t w = FA_SCAN_FLAG_LOAD(reinterpret_cast<const uint16_t *>(flags + idx));
#pragma unroll
            for (int e = 0; e < 2; e++) fm[r] |= ((w >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
          }
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        const bool in = idx + e < n;
        x[r][e] = in ? xs[idx + e] : Op::identity();
        if constexpr (FLAGS) {
          if (in && flags[idx + e] != 0) fm[r] |= 1u << e;
        }
      }
    }
  }
  if constexpr (FLAGS) {
    if (flags_staged) {
      // Same wave wrote the chunk: LDS operations of a wave complete in order.
      __builtin_amdgcn_wave_barrier();
      const unsigned char *wf = reinterpret_cast<const unsigned char *>(s_flags) + wave * WCHUNK;
#pragma unroll
      for (int r = 0; r < SCAN_ROWS; r++) {
        uint32_t w;
        if constexpr (VEC == 4) w = *reinterpret_cast<const uint32_t *>(wf + (r * WAVE + lane) * 4);
        else w = *reinterpret_cast<const uint16_t *>(wf + (r * WAVE + lane) * 2);
#pragma unroll
        for (int e = 0; e < VEC; e++) fm[r] |= ((w >> (8 * e)) & 0xffu) ? (1u << e) : 0u;
      }
    }
  }

  // Rows of equal length: the start masks come from the position of this
  // lane's first element inside its row, kept up from one 16-byte row of the
  // wave to the next (one division per thread), while the loads are in flight.
  if constexpr (SEGKIND == SEG_ROWS) {
    int64_t row_pos = (wbase + (int64_t)lane * VEC) % seg_len;
#pragma unroll
    for (int r = 0; r < SCAN_ROWS; r++) {
      fm[r] = regular_start_mask<VEC>(row_pos, seg_len);
      if (seg_len > WAVE * VEC) {
        row_pos += WAVE * VEC;
        if (row_pos >= seg_len) row_pos -= seg_len;
      } else {
        row_pos = (int64_t)((uint32_t)(row_pos + WAVE * VEC) % (uint32_t)seg_len);
      }
    }
  }

  // ---- scan inside each thread's VEC consecutive elements.
#pragma unroll
  for (int r = 0; r < SCAN_ROWS; r++) {
#pragma unroll
    for (int e = 1; e < VEC; e++) {
      if constexpr (SEG) {
        x[r][e] = ((fm[r] >> e) & 1u) ? x[r][e] : Op::apply(x[r][e - 1], x[r][e]);
      } else {
        x[r][e] = Op::apply(x[r][e - 1], x[r][e]);
      }
    }
  }

  // ---- scan across lanes per row, then chain the rows of the wave.
  Pair pre[SCAN_ROWS];  // what precedes this lane's elements inside the wave
  Pair carry = {Op::identity(), 0u};
#pragma unroll
  for (int r = 0; r < SCAN_ROWS; r++) {
    Pair incl, excl;
    if constexpr (SEG) {
      Pair tot = {x[r][VEC - 1], fm[r] ? 1u : 0u};
      incl = wave_incl_scan_seg<T, Op>(tot);
      excl.v = wave_shift_up1<T, Op>(incl.v);
      excl.f = dpp_move<DPP_WAVE_SHR1, 0xf>(0u, incl.f);
      pre[r] = seg_apply<T, Op>(carry, excl);
      Pair rowtot = {read_lane(incl.v, 63), read_lane(incl.f, 63)};
      carry = seg_apply<T, Op>(carry, rowtot);
    } else {
      incl.v = wave_incl_scan<T, Op>(x[r][VEC - 1]);
      excl.v = wave_shift_up1<T, Op>(incl.v);
      pre[r].v = Op::apply(carry.v, excl.v);
      pre[r].f = 0u;
      carry.v = Op::apply(carry.v, read_lane(incl.v, 63));
    }
  }
  if (lane == 63) {
    s_wv[wave] = carry.v;
    s_wf[wave] = carry.f;
  }
  __syncthreads();

  Pair wp = {Op::identity(), 0u};  // what precedes this wave inside the tile
  Pair bt = {Op::identity(), 0u};  // tile aggregate
#pragma unroll
  for (int w = 0; w < SCAN_WAVES; w++) {
    if (w == wave) wp = bt;
    Pair t = {s_wv[w], SEG ? s_wf[w] : 0u};
    if constexpr (SEG) bt = seg_apply<T, Op>(bt, t);
    else bt.v = Op::apply(bt.v, t.v);
  }

  // ---- writing a row: what precedes the wave (`b`, which includes the tile's
  //      prefix once that is known) and what precedes the lane inside the wave.
  auto emit_row = [&](int r, const Pair &b) {
    T pv;
    if constexpr (SEG) pv = seg_apply<T, Op>(b, pre[r]).v;
    else pv = Op::apply(b.v, pre[r].v);

    Vec16<T> o;
    uint32_t seen = 0u;
    T prev = pv;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      const uint32_t fbit = SEG ? ((fm[r] >> e) & 1u) : 0u;
      seen |= fbit;
      const T incl = (SEG && seen) ? x[r][e] : Op::apply(pv, x[r][e]);
      if constexpr (EXCL) o.e[e] = fbit ? Op::identity() : prev;
      else o.e[e] = incl;
      prev = incl;
    }

    const int64_t idx = wbase + (int64_t)(r * WAVE + lane) * VEC;
    if (idx + VEC <= n) {
      FA_SCAN_STORE(out + idx, o);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++)
        if (idx + e < n) out[idx + e] = o.e[e];
    }
  };

  // In a segmented scan everything after the first segment start of the tile
  // is independent of what precedes the tile.  Scans of rows (4-byte elements)
  // write those rows at once, while wave 0 looks back, so that the round trip
  // of the look-back is covered by the tile's own stores; only the rows before
  // the first start wait for the prefix.  Wave 0 itself looks back first (its
  // descriptor loads would otherwise queue behind its stores) and writes all
  // its rows afterwards.  Measured on 2^26 f32: rows of 4 to 2^20 elements
  // 109-112 -> 102-108 us.  The same order made the flag-driven scan slower
  // (117 -> 125 us) and 8-byte rows too (264 -> 292 us), so they keep the
  // plain order: look back, then write.
  constexpr bool EARLY = SEGKIND == SEG_ROWS && sizeof(T) == 4;
  const bool early = EARLY && bt.f != 0u && wave != 0;
  if constexpr (EARLY) {
    if (early) {
#pragma unroll
      for (int r = 0; r < SCAN_ROWS; r++)
        if ((wp.f | pre[r].f) != 0u) emit_row(r, wp);
    }
  }

  // ---- publish the aggregate, look back for the exclusive prefix of the tile.
  if (wave == 0) {
    Pair acc = {Op::identity(), 0u};
    if (tile == 0) {
      if (lane == 0) desc_publish<T>(desc, tile, epoch, ST_P, bt.f, bt.v);
    } else {
      // A tile that contains a segment start already knows its inclusive
      // prefix: nothing before the start can reach past it.
      const bool self_contained = SEG && bt.f;
      if (lane == 0)
        desc_publish<T>(desc, tile, epoch, self_contained ? ST_P : ST_A, bt.f, bt.v);
      // The window is SCAN_LB descriptors per lane, 64 * SCAN_LB tiles.
      int64_t j = tile - 1;  // newest tile of the window
      while (true) {
        const int64_t first_idx = j - (int64_t)(WAVE * SCAN_LB - 1) + (int64_t)lane * SCAN_LB;
        // Fold this lane's descriptors in tile order; one with a published
        // prefix (or, in a segmented scan, a segment start) restarts the fold.
        // All descriptors of the lane are requested before any is examined, so
        // a window costs one round trip however many the lane holds.
        uint32_t st[SCAN_LB], fl[SCAN_LB];
        T v[SCAN_LB];
        bool ok[SCAN_LB];
#pragma unroll
        for (int k = 0; k < SCAN_LB; k++) {
          st[k] = ST_P;
          fl[k] = 0u;
          v[k] = Op::identity();
          ok[k] = first_idx + k < 0 || desc_read<T>(desc, first_idx + k, epoch, st[k], fl[k], v[k]);
        }
#pragma unroll
        for (int k = 0; k < SCAN_LB; k++) {
          while (!ok[k]) {
            __builtin_amdgcn_s_sleep(1);
            ok[k] = desc_read<T>(desc, first_idx + k, epoch, st[k], fl[k], v[k]);
          }
        }
        Pair part = {Op::identity(), 0u};
        bool term = false;
#pragma unroll
        for (int k = 0; k < SCAN_LB; k++) {
          const Pair e = {v[k], SEG ? fl[k] : 0u};
          if (st[k] == ST_P) {
            part = e;
          } else {
            if constexpr (SEG) part = seg_apply<T, Op>(part, e);
            else part.v = Op::apply(part.v, v[k]);
          }
          term = term || (st[k] == ST_P) || (SEG && fl[k]);
        }
        const uint64_t mask = __ballot(term);
        Pair mine = part;
        if (mask) {
          const int first = 63 - __builtin_clzll(mask);
          if (lane < first) {
            mine.v = Op::identity();
            mine.f = 0u;
          }
        }
        Pair win;
        if constexpr (SEG) {
          Pair sc = wave_incl_scan_seg<T, Op>(mine);
          win.v = read_lane(sc.v, 63);
          win.f = read_lane(sc.f, 63);
          acc = seg_apply<T, Op>(win, acc);
        } else {
          win.v = read_lane(wave_incl_scan<T, Op>(mine.v), 63);
          acc.v = Op::apply(win.v, acc.v);
        }
        if (mask) break;
        j -= WAVE * SCAN_LB;
      }
      if (lane == 0 && !self_contained) {
        Pair inc;
        if constexpr (SEG) inc = seg_apply<T, Op>(acc, bt);
        else { inc.v = Op::apply(acc.v, bt.v); inc.f = 0u; }
        desc_publish<T>(desc, tile, epoch, ST_P, inc.f, inc.v);
      }
    }
    if (lane == 0) {
      s_pv = acc.v;
      s_pf = acc.f;
    }
  }
  __syncthreads();

  Pair base = {s_pv, SEG ? s_pf : 0u};
  if constexpr (SEG) base = seg_apply<T, Op>(base, wp);
  else base.v = Op::apply(base.v, wp.v);

  // ---- apply the prefix and write what has not been written yet.
#pragma unroll
  for (int r = 0; r < SCAN_ROWS; r++) {
    if (EARLY && early && (wp.f | pre[r].f) != 0u) continue;
    emit_row(r, base);
  }
}

template <class T> static int64_t scan_num_tiles(int64_t n) {
  return ceil_div(n, (int64_t)scan_tile_elems<T>());
}

template <class T, class Op>
static int launch_scan(hipStream_t s, const void *xs, const uint8_t *flags, int64_t seg_len,
                       int64_t n, int exclusive, void *out, void *scratch, size_t scratch_bytes,
                       uint32_t epoch, const uint32_t *epoch_dev = nullptr) {
  if (n == 0) return 0;
  const int64_t tiles = scan_num_tiles<T>(n);
  if (scratch_bytes < SCAN_HEADER_BYTES + (size_t)tiles * SCAN_DESC_BYTES) return FA_ESCRATCH;
  if (!is_aligned(xs, 16) || !is_aligned(out, 16) || !is_aligned(scratch, 16) ||
      (flags && !is_aligned(flags, 4)))
    return FA_EALIGN;
  if (tiles > INT32_MAX) return FA_EINVAL;
  uint32_t *ticket = (uint32_t *)scratch;
  uint64_t *desc = (uint64_t *)((char *)scratch + SCAN_HEADER_BYTES);
  const dim3 grid((unsigned)tiles), block(scan_block<T>());
#define FA_LAUNCH(SEGV, EXV)                                                              \
  hipLaunchKernelGGL((segscan_kernel<T, Op, SEGV, EXV>), grid, block, 0, s, (const T *)xs, \
                     flags, n, (T *)out, ticket, desc, epoch, epoch_dev, tiles, seg_len)
  if (seg_len > 0) {
    if (exclusive) FA_LAUNCH(SEG_ROWS, true);
    else FA_LAUNCH(SEG_ROWS, false);
  } else if (flags) {
    if (exclusive) FA_LAUNCH(SEG_FLAGS, true);
    else FA_LAUNCH(SEG_FLAGS, false);
  } else {
    if (exclusive) FA_LAUNCH(SEG_NONE, true);
    else FA_LAUNCH(SEG_NONE, false);
  }
#undef FA_LAUNCH
  return launch_status();
}

// ---- scratch for the entry point that allocates nothing
constexpr size_t SCAN_STATIC_BYTES = 256 * 1024;
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
                            header + SCAN_STATIC_EPOCH_WORD);
}

}  // namespace fa

extern "C" int64_t fa_segscan_static_max_n(fa_dtype t) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  const int64_t tile = (es == 4) ? scan_tile_elems<int32_t>() : scan_tile_elems<int64_t>();
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

extern "C" size_t fa_segscan_scratch_bytes(fa_dtype t, int64_t n) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  if (n < 0) n = 0;
  const int64_t tile = (es == 4) ? scan_tile_elems<int32_t>() : scan_tile_elems<int64_t>();
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
                                                                out, scratch, scratch_bytes, epoch)
                            : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xs, flags, (int64_t)0, n, exclusive, out, scratch,
                      scratch_bytes, epoch);
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
                                                   out, scratch, scratch_bytes, epoch)
               : FA_ENOTSUP;
  FA_DISPATCH_TYPE_OP(launch_scan, t, op, s, xss, (const uint8_t *)nullptr, k, n, exclusive, out,
                      scratch, scratch_bytes, epoch);
}
