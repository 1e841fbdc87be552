// Irregular segmented reduction for gfx950.
//
// What is computed follows genSegRed of the reference
// (src/Futhark/Pass/Flatten/Builtins.hs:582-602): a segmented scan of the
// values under the flag-tuple operator (:374-393), of which only the element
// at the end of every segment is kept (`ne` for an empty segment).  The
// reference materialises the whole scan; here nothing of it reaches memory, and
// no block waits for another one:
//   1. segred_bounds_kernel finds, for every tile boundary, the first segment
//      that starts at or after it and the first that ends after it (every
//      segment marks the boundaries it owns; segments are in order);
//   2. segred_tiles_kernel scans every 32 KiB tile on its own (start flags from
//      `offsets` as an LDS bitmap, DPP wave scans, scanned tile kept in LDS),
//      writes the result of every segment that lies inside the tile, and leaves
//      three words per tile: the value at the end of the segment that entered
//      the tile from the left (head), the scan value at the tile's last
//      element (tail: since the last start in the tile, or the whole tile's
//      total if nothing starts in it) and whether anything starts in it;
//   3. segred_fixup_kernel finishes the segments that cross tile boundaries:
//      one wave per tile with a head walks left over the tails, 64 tiles per
//      step, up to the tile in which the segment starts.
// Tiles are small and independent, so four blocks share a CU and their memory
// latencies (bounds, offsets, lens: one round trip each) hide one another.
#include "dispatch.hip.h"

namespace fa {

constexpr int SRI_BLOCK = 256;
constexpr int SRI_WAVES = SRI_BLOCK / WAVE;
// 16-byte loads per thread.  Measured on 2^26 elements, 4 against 8: f32
// 52.7 -> 51.6 us, i64 121.6 -> 103.8 us (and 100.2 us with non-temporal loads,
// which do nothing for f32); 2 is slower for both.
constexpr int SRI_ROWS = 8;

template <class T> constexpr int sri_tile_elems() { return SRI_BLOCK * SRI_ROWS * Vec16<T>::N; }

// Per-tile records left by the tile kernel for the fix-up kernel.
struct SriTileRec {
  uint64_t head_val;  // value bits (low bytes) at the end of the entering segment
  int64_t head_seg;   // its index, or -1 if no segment enters from the left and ends here
  uint64_t tail_val;  // scan value at the last element of the tile
  uint64_t has_start;  // nonzero if a segment starts in the tile
};

// bounds[2t]   = first segment with offsets[i] >= p_t,
// bounds[2t+1] = first segment with offsets[i] + lens[i] > p_t (0 for t == 0, so
//                that empty segments at position 0 belong to tile 0; m for the
//                last boundary),
// for p_t = min(t * tile_elems, n), t = 0..num_tiles.
//
// Computed from the segments' side: thread i (0..m, m standing for a sentinel
// segment at infinity) owns the boundaries between its predecessor's start
// (end) and its own, and writes its index there.  Starts and ends are
// non-decreasing, so every boundary has exactly one owner.  A segment that
// spans many tiles hands its boundaries to the whole wave.
__device__ __forceinline__ void sri_mark(int64_t *bounds, int which, int64_t t_lo, int64_t t_hi,
                                         int64_t value, int lane) {
  const int64_t count = t_hi - t_lo + 1;
  if (count > 0 && count <= 4) {
    for (int64_t t = t_lo; t <= t_hi; t++) bounds[2 * t + which] = value;
  }
  uint64_t wide = __ballot(count > 4);
  while (wide) {
    const int src = __builtin_ctzll(wide);
    wide &= wide - 1;
    const int64_t lo = read_lane(t_lo, src), hi = read_lane(t_hi, src);
    const int64_t v = read_lane(value, src);
    for (int64_t t = lo + lane; t <= hi; t += WAVE) bounds[2 * t + which] = v;
  }
}

static __global__ __launch_bounds__(256) void segred_bounds_kernel(
    const int64_t *__restrict__ offsets, const int64_t *__restrict__ lens, int64_t m, int64_t n,
    int64_t tile_elems, int64_t num_tiles, int64_t *__restrict__ bounds, int32_t *failure,
    int32_t code) {
  const int lane = lane_id();
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = i <= m;  // whole waves stay in the loops of sri_mark
  const int64_t inf = INT64_MAX / 2;
  int64_t s_prev = -1, s_here = inf, e_prev = 0, e_here = inf;
  if (live) {
    if (i > 0) {
      s_prev = offsets[i - 1];
      e_prev = s_prev + lens[i - 1];
    }
    if (i < m) {
      s_here = offsets[i];
      const int64_t l = lens[i];
      e_here = s_here + l;
      // What the kernels require of segment i (and of its place after segment
      // i - 1), checked while its numbers are here anyway.
      if (failure != nullptr) {
        const bool ok = s_here >= 0 && l >= 0 && s_here <= n && l <= n - s_here &&
                        (i == 0 || e_prev <= s_here);
        if (!ok) *failure = code;
      }
    }
  }
  // Interior boundaries are t = 0..num_tiles-1 at p_t = t * tile_elems.
  // Starts: s_prev < p_t <= s_here.
  {
    const int64_t t_lo = s_prev < 0 ? 0 : s_prev / tile_elems + 1;
    int64_t t_hi = s_here / tile_elems;
    if (t_hi > num_tiles - 1) t_hi = num_tiles - 1;
    sri_mark(bounds, 0, live ? t_lo : 1, live ? t_hi : 0, i, lane);
    if (live && s_prev < n && n <= s_here) bounds[2 * num_tiles] = i;  // p = n
  }
  // Ends: e_prev <= p_t < e_here, t >= 1.
  {
    int64_t t_lo = (e_prev + tile_elems - 1) / tile_elems;
    if (t_lo < 1) t_lo = 1;
    int64_t t_hi = e_here >= 1 ? (e_here - 1) / tile_elems : -1;
    if (t_hi > num_tiles - 1) t_hi = num_tiles - 1;
    sri_mark(bounds, 1, live ? t_lo : 1, live ? t_hi : 0, i, lane);
    if (i == 0) {
      bounds[1] = 0;
      bounds[2 * num_tiles + 1] = m;
    }
  }
}

template <class T> __device__ __forceinline__ uint64_t sri_bits(T v) {
  if constexpr (sizeof(T) == 4) return (uint64_t)bit_cast<uint32_t>(v);
  else return bit_cast<uint64_t>(v);
}
template <class T> __device__ __forceinline__ T sri_value(uint64_t b) {
  if constexpr (sizeof(T) == 4) return bit_cast<T>((uint32_t)b);
  else return bit_cast<T>(b);
}

template <class T, class Op>
__global__ __launch_bounds__(SRI_BLOCK) void segred_tiles_kernel(
    const T *__restrict__ vs, int64_t n, const int64_t *__restrict__ offsets,
    const int64_t *__restrict__ lens, const int64_t *__restrict__ bounds, T *__restrict__ out,
    SriTileRec *__restrict__ recs) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int WCHUNK = SRI_ROWS * WAVE * VEC;
  constexpr int TILE = SRI_WAVES * WCHUNK;
  using Pair = SegPair<T>;

  __shared__ int64_t s_bounds[4];
  __shared__ uint32_t s_bits[TILE / 32];
  __shared__ T s_wv[SRI_WAVES];
  __shared__ uint32_t s_wf[SRI_WAVES];
  __shared__ __align__(16) T s_vals[TILE];

  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int64_t tile = blockIdx.x;
  const int64_t t0 = tile * TILE;
  const int tile_n = (int)(n - t0 < TILE ? n - t0 : TILE);
  const int64_t wbase = t0 + (int64_t)wave * WCHUNK;

  // Segment ranges of the tile first (a short dependent chain), then the data.
  if (tid < 4) s_bounds[tid] = bounds[2 * tile + (tid & 1) * 2 + (tid >> 1)];
  for (int i = tid; i < TILE / 32; i += SRI_BLOCK) s_bits[i] = 0u;

  T x[SRI_ROWS][VEC];
#pragma unroll
  for (int r = 0; r < SRI_ROWS; r++) {
    const int64_t idx = wbase + (int64_t)(r * WAVE + lane) * VEC;
    if (idx + VEC <= n) {
      const Vec16<T> v = sizeof(T) == 8 ? load_vec16_nt(vs + idx) : load_vec16(vs + idx);
#pragma unroll
      for (int e = 0; e < VEC; e++) x[r][e] = v.e[e];
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++) x[r][e] = idx + e < n ? vs[idx + e] : Op::identity();
    }
  }
  __syncthreads();
  const int64_t s_first = s_bounds[0], s_last = s_bounds[1];  // segments starting in the tile
  const int64_t e_first = s_bounds[2], e_last = s_bounds[3];  // segments ending in the tile

  // Requested now, used after the scan.
  int64_t pre_len = 0, pre_off = 0;
  if (e_first + tid < e_last) {
    pre_len = lens[e_first + tid];
    pre_off = offsets[e_first + tid];
  }
  for (int64_t i = s_first + tid; i < s_last; i += SRI_BLOCK) {
    const int64_t p = offsets[i] - t0;
    if ((uint64_t)p < (uint64_t)TILE) atomicOr(&s_bits[p >> 5], 1u << (p & 31));
  }
  __syncthreads();

  // ---- segmented scan of the tile, starting afresh at its first element.
  uint32_t fm[SRI_ROWS];
#pragma unroll
  for (int r = 0; r < SRI_ROWS; r++) {
    const int p = wave * WCHUNK + (r * WAVE + lane) * VEC;
    fm[r] = (s_bits[p >> 5] >> (p & 31)) & ((1u << VEC) - 1u);
#pragma unroll
    for (int e = 1; e < VEC; e++)
      x[r][e] = ((fm[r] >> e) & 1u) ? x[r][e] : Op::apply(x[r][e - 1], x[r][e]);
  }
  Pair pre[SRI_ROWS];
  Pair carry = {Op::identity(), 0u};
#pragma unroll
  for (int r = 0; r < SRI_ROWS; r++) {
    const Pair tot = {x[r][VEC - 1], fm[r] ? 1u : 0u};
    const Pair incl = wave_incl_scan_seg<T, Op>(tot);
    Pair excl;
    excl.v = wave_shift_up1<T, Op>(incl.v);
    excl.f = dpp_move<DPP_WAVE_SHR1, 0xf>(0u, incl.f);
    pre[r] = seg_apply<T, Op>(carry, excl);
    const Pair rowtot = {read_lane(incl.v, 63), read_lane(incl.f, 63)};
    carry = seg_apply<T, Op>(carry, rowtot);
  }
  if (lane == 63) {
    s_wv[wave] = carry.v;
    s_wf[wave] = carry.f;
  }
  __syncthreads();
  Pair wp = {Op::identity(), 0u};
#pragma unroll
  for (int w = 0; w < SRI_WAVES; w++) {
    if (w < wave) wp = seg_apply<T, Op>(wp, Pair{s_wv[w], s_wf[w]});
  }
#pragma unroll
  for (int r = 0; r < SRI_ROWS; r++) {
    const T pv = seg_apply<T, Op>(wp, pre[r]).v;
    const int p = wave * WCHUNK + (r * WAVE + lane) * VEC;
    Vec16<T> o;
    uint32_t seen = 0u;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      seen |= (fm[r] >> e) & 1u;
      o.e[e] = seen ? x[r][e] : Op::apply(pv, x[r][e]);
    }
    *reinterpret_cast<uint4 *>(&s_vals[p]) = bit_cast<uint4>(o);
  }
  __syncthreads();

  // ---- results of the segments that end in the tile.
  bool have_head = false;
  for (int64_t i = e_first + tid; i < e_last; i += SRI_BLOCK) {
    const bool first_round = i < e_first + SRI_BLOCK;
    const int64_t len = first_round ? pre_len : lens[i];
    const int64_t off = first_round ? pre_off : offsets[i];
    if (len == 0) {
      out[i] = Op::identity();
      continue;
    }
    const int64_t p = off + len - 1 - t0;
    const T v = (uint64_t)p < (uint64_t)TILE ? s_vals[p] : Op::identity();
    if (i >= s_first) {
      out[i] = v;  // starts and ends here
    } else {       // entered from the left: the fix-up kernel adds what lies before the tile
      recs[tile].head_val = sri_bits<T>(v);
      recs[tile].head_seg = i;
      have_head = true;
    }
  }
  // Segments are disjoint and in order, so at most the first segment of the
  // range (handled by thread 0) can have entered from the left.
  if (tid == 0) {
    if (!have_head) recs[tile].head_seg = -1;
    recs[tile].tail_val = sri_bits<T>(s_vals[tile_n - 1]);
    recs[tile].has_start = s_last > s_first ? 1u : 0u;
  }
}

// One wave per tile whose head segment started in an earlier tile: fold the
// tails of the tiles to its left, nearest first, up to and including the tile
// in which the segment starts.
template <class T, class Op>
__global__ __launch_bounds__(256) void segred_fixup_kernel(const SriTileRec *__restrict__ recs,
                                                           int64_t num_tiles,
                                                           T *__restrict__ out) {
  const int lane = lane_id();
  const int64_t tile = (int64_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
  if (tile >= num_tiles) return;
  const int64_t seg = recs[tile].head_seg;
  if (seg < 0) return;
  T acc = sri_value<T>(recs[tile].head_val);
  int64_t j = tile - 1;  // newest tile of the window
  while (j >= 0) {
    const int64_t u = j - (WAVE - 1) + lane;
    T v = Op::identity();
    bool start = false;
    if (u >= 0) {
      v = sri_value<T>(recs[u].tail_val);
      start = recs[u].has_start != 0;
    }
    const uint64_t mask = __ballot(start);
    if (mask) {
      const int first = 63 - __builtin_clzll(mask);
      if (lane < first) v = Op::identity();
    }
    acc = Op::apply(read_lane(wave_incl_scan<T, Op>(v), 63), acc);
    if (mask) break;
    j -= WAVE;
  }
  if (lane == 0) out[seg] = acc;
}

template <class T>
static __global__ void sri_fill_kernel(T *dst, int64_t n, T v) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

static size_t sri_scratch_bytes(int64_t tiles) {
  if (tiles < 1) tiles = 1;
  return (size_t)(tiles + 1) * 16 + (size_t)tiles * sizeof(SriTileRec);
}

template <class T, class Op>
static int launch_segred_irregular(hipStream_t s, const void *vs, int64_t n,
                                   const int64_t *offsets, const int64_t *lens, int64_t m,
                                   void *out, void *scratch, size_t scratch_bytes,
                                   int32_t *failure, int32_t code) {
  if (m == 0) return 0;
  if (n == 0) {  // every segment is empty
    int grid = (int)(ceil_div(m, 256) < 4096 ? ceil_div(m, 256) : 4096);
    hipLaunchKernelGGL((sri_fill_kernel<T>), dim3(grid), dim3(256), 0, s, (T *)out, m,
                       Op::identity());
    return launch_status();
  }
  const int64_t tile_elems = sri_tile_elems<T>();
  const int64_t tiles = ceil_div(n, tile_elems);
  if (scratch_bytes < sri_scratch_bytes(tiles)) return FA_ESCRATCH;
  if (!is_aligned(vs, 16) || !is_aligned(scratch, 16) || !is_aligned(offsets, 8) ||
      !is_aligned(lens, 8))
    return FA_EALIGN;
  if (tiles > INT32_MAX) return FA_EINVAL;
  int64_t *bounds = (int64_t *)scratch;
  SriTileRec *recs = (SriTileRec *)((char *)scratch + (size_t)(tiles + 1) * 16);
  hipLaunchKernelGGL(segred_bounds_kernel, dim3((unsigned)ceil_div(m + 1, (int64_t)256)),
                     dim3(256), 0, s, offsets, lens, m, n, tile_elems, tiles, bounds, failure, code);
  hipLaunchKernelGGL((segred_tiles_kernel<T, Op>), dim3((unsigned)tiles), dim3(SRI_BLOCK), 0, s,
                     (const T *)vs, n, offsets, lens, (const int64_t *)bounds, (T *)out, recs);
  hipLaunchKernelGGL((segred_fixup_kernel<T, Op>),
                     dim3((unsigned)ceil_div(tiles, (int64_t)(256 / WAVE))), dim3(256), 0, s,
                     (const SriTileRec *)recs, tiles, (T *)out);
  return launch_status();
}

}  // namespace fa

extern "C" size_t fa_segred_irregular_scratch_bytes(fa_dtype t, int64_t n) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  if (n < 0) n = 0;
  const int64_t tile = (es == 4) ? sri_tile_elems<int32_t>() : sri_tile_elems<int64_t>();
  return sri_scratch_bytes(ceil_div(n, tile));
}

namespace fa {
// Segments must be in order, disjoint and inside [0, n): one thread per segment
// looks at itself and its successor and raises *failure otherwise.
__global__ __launch_bounds__(256) void segments_check_kernel(const int64_t *__restrict__ offsets,
                                                             const int64_t *__restrict__ lens,
                                                             int64_t m, int64_t n, int32_t *failure,
                                                             int32_t code) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= m) return;
  const int64_t o = offsets[i], l = lens[i];
  bool ok = o >= 0 && l >= 0 && o <= n && l <= n - o;
  if (ok && i + 1 < m) ok = o + l <= offsets[i + 1];
  if (!ok) *failure = code;
}
}  // namespace fa

extern "C" int fa_segments_check(fa_stream_t stream, const int64_t *offsets, const int64_t *lens,
                                 int64_t m, int64_t n, int32_t *failure, int32_t code) {
  if (m < 0 || n < 0 || failure == nullptr || (m > 0 && (offsets == nullptr || lens == nullptr)))
    return FA_EINVAL;
  if (m == 0) return 0;
  hipLaunchKernelGGL(fa::segments_check_kernel, dim3((unsigned)ceil_div(m, (int64_t)256)), dim3(256), 0,
                     (hipStream_t)stream, offsets, lens, m, n, failure, code);
  return launch_status();
}

extern "C" int fa_segred_irregular(fa_stream_t stream, fa_dtype t, fa_op op, const void *vs,
                                   int64_t n, const int64_t *offsets, const int64_t *lens,
                                   int64_t m, void *out, void *scratch, size_t scratch_bytes) {
  if (n < 0 || m < 0 || (m > 0 && (offsets == nullptr || lens == nullptr || out == nullptr)) ||
      (n > 0 && m > 0 && (vs == nullptr || scratch == nullptr)))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_segred_irregular, t, op, s, vs, n, offsets, lens, m, out, scratch,
                      scratch_bytes, (int32_t *)nullptr, 0);
}

extern "C" int fa_segred_irregular_checked(fa_stream_t stream, fa_dtype t, fa_op op, const void *vs,
                                           int64_t n, const int64_t *offsets, const int64_t *lens,
                                           int64_t m, void *out, void *scratch,
                                           size_t scratch_bytes, int32_t *failure, int32_t code) {
  if (failure == nullptr) return FA_EINVAL;
  if (n < 0 || m < 0 || (m > 0 && (offsets == nullptr || lens == nullptr || out == nullptr)) ||
      (n > 0 && m > 0 && (vs == nullptr || scratch == nullptr)))
    return FA_EINVAL;
  hipStream_t s = (hipStream_t)stream;
  if (m > 0 && n == 0) {  // no kernel of the reduction looks at the segments then
    const int rc = fa_segments_check(stream, offsets, lens, m, n, failure, code);
    if (rc != 0) return rc;
  }
  FA_DISPATCH_TYPE_OP(launch_segred_irregular, t, op, s, vs, n, offsets, lens, m, out, scratch,
                      scratch_bytes, failure, code);
}
