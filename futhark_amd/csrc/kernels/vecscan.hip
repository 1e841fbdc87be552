// Scan with a vector operator, scan (map2 op) (replicate k ne) xss for
// xss : [n][k]T: column j of the result is the scan of column j.
//
// The reference gives such a SegScan to its two-pass code (the single-pass
// kernel takes scalar operators only, SegScan/SinglePass.hs canBeSinglePass;
// SegScan/TwoPass.hs).  Here, for rows that are whole 16-byte units, every
// access to HBM is a coalesced 16-byte one and no transposed copy is made:
//   * other rows of 256 bytes and more: a lane owns the same 16 bytes of every row,
//     a wave a strip of 1 KiB of columns (the lanes of the last strip that lie
//     beyond the row idle);
//   * rows of 16, 32, ... 512 bytes: a wave-wide load covers 1024 / row-bytes
//     rows, the lanes that own the same columns in different rows are scanned
//     across the wave with lane shifts, and the carry travels in registers.
// The rows are cut into C chunks so that strips x chunks tasks fill the chip:
//   1. a wave folds its strip of one chunk into partial[c][k];
//   2. one block per strip turns partial[0..C)[strip] into exclusive prefixes
//      over the chunks;
//   3. a wave walks its strip of its chunk again, from the chunk's prefix, and
//      writes the running value (streaming stores).
// With enough strips to fill the chip by themselves (1024 and more) there is
// one chunk, steps 1 and 2 are skipped, and the input is read once.  Otherwise
// it is read twice, but not twice from HBM: the memory-side cache (256 MiB)
// still holds what step 1 read last, so step 1 walks every chunk from its last
// row to its first, step 3 starts where step 1 ended, and both load with the
// default policy (non-temporal loads leave nothing behind).  [65536][1024] f32:
// 143 us with non-temporal loads and both steps walking forwards, 132 us with
// plain loads in step 1, 127 us with step 1 backwards, 122 us with plain loads
// in step 3 too; plain stores in step 3: 161 us.  A look-back chain along the
// rows instead of the first two steps would need one descriptor per column and
// tile, and a tile would find hundreds of its predecessors still without a
// prefix (all of the chip works on the few strips of the same rows): reading
// their aggregates costs more than reading the chunk again.
// Rows that are not whole 16-byte units, and short rows whose byte count is no
// power of two, go through transpose, scan of rows, transpose (3 x).
// All operators of the library commute, so the partial folds may take the rows
// in any grouping; the order of the operands of every combination is kept anyway.
#include "dispatch.hip.h"

namespace fa {

constexpr int VS_BLOCK = 256;        // four waves, each with a task of its own
constexpr int VS_STRIP_BYTES = 1024; // one wave-wide 16-byte load
constexpr int VS_UNROLL = 8;         // rows in flight per wave (16: no faster)
// Tasks (strips x chunks) wanted: with 4096 the prefixes over 1024 chunks take
// 37 us of 170 ([65536][1024] f32); 2048: 155 us; 1024: 145 us; 768: 159 us; 512: 198 us.
constexpr int VS_WANT_TASKS = 1024;
constexpr int VS_OFFSET_BLOCK = 1024;
constexpr int VS_MAX_CHUNKS = 1024;

template <class T, class Op>
__global__ __launch_bounds__(VS_BLOCK) void vs_partial_kernel(const T *__restrict__ xss, int64_t n,
                                                              int64_t k, int64_t rows_per_chunk,
                                                              int64_t strips, int64_t tasks,
                                                              T *__restrict__ partial) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t task = (int64_t)blockIdx.x * (VS_BLOCK / WAVE) + threadIdx.x / WAVE;
  if (task >= tasks) return;
  const int64_t c = task / strips, s = task % strips;
  // Lanes of the last strip beyond the end of the row load what lane 0 of the
  // strip loads (loads are unconditional) and store nothing.
  const int64_t own = s * (VS_STRIP_BYTES / (int)sizeof(T)) + lane_id() * VEC;
  const bool active = own < k;
  const int64_t col = active ? own : s * (VS_STRIP_BYTES / (int)sizeof(T));
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  // Last rows first: what the next kernel reads first is what was read last.
  const T *p = xss + r1 * k + col;
  int64_t r = r1;
  for (; r - VS_UNROLL >= r0; r -= VS_UNROLL) {
    p -= VS_UNROLL * k;
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) v[u] = load_vec16(p + (VS_UNROLL - 1 - u) * k);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(v[u].e[e], acc[e]);
  }
  for (; r > r0; r--) {
    p -= k;
    const Vec16<T> v = load_vec16(p);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = Op::apply(v.e[e], acc[e]);
  }
  Vec16<T> o;
#pragma unroll
  for (int e = 0; e < VEC; e++) o.e[e] = acc[e];
  if (active) store_vec16(partial + c * k + col, o);
}

// partial[c][strip] := fold of partial[0..c)[strip], one block per strip.
template <class T, class Op>
__global__ __launch_bounds__(VS_OFFSET_BLOCK) void vs_offsets_kernel(T *__restrict__ partial,
                                                                     int64_t chunks, int64_t k) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int WAVES = VS_OFFSET_BLOCK / WAVE;
  __shared__ __align__(16) T totals[WAVES][WAVE * VEC];
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int64_t own = (int64_t)blockIdx.x * (VS_STRIP_BYTES / (int)sizeof(T)) + lane * VEC;
  const bool active = own < k;
  const int64_t col = active ? own : (int64_t)blockIdx.x * (VS_STRIP_BYTES / (int)sizeof(T));
  const int64_t per = ceil_div(chunks, (int64_t)WAVES);
  const int64_t c0 = wave * per < chunks ? wave * per : chunks;
  const int64_t c1 = c0 + per < chunks ? c0 + per : chunks;
  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  constexpr int U = 8;  // loads in flight
  int64_t c = c0;
  for (; c + U <= c1; c += U) {
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = load_vec16(partial + (c + u) * k + col);
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
  }
  for (; c < c1; c++) {
    const Vec16<T> v = load_vec16(partial + c * k + col);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v.e[e]);
  }
#pragma unroll
  for (int e = 0; e < VEC; e++) totals[wave][lane * VEC + e] = acc[e];
  __syncthreads();
  T run[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) run[e] = Op::identity();
  for (int w = 0; w < wave; w++)
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = Op::apply(run[e], totals[w][lane * VEC + e]);
  c = c0;
  for (; c + U <= c1; c += U) {
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = load_vec16(partial + (c + u) * k + col);
#pragma unroll
    for (int u = 0; u < U; u++) {
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        o.e[e] = run[e];
        run[e] = Op::apply(run[e], v[u].e[e]);
      }
      if (active) store_vec16(partial + (c + u) * k + col, o);
    }
  }
  for (; c < c1; c++) {
    T *q = partial + c * k + col;
    const Vec16<T> v = load_vec16(q);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      o.e[e] = run[e];
      run[e] = Op::apply(run[e], v.e[e]);
    }
    if (active) store_vec16(q, o);
  }
}

template <class T, class Op>
__global__ __launch_bounds__(VS_BLOCK) void vs_scan_kernel(const T *__restrict__ xss, int64_t n,
                                                           int64_t k, int64_t rows_per_chunk,
                                                           int64_t strips, int64_t tasks,
                                                           const T *__restrict__ prefix,
                                                           T *__restrict__ out) {
  constexpr int VEC = Vec16<T>::N;
  const int64_t task = (int64_t)blockIdx.x * (VS_BLOCK / WAVE) + threadIdx.x / WAVE;
  if (task >= tasks) return;
  const int64_t c = task / strips, s = task % strips;
  const int64_t own = s * (VS_STRIP_BYTES / (int)sizeof(T)) + lane_id() * VEC;
  const bool active = own < k;
  const int64_t col = active ? own : s * (VS_STRIP_BYTES / (int)sizeof(T));
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  T run[VEC];
  if (prefix != nullptr) {  // (no prefixes: the one chunk starts from the neutral element)
    const Vec16<T> v = load_vec16(prefix + c * k + col);
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = v.e[e];
  } else {
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = Op::identity();
  }
  const T *p = xss + r0 * k + col;
  T *q = out + r0 * k + col;
  int64_t r = r0;
  for (; r + VS_UNROLL <= r1; r += VS_UNROLL, p += VS_UNROLL * k, q += VS_UNROLL * k) {
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) v[u] = load_vec16(p + u * k);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) {
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < VEC; e++) o.e[e] = run[e] = Op::apply(run[e], v[u].e[e]);
      if (active) store_vec16_nt(q + u * k, o);
    }
  }
  for (; r < r1; r++, p += k, q += k) {
    const Vec16<T> v = load_vec16(p);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < VEC; e++) o.e[e] = run[e] = Op::apply(run[e], v.e[e]);
    if (active) store_vec16_nt(q, o);
  }
}

// ---------------------------------------------------------------- narrow rows
// Rows of RB = 16 ... 512 bytes (a power of two).  A wave-wide load of 1 KiB is
// G = 1024 / RB consecutive rows: lane l holds 16 bytes of row l / LPR, columns
// (l % LPR) * VEC ..., with LPR = RB / 16 lanes per row.
template <class T> __device__ __forceinline__ T vs_shift_up(T v, int d) {
  if constexpr (sizeof(T) == 4) {
    return bit_cast<T>(__shfl_up(bit_cast<int>(v), d, WAVE));
  } else {
    return bit_cast<T>((unsigned long long)__shfl_up((unsigned long long)bit_cast<uint64_t>(v), d, WAVE));
  }
}
template <class T> __device__ __forceinline__ T vs_from_lane(T v, int src) {
  if constexpr (sizeof(T) == 4) {
    return bit_cast<T>(__shfl(bit_cast<int>(v), src, WAVE));
  } else {
    return bit_cast<T>((unsigned long long)__shfl((unsigned long long)bit_cast<uint64_t>(v), src, WAVE));
  }
}

// Inclusive scan over the G rows of one wave-wide load, for every column: lanes
// LPR apart hold the same columns of consecutive rows.  One row per lane is the
// wave scan; 2, 4 or 8 lanes per row scan inside each group of 16 lanes with
// DPP row shifts (a shift by d lanes that leaves the 16 lanes yields the
// neutral element, which is what the first d / LPR rows of the group need) and
// then pull in what the groups of 16 before hold, as the wave scan does with
// its two broadcasts, with two lane reads; 16 and 32 lanes per row are four and
// two rows, one or two shifts.
template <class T, class Op, int LPR> __device__ __forceinline__ T vs_rows_scan(T x, int lane) {
  if constexpr (LPR == 1) {
    return wave_incl_scan<T, Op>(x);
  } else if constexpr (LPR < 16) {
    const T id = Op::identity();
    if constexpr (LPR <= 2) x = Op::apply(dpp_move<DPP_ROW_SHR2, 0xf>(id, x), x);
    if constexpr (LPR <= 4) x = Op::apply(dpp_move<DPP_ROW_SHR4, 0xf>(id, x), x);
    if constexpr (LPR <= 8) x = Op::apply(dpp_move<DPP_ROW_SHR8, 0xf>(id, x), x);
    const int col = lane % LPR, group = lane >> 4;
    // groups 1 and 3 take the last row of the group before them, then groups 2
    // and 3 the last row of group 1 (which by then holds groups 0 and 1)
    T t = vs_from_lane(x, ((lane & 48) - LPR + col) & 63);
    if (group & 1) x = Op::apply(t, x);
    t = vs_from_lane(x, 32 - LPR + col);
    if (group >= 2) x = Op::apply(t, x);
    return x;
  } else {
#pragma unroll
    for (int d = LPR; d < WAVE; d *= 2) {
      const T other = vs_shift_up(x, d);
      if (lane >= d) x = Op::apply(other, x);
    }
    return x;
  }
}

// partial[c][k]: the fold of the rows of chunk c, one wave per chunk.
template <class T, class Op, int LPR>
__global__ __launch_bounds__(VS_BLOCK) void vs_partial_narrow_kernel(const T *__restrict__ xss,
                                                                     int64_t n, int64_t rows_per_chunk,
                                                                     int64_t chunks,
                                                                     T *__restrict__ partial) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int G = WAVE / LPR;     // rows per wave-wide load
  constexpr int K = LPR * VEC;      // elements per row
  const int64_t c = (int64_t)blockIdx.x * (VS_BLOCK / WAVE) + threadIdx.x / WAVE;
  if (c >= chunks) return;
  const int lane = lane_id();
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  // Lane l takes rows r0 + l / LPR, + G, + 2 G, ...
  // The end of the chunk first, as in vs_partial_kernel.
  constexpr int64_t STEP = (int64_t)VS_UNROLL * G;
  const int64_t full = (r1 - r0) / STEP;
  for (int64_t r = r0 + full * STEP; r < r1; r += G) {
    const bool have = r + lane / LPR < r1;
    const Vec16<T> v = load_vec16(xss + (have ? r * K + lane * VEC : r0 * K));
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], have ? v.e[e] : Op::identity());
  }
  for (int64_t g = full - 1; g >= 0; g--) {
    const int64_t r = r0 + g * STEP;
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++)
      v[u] = load_vec16(xss + (r + (VS_UNROLL - 1 - u) * G) * K + lane * VEC);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
  }
  // Fold the G lanes that own the same columns; the result ends up in the lanes
  // of the last row.  (The order of the rows inside a lane and across lanes is
  // interleaved, which operators that commute allow; all of the library's do.)
#pragma unroll
  for (int d = LPR; d < WAVE; d *= 2)
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      const T other = vs_shift_up(acc[e], d);
      if (lane >= d) acc[e] = Op::apply(other, acc[e]);
    }
  if (lane >= WAVE - LPR) {
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < VEC; e++) o.e[e] = acc[e];
    store_vec16(partial + c * K + (lane - (WAVE - LPR)) * VEC, o);
  }
}

// partial[c][j] := fold of partial[0..c)[j]: a thread per chunk (there are at
// most VS_MAX_CHUNKS = 1024), a block scan per column, VS_NARROW_COLS columns
// per block.  (One thread per column walking the chunks one after the other
// waits out a load latency per chunk: 100 us for 1024 chunks.)
constexpr int VS_NARROW_COLS = 4;
template <class T, class Op>
__global__ __launch_bounds__(VS_MAX_CHUNKS) void vs_offsets_narrow_kernel(T *__restrict__ partial,
                                                                          int64_t chunks, int k) {
  __shared__ T totals[VS_NARROW_COLS][VS_MAX_CHUNKS / WAVE];
  const int c = threadIdx.x, wave = c / WAVE, lane = lane_id();
  const int j0 = blockIdx.x * VS_NARROW_COLS;
  T excl[VS_NARROW_COLS];
#pragma unroll
  for (int q = 0; q < VS_NARROW_COLS; q++) {
    const int j = j0 + q;
    const T v = c < chunks && j < k ? partial[(int64_t)c * k + j] : Op::identity();
    const T incl = wave_incl_scan<T, Op>(v);
    excl[q] = wave_shift_up1<T, Op>(incl);
    if (lane == WAVE - 1) totals[q][wave] = incl;
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < VS_NARROW_COLS; q++) {
    const int j = j0 + q;
    T base = Op::identity();
    for (int w = 0; w < wave; w++) base = Op::apply(base, totals[q][w]);
    if (c < chunks && j < k) partial[(int64_t)c * k + j] = Op::apply(base, excl[q]);
  }
}

template <class T, class Op, int LPR>
__global__ __launch_bounds__(VS_BLOCK) void vs_scan_narrow_kernel(const T *__restrict__ xss, int64_t n,
                                                                  int64_t rows_per_chunk,
                                                                  int64_t chunks,
                                                                  const T *__restrict__ prefix,
                                                                  T *__restrict__ out) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int G = WAVE / LPR;
  constexpr int K = LPR * VEC;
  const int64_t c = (int64_t)blockIdx.x * (VS_BLOCK / WAVE) + threadIdx.x / WAVE;
  if (c >= chunks) return;
  const int lane = lane_id();
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  // What precedes the rows of the current load, for this lane's columns.
  T run[VEC];
  if (prefix != nullptr) {
    const Vec16<T> v = load_vec16(prefix + c * K + (lane % LPR) * VEC);
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = v.e[e];
  } else {
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = Op::identity();
  }
  auto step = [&](Vec16<T> v, int64_t r) {
    const bool have = r + lane / LPR < r1;
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      // inclusive scan over the rows of the load, earlier rows on the left
      T x = vs_rows_scan<T, Op, LPR>(have ? v.e[e] : Op::identity(), lane);
      x = Op::apply(run[e], x);
      o.e[e] = x;
      // what precedes the next load: the last row of this one
      if constexpr (LPR == 1) run[e] = read_lane(x, WAVE - 1);
      else run[e] = vs_from_lane(x, WAVE - LPR + lane % LPR);
    }
    if (have) store_vec16_nt(out + r * K + lane * VEC, o);
  };
  int64_t r = r0;
  for (; r + (int64_t)VS_UNROLL * G <= r1; r += (int64_t)VS_UNROLL * G) {
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) v[u] = load_vec16(xss + (r + u * G) * K + lane * VEC);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) step(v[u], r + u * G);
  }
  for (; r < r1; r += G) {
    const bool have = r + lane / LPR < r1;
    step(load_vec16(xss + (have ? r * K + lane * VEC : r0 * K)), r);
  }
}

struct VsPlan {
  int64_t strips, chunks, rows_per_chunk;
  int lanes_per_row;  // 0: strips; else narrow rows with this many lanes each
};

constexpr int VS_MIN_STRIP_ROW_BYTES = 256;  // shorter rows leave most lanes of a strip idle

// Chunks: VS_WANT_TASKS tasks (strips x chunks), at least 16 rows (16 wave-wide
// loads of narrow rows) each.  chunks == 0: no plan for this shape.
static VsPlan vs_plan(size_t es, int64_t n, int64_t k) {
  VsPlan p = {0, 0, 0, 0};
  if (n < 1 || k < 1 || (size_t)k > SIZE_MAX / es) return p;
  const size_t rb = (size_t)k * es;
  if (rb % 16 != 0) return p;
  int64_t unit_rows = 1;  // rows come in units of this many
  if (rb < (size_t)VS_STRIP_BYTES && (rb & (rb - 1)) == 0) {
    p.strips = 1;
    p.lanes_per_row = (int)(rb / 16);
    unit_rows = WAVE / p.lanes_per_row;
  } else if (rb >= (size_t)VS_MIN_STRIP_ROW_BYTES) {
    p.strips = (int64_t)ceil_div((int64_t)rb, (int64_t)VS_STRIP_BYTES);
  } else {
    return p;
  }
  int64_t want = ceil_div((int64_t)VS_WANT_TASKS, p.strips);
  if (want > VS_MAX_CHUNKS) want = VS_MAX_CHUNKS;
  if (want > n / (16 * unit_rows)) want = n / (16 * unit_rows);
  if (want < 1) want = 1;
  p.rows_per_chunk = ceil_div(ceil_div(n, want), unit_rows) * unit_rows;
  p.chunks = ceil_div(n, p.rows_per_chunk);
  return p;
}

template <class T, class Op, int LPR>
static int launch_vecscan_narrow(hipStream_t st, const VsPlan &p, const T *xss, int64_t n, T *out,
                                 T *partial) {
  const dim3 grid((unsigned)ceil_div(p.chunks, (int64_t)(VS_BLOCK / WAVE)));
  int rc = 0;
  if (p.chunks > 1) {
    hipLaunchKernelGGL((vs_partial_narrow_kernel<T, Op, LPR>), grid, dim3(VS_BLOCK), 0, st, xss, n,
                       p.rows_per_chunk, p.chunks, partial);
    if ((rc = launch_status()) != 0) return rc;
    constexpr int K = LPR * Vec16<T>::N;
    hipLaunchKernelGGL((vs_offsets_narrow_kernel<T, Op>), dim3((K + VS_NARROW_COLS - 1) / VS_NARROW_COLS),
                       dim3(VS_MAX_CHUNKS), 0, st, partial, p.chunks, K);
    if ((rc = launch_status()) != 0) return rc;
  }
  hipLaunchKernelGGL((vs_scan_narrow_kernel<T, Op, LPR>), grid, dim3(VS_BLOCK), 0, st, xss, n,
                     p.rows_per_chunk, p.chunks, p.chunks > 1 ? (const T *)partial : (const T *)nullptr,
                     out);
  return launch_status();
}

template <class T, class Op>
static int launch_vecscan(hipStream_t st, const void *xss, int64_t n, int64_t k, void *out,
                          void *workspace) {
  const VsPlan p = vs_plan(sizeof(T), n, k);
  T *partial = (T *)workspace;
  switch (p.lanes_per_row) {
    case 0: break;
    case 1: return launch_vecscan_narrow<T, Op, 1>(st, p, (const T *)xss, n, (T *)out, partial);
    case 2: return launch_vecscan_narrow<T, Op, 2>(st, p, (const T *)xss, n, (T *)out, partial);
    case 4: return launch_vecscan_narrow<T, Op, 4>(st, p, (const T *)xss, n, (T *)out, partial);
    case 8: return launch_vecscan_narrow<T, Op, 8>(st, p, (const T *)xss, n, (T *)out, partial);
    case 16: return launch_vecscan_narrow<T, Op, 16>(st, p, (const T *)xss, n, (T *)out, partial);
    case 32: return launch_vecscan_narrow<T, Op, 32>(st, p, (const T *)xss, n, (T *)out, partial);
    default: return FA_EINVAL;
  }
  const int64_t tasks = p.strips * p.chunks;
  const dim3 grid((unsigned)ceil_div(tasks, (int64_t)(VS_BLOCK / WAVE)));
  int rc = 0;
  if (p.chunks > 1) {
    hipLaunchKernelGGL((vs_partial_kernel<T, Op>), grid, dim3(VS_BLOCK), 0, st, (const T *)xss, n, k,
                       p.rows_per_chunk, p.strips, tasks, partial);
    if ((rc = launch_status()) != 0) return rc;
    hipLaunchKernelGGL((vs_offsets_kernel<T, Op>), dim3((unsigned)p.strips), dim3(VS_OFFSET_BLOCK), 0,
                       st, partial, p.chunks, k);
    if ((rc = launch_status()) != 0) return rc;
  }
  hipLaunchKernelGGL((vs_scan_kernel<T, Op>), grid, dim3(VS_BLOCK), 0, st, (const T *)xss, n, k,
                     p.rows_per_chunk, p.strips, tasks,
                     p.chunks > 1 ? (const T *)partial : (const T *)nullptr, (T *)out);
  return launch_status();
}

}  // namespace fa

extern "C" size_t fa_vecscan_workspace_bytes(fa_dtype t, int64_t n, int64_t k) {
  const size_t es = dtype_size(t);
  if (es != 4 && es != 8) return 0;
  const VsPlan p = vs_plan(es, n, k);
  if (p.chunks == 0 || p.strips > 65535 * 16) return 0;
  return (size_t)p.chunks * (size_t)k * es;
}

extern "C" int fa_vecscan(fa_stream_t stream, fa_dtype t, fa_op op, const void *xss, int64_t n,
                          int64_t k, void *out, void *workspace, size_t workspace_bytes) {
  if (n < 0 || k < 0) return FA_EINVAL;
  if (n == 0 || k == 0) return 0;
  const size_t need = fa_vecscan_workspace_bytes(t, n, k);
  if (need == 0) return FA_ENOTSUP;  // the caller transposes and scans rows instead
  if (xss == nullptr || out == nullptr || workspace == nullptr) return FA_EINVAL;
  if (workspace_bytes < need) return FA_ESCRATCH;
  if (!is_aligned(xss, 16) || !is_aligned(out, 16) || !is_aligned(workspace, 16)) return FA_EALIGN;
  hipStream_t st = (hipStream_t)stream;
  FA_DISPATCH_TYPE_OP(launch_vecscan, t, op, st, xss, n, k, out, workspace);
}
