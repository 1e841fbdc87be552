// Scan with a vector operator, scan (map2 op) (replicate k ne) xss for
// xss : [n][k]T: column j of the result is the scan of column j.
//
// The reference gives such a SegScan to its two-pass code (the single-pass
// kernel takes scalar operators only, SegScan/SinglePass.hs canBeSinglePass;
// SegScan/TwoPass.hs).  Here, for rows that are whole 1 KiB strips (k * sizeof T
// a multiple of 1024), three launches in the reduce-then-scan manner, every
// access to HBM a coalesced 16-byte one and no transposed copy:
//   1. the rows are cut into C chunks; a wave folds one strip of one chunk
//      (a lane owns the same 16 bytes of every row) into partial[c][k];
//   2. per strip, one block turns partial[0..C)[strip] into exclusive
//      prefixes over the chunks (16 waves take a run of chunks each, fold it,
//      exchange the 16 totals through LDS, and walk the run again);
//   3. a wave walks its strip of its chunk again, from the chunk's prefix, and
//      writes the running value (streaming stores).
// The input is read twice and the output written once: 1.5 x the algorithmic
// bytes, against 3 x for transpose, scan of rows, transpose, which remains the
// path for every other shape.  All operators of the library commute, so the
// partial folds may take the rows in any grouping; the order of the operands
// of every combination is kept anyway.
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
  const int64_t col = s * (VS_STRIP_BYTES / (int)sizeof(T)) + lane_id() * VEC;
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  T acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) acc[e] = Op::identity();
  const T *p = xss + r0 * k + col;
  int64_t r = r0;
  for (; r + VS_UNROLL <= r1; r += VS_UNROLL, p += VS_UNROLL * k) {
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) v[u] = load_vec16_nt(p + u * k);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++)
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v[u].e[e]);
  }
  for (; r < r1; r++, p += k) {
    const Vec16<T> v = load_vec16_nt(p);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[e] = Op::apply(acc[e], v.e[e]);
  }
  Vec16<T> o;
#pragma unroll
  for (int e = 0; e < VEC; e++) o.e[e] = acc[e];
  store_vec16(partial + c * k + col, o);
}

// partial[c][strip] := fold of partial[0..c)[strip], one block per strip.
template <class T, class Op>
__global__ __launch_bounds__(VS_OFFSET_BLOCK) void vs_offsets_kernel(T *__restrict__ partial,
                                                                     int64_t chunks, int64_t k) {
  constexpr int VEC = Vec16<T>::N;
  constexpr int WAVES = VS_OFFSET_BLOCK / WAVE;
  __shared__ __align__(16) T totals[WAVES][WAVE * VEC];
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int64_t col = (int64_t)blockIdx.x * (VS_STRIP_BYTES / (int)sizeof(T)) + lane * VEC;
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
      store_vec16(partial + (c + u) * k + col, o);
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
    store_vec16(q, o);
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
  const int64_t col = s * (VS_STRIP_BYTES / (int)sizeof(T)) + lane_id() * VEC;
  const int64_t r0 = c * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < n ? r0 + rows_per_chunk : n;
  T run[VEC];
  {
    const Vec16<T> v = load_vec16(prefix + c * k + col);
#pragma unroll
    for (int e = 0; e < VEC; e++) run[e] = v.e[e];
  }
  const T *p = xss + r0 * k + col;
  T *q = out + r0 * k + col;
  int64_t r = r0;
  for (; r + VS_UNROLL <= r1; r += VS_UNROLL, p += VS_UNROLL * k, q += VS_UNROLL * k) {
    Vec16<T> v[VS_UNROLL];
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) v[u] = load_vec16_nt(p + u * k);
#pragma unroll
    for (int u = 0; u < VS_UNROLL; u++) {
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < VEC; e++) o.e[e] = run[e] = Op::apply(run[e], v[u].e[e]);
      store_vec16_nt(q + u * k, o);
    }
  }
  for (; r < r1; r++, p += k, q += k) {
    const Vec16<T> v = load_vec16_nt(p);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < VEC; e++) o.e[e] = run[e] = Op::apply(run[e], v.e[e]);
    store_vec16_nt(q, o);
  }
}

struct VsPlan {
  int64_t strips, chunks, rows_per_chunk;
};

// Chunks: VS_WANT_TASKS tasks (strips x chunks), at least 16 rows each.
static VsPlan vs_plan(size_t es, int64_t n, int64_t k) {
  VsPlan p = {0, 0, 0};
  if (n < 1 || k < 1 || ((size_t)k * es) % VS_STRIP_BYTES != 0) return p;
  p.strips = (int64_t)((size_t)k * es / VS_STRIP_BYTES);
  int64_t want = ceil_div((int64_t)VS_WANT_TASKS, p.strips);
  if (want > VS_MAX_CHUNKS) want = VS_MAX_CHUNKS;
  if (want > n / 16) want = n / 16;
  if (want < 1) want = 1;
  p.rows_per_chunk = ceil_div(n, want);
  p.chunks = ceil_div(n, p.rows_per_chunk);
  return p;
}

template <class T, class Op>
static int launch_vecscan(hipStream_t st, const void *xss, int64_t n, int64_t k, void *out,
                          void *workspace) {
  const VsPlan p = vs_plan(sizeof(T), n, k);
  const int64_t tasks = p.strips * p.chunks;
  const dim3 grid((unsigned)ceil_div(tasks, (int64_t)(VS_BLOCK / WAVE)));
  T *partial = (T *)workspace;
  hipLaunchKernelGGL((vs_partial_kernel<T, Op>), grid, dim3(VS_BLOCK), 0, st, (const T *)xss, n, k,
                     p.rows_per_chunk, p.strips, tasks, partial);
  int rc = launch_status();
  if (rc != 0) return rc;
  hipLaunchKernelGGL((vs_offsets_kernel<T, Op>), dim3((unsigned)p.strips), dim3(VS_OFFSET_BLOCK), 0,
                     st, partial, p.chunks, k);
  if ((rc = launch_status()) != 0) return rc;
  hipLaunchKernelGGL((vs_scan_kernel<T, Op>), grid, dim3(VS_BLOCK), 0, st, (const T *)xss, n, k,
                     p.rows_per_chunk, p.strips, tasks, (const T *)partial, (T *)out);
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
