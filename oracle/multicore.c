/*
 * multicore.c -- futhark-multicore-style CPU baseline (restated), pthreads.
 *
 * TEST/BENCH INFRASTRUCTURE ONLY: timed by bench.py as the reported CPU
 * baseline and cross-checked against oracle.c in tests/.  It restates the code
 * the multicore backend generates for the benchmark programs:
 *   reduce  per-task accumulators, then a sequential combine
 *           (src/Futhark/CodeGen/ImpGen/Multicore/SegRed.hs:297-320,345-376)
 *   scan    decoupled look-back over blocks sized to the cache constant, block
 *           ids handed out by an atomic counter, flags 0/1/2, with the
 *           sequential fast path when the predecessor is already final
 *           (Multicore/SegScan.hs:407-566); segmented scans arrive as the
 *           flag-tuple operator (SegScan.hs:578-582)
 *   hist    one private sub-histogram per task plus a column reduce when
 *           tasks*H <= n, otherwise atomic updates of the shared histogram
 *           (Multicore/SegHist.hs:50-71,103-151,180-320)
 *   segmented reduce over irregular segments, matmul and radix sort: the
 *           compositions stated at each function below
 * Work is split statically into one task per thread, as the scheduler does for
 * a parallel loop without nested parallelism (rts/c/scheduler.h:788-968).
 */
#define _GNU_SOURCE
#include <pthread.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <unistd.h>

int mc_num_threads(void) {
  const char *env = getenv("ORACLE_MC_THREADS");
  if (env && atoi(env) > 0) return atoi(env);
  long n = sysconf(_SC_NPROCESSORS_ONLN);
  return n > 0 ? (int)n : 1;
}

typedef void (*task_fn)(int tid, int ntasks, void *arg);
struct task_arg {
  task_fn fn;
  int tid, ntasks;
  void *arg;
};
static void *task_main(void *p) {
  struct task_arg *a = (struct task_arg *)p;
  a->fn(a->tid, a->ntasks, a->arg);
  return NULL;
}
static void par_loop(int ntasks, task_fn fn, void *arg) {
  pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)ntasks);
  struct task_arg *as = (struct task_arg *)calloc((size_t)ntasks, sizeof(struct task_arg));
  for (int t = 0; t < ntasks; t++) {
    as[t].fn = fn; as[t].tid = t; as[t].ntasks = ntasks; as[t].arg = arg;
    if (t > 0) pthread_create(&th[t], NULL, task_main, &as[t]);
  }
  task_main(&as[0]);
  for (int t = 1; t < ntasks; t++) pthread_join(th[t], NULL);
  free(th);
  free(as);
}
static void split(int64_t n, int tid, int ntasks, int64_t *lo, int64_t *hi) {
  const int64_t per = n / ntasks, rem = n % ntasks;
  *lo = tid * per + (tid < rem ? tid : rem);
  *hi = *lo + per + (tid < rem ? 1 : 0);
}

/* ------------------------------------------------------------------ reduce */
#define MC_REDUCE(S, T, COMBINE)                                                    \
  struct red_##S { const T *xs; int64_t n; T *partial; };                           \
  static void red_task_##S(int tid, int nt, void *p) {                              \
    struct red_##S *a = (struct red_##S *)p;                                        \
    int64_t lo, hi;                                                                 \
    split(a->n, tid, nt, &lo, &hi);                                                 \
    T acc = 0;                                                                      \
    for (int64_t i = lo; i < hi; i++) acc = COMBINE(acc, a->xs[i]);                 \
    a->partial[tid] = acc;                                                          \
  }                                                                                 \
  T mc_reduce_add_##S(const T *xs, int64_t n, int threads) {                        \
    T *partial = (T *)calloc((size_t)threads, sizeof(T));                           \
    struct red_##S a = {xs, n, partial};                                            \
    par_loop(threads, red_task_##S, &a);                                            \
    T acc = 0;                                                                      \
    for (int t = 0; t < threads; t++) acc = COMBINE(acc, partial[t]);               \
    free(partial);                                                                  \
    return acc;                                                                     \
  }
#define ADD_I32(a, b) ((int32_t)((uint32_t)(a) + (uint32_t)(b)))
#define ADD_I64(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define ADD_F(a, b) ((a) + (b))
MC_REDUCE(i32, int32_t, ADD_I32)
MC_REDUCE(i64, int64_t, ADD_I64)
MC_REDUCE(f32, float, ADD_F)

/* -------------------------------------------------------------------- scan
 * One generic routine over (flag, value) pairs; flags == NULL gives the plain
 * scan.  OPK: 0 add, 1 max. */
enum { MC_CACHE_BYTES = 64 * 1024 };

#define MC_SCAN(S, T, ADD, MAXF)                                                                 \
  struct scan_##S {                                                                              \
    const T *xs; const uint8_t *flags; T *out; int64_t n; int opk;                               \
    int64_t block, nblocks;                                                                      \
    _Atomic int64_t *status; T *aggr; uint8_t *aggr_f; T *pref; uint8_t *pref_f;                 \
    _Atomic int64_t work_index;                                                                  \
  };                                                                                             \
  static inline T scan_op_##S(int opk, T a, T b) { return opk == 0 ? ADD(a, b) : MAXF(a, b); }   \
  static inline T scan_ne_##S(int opk) { return opk == 0 ? (T)0 : (T)MC_LOWEST_##S; }            \
  static void scan_task_##S(int tid, int nt, void *p) {                                          \
    (void)tid; (void)nt;                                                                         \
    struct scan_##S *a = (struct scan_##S *)p;                                                   \
    int seq = 1;                                                                                 \
    T pv = scan_ne_##S(a->opk);                                                                  \
    for (int64_t b = atomic_fetch_add(&a->work_index, 1); b < a->nblocks;                        \
         b = atomic_fetch_add(&a->work_index, 1)) {                                              \
      const int64_t lo = b * a->block, hi = lo + a->block < a->n ? lo + a->block : a->n;         \
      if (seq) {                                                                                 \
        if (b == 0) pv = scan_ne_##S(a->opk);                                                    \
        else if (atomic_load_explicit(&a->status[b - 1], memory_order_acquire) == 2)             \
          pv = a->pref[b - 1];                                                                   \
        else seq = 0;                                                                            \
      }                                                                                          \
      if (seq) { /* fast path: predecessor final, scan straight through */                       \
        T acc = pv; uint8_t af = 0;                                                              \
        for (int64_t i = lo; i < hi; i++) {                                                      \
          const uint8_t f = a->flags ? a->flags[i] != 0 : 0;                                     \
          acc = f ? a->xs[i] : scan_op_##S(a->opk, acc, a->xs[i]);                               \
          af |= f;                                                                               \
          a->out[i] = acc;                                                                       \
        }                                                                                        \
        a->pref[b] = acc; a->pref_f[b] = af;                                                     \
        atomic_store_explicit(&a->status[b], 2, memory_order_release);                           \
        pv = acc;                                                                                \
      } else {                                                                                   \
        T agg = scan_ne_##S(a->opk); uint8_t af = 0;                                             \
        for (int64_t i = lo; i < hi; i++) {                                                      \
          const uint8_t f = a->flags ? a->flags[i] != 0 : 0;                                     \
          agg = f ? a->xs[i] : scan_op_##S(a->opk, agg, a->xs[i]);                               \
          af |= f;                                                                               \
        }                                                                                        \
        a->aggr[b] = agg; a->aggr_f[b] = af;                                                     \
        atomic_store_explicit(&a->status[b], 1, memory_order_release);                           \
        /* look back: fold aggregates right-to-left until a final prefix */                      \
        T acc = scan_ne_##S(a->opk); uint8_t accf = 0; int has = 0;                              \
        int64_t lb = b - 1;                                                                      \
        for (;;) {                                                                               \
          const int64_t st = atomic_load_explicit(&a->status[lb], memory_order_acquire);         \
          if (st == 0) continue;                                                                 \
          const T v = st == 2 ? a->pref[lb] : a->aggr[lb];                                       \
          const uint8_t vf = st == 2 ? a->pref_f[lb] : a->aggr_f[lb];                            \
          if (!has) { acc = v; accf = vf; has = 1; }                                             \
          else { acc = accf ? acc : scan_op_##S(a->opk, v, acc); accf |= vf; }                   \
          if (st == 2 || accf) break;                                                            \
          lb--;                                                                                  \
        }                                                                                        \
        a->pref[b] = af ? agg : scan_op_##S(a->opk, acc, agg);                                   \
        a->pref_f[b] = af | accf;                                                                \
        atomic_store_explicit(&a->status[b], 2, memory_order_release);                           \
        T run = acc;                                                                             \
        for (int64_t i = lo; i < hi; i++) {                                                      \
          const uint8_t f = a->flags ? a->flags[i] != 0 : 0;                                     \
          run = f ? a->xs[i] : scan_op_##S(a->opk, run, a->xs[i]);                               \
          a->out[i] = run;                                                                       \
        }                                                                                        \
        seq = 1; pv = run; /* next block may again find its predecessor final */                 \
        seq = 1;                                                                                 \
      }                                                                                          \
    }                                                                                            \
  }                                                                                              \
  void mc_segscan_##S(const uint8_t *flags, const T *xs, int64_t n, T *out, int opk,             \
                      int threads) {                                                             \
    if (n == 0) return;                                                                          \
    struct scan_##S a;                                                                           \
    a.xs = xs; a.flags = flags; a.out = out; a.n = n; a.opk = opk;                               \
    a.block = MC_CACHE_BYTES / (int64_t)(sizeof(T) + (flags ? 1 : 0));                           \
    a.nblocks = (n + a.block - 1) / a.block;                                                     \
    a.status = (_Atomic int64_t *)calloc((size_t)a.nblocks, sizeof(int64_t));                    \
    a.aggr = (T *)malloc(sizeof(T) * (size_t)a.nblocks);                                         \
    a.pref = (T *)malloc(sizeof(T) * (size_t)a.nblocks);                                         \
    a.aggr_f = (uint8_t *)calloc((size_t)a.nblocks, 1);                                          \
    a.pref_f = (uint8_t *)calloc((size_t)a.nblocks, 1);                                          \
    atomic_init(&a.work_index, 0);                                                               \
    par_loop(threads, scan_task_##S, &a);                                                        \
    free((void *)a.status); free(a.aggr); free(a.pref); free(a.aggr_f); free(a.pref_f);          \
  }

#define MC_LOWEST_i32 INT32_MIN
#define MC_LOWEST_i64 INT64_MIN
#define MC_LOWEST_f32 (-INFINITY)
#define MAX_INT(a, b) ((a) < (b) ? (b) : (a))
MC_SCAN(i32, int32_t, ADD_I32, MAX_INT)
MC_SCAN(i64, int64_t, ADD_I64, MAX_INT)
MC_SCAN(f32, float, ADD_F, fmaxf)

/* -------------------------------------------------------------------- hist */
struct hist_i32 {
  const int32_t *is; const int32_t *vs; int64_t n, H; int32_t *subs; int32_t *dest; int use_atomic;
};
static void hist_task_i32(int tid, int nt, void *p) {
  struct hist_i32 *a = (struct hist_i32 *)p;
  int64_t lo, hi;
  split(a->n, tid, nt, &lo, &hi);
  if (a->use_atomic) {
    for (int64_t i = lo; i < hi; i++) {
      const int64_t b = a->is[i];
      if (b >= 0 && b < a->H)
        __atomic_fetch_add(&a->dest[b], a->vs[i], __ATOMIC_RELAXED);
    }
  } else {
    int32_t *sub = a->subs + (int64_t)tid * a->H;
    for (int64_t i = lo; i < hi; i++) {
      const int64_t b = a->is[i];
      if (b >= 0 && b < a->H) sub[b] = ADD_I32(sub[b], a->vs[i]);
    }
  }
}
struct col_i32 { int32_t *subs; int32_t *dest; int64_t H; int ntasks; };
static void col_task_i32(int tid, int nt, void *p) {
  struct col_i32 *a = (struct col_i32 *)p;
  int64_t lo, hi;
  split(a->H, tid, nt, &lo, &hi);
  for (int64_t b = lo; b < hi; b++) {
    int32_t acc = a->dest[b];
    for (int t = 0; t < a->ntasks; t++) acc = ADD_I32(acc, a->subs[(int64_t)t * a->H + b]);
    a->dest[b] = acc;
  }
}
void mc_rbi_add_i32(int32_t *dest, int64_t H, const int32_t *is, const int32_t *vs, int64_t n,
                    int threads) {
  struct hist_i32 a = {is, vs, n, H, NULL, dest, 0};
  a.use_atomic = !((int64_t)threads * H <= n);
  if (!a.use_atomic) a.subs = (int32_t *)calloc((size_t)threads * (size_t)(H > 0 ? H : 1), 4);
  par_loop(threads, hist_task_i32, &a);
  if (!a.use_atomic) {
    struct col_i32 c = {a.subs, dest, H, threads};
    par_loop(threads, col_task_i32, &c);
    free(a.subs);
  }
}

/* f32 histograms: the same schedule with the float operator (sub-histograms
 * start at the neutral element; the column reduce folds them into dest). */
#define MC_HIST_F32(NAME, NE, OPF)                                                               \
  struct histf_##NAME { const int32_t *is; const float *vs; int64_t n, H; float *subs; float *dest; }; \
  static void histf_task_##NAME(int tid, int nt, void *p) {                                      \
    struct histf_##NAME *a = (struct histf_##NAME *)p;                                           \
    int64_t lo, hi;                                                                              \
    split(a->n, tid, nt, &lo, &hi);                                                              \
    float *sub = a->subs + (int64_t)tid * a->H;                                                  \
    for (int64_t b = 0; b < a->H; b++) sub[b] = (NE);                                            \
    for (int64_t i = lo; i < hi; i++) {                                                          \
      const int64_t b = a->is[i];                                                                \
      if (b >= 0 && b < a->H) sub[b] = OPF(sub[b], a->vs[i]);                                    \
    }                                                                                            \
  }                                                                                              \
  static void colf_task_##NAME(int tid, int nt, void *p) {                                       \
    struct histf_##NAME *a = (struct histf_##NAME *)p;                                           \
    int64_t lo, hi;                                                                              \
    split(a->H, tid, nt, &lo, &hi);                                                              \
    for (int64_t b = lo; b < hi; b++) {                                                          \
      float acc = a->dest[b];                                                                    \
      for (int t = 0; t < nt; t++) acc = OPF(acc, a->subs[(int64_t)t * a->H + b]);               \
      a->dest[b] = acc;                                                                          \
    }                                                                                            \
  }                                                                                              \
  void mc_rbi_##NAME##_f32(float *dest, int64_t H, const int32_t *is, const float *vs,           \
                           int64_t n, int threads) {                                             \
    struct histf_##NAME a = {is, vs, n, H, NULL, dest};                                          \
    a.subs = (float *)malloc((size_t)threads * (size_t)(H > 0 ? H : 1) * sizeof(float));         \
    par_loop(threads, histf_task_##NAME, &a);                                                    \
    par_loop(threads, colf_task_##NAME, &a);                                                     \
    free(a.subs);                                                                                \
  }
MC_HIST_F32(add, 0.0f, ADD_F)
MC_HIST_F32(max, -INFINITY, fmaxf)

/* ------------------------------------------------- irregular segmented reduce
 * What flattening makes of it (Pass/Flatten/Builtins.hs:582-602): a segmented
 * scan with flags written from the offsets, then one read per segment of the
 * scanned value at its last element (the neutral element for an empty one). */
struct gather_f32 { const int64_t *offsets, *lens; int64_t m; const float *scanned; float *out; };
static void gather_task_f32(int tid, int nt, void *p) {
  struct gather_f32 *a = (struct gather_f32 *)p;
  int64_t lo, hi;
  split(a->m, tid, nt, &lo, &hi);
  for (int64_t i = lo; i < hi; i++)
    a->out[i] = a->lens[i] == 0 ? 0.0f : a->scanned[a->offsets[i] + a->lens[i] - 1];
}
void mc_segred_add_f32(const int64_t *offsets, const int64_t *lens, int64_t m, const float *xs,
                       int64_t n, float *out, uint8_t *flags_tmp, float *scan_tmp, int threads) {
  memset(flags_tmp, 0, (size_t)n);
  for (int64_t i = 0; i < m; i++)
    if (lens[i] > 0) flags_tmp[offsets[i]] = 1;
  mc_segscan_f32(flags_tmp, xs, n, scan_tmp, 0, threads);
  struct gather_f32 g = {offsets, lens, m, scan_tmp, out};
  par_loop(threads, gather_task_f32, &g);
}

/* ------------------------------------------------------------------ matmul
 * C[b][i][j] = sum_k A[b][i][k] * B[b][k][j] as the nested map-reduce of
 * tests/reg-tiling/mmm.fut:17-21 comes out of the multicore backend: the outer
 * map over rows is the parallel loop (rows [row_lo, row_hi) of the flattened
 * b*M rows, so that a bounded sample can be timed), the inner map and the
 * reduction are sequential loops; `transpose B` is materialised once so that a
 * column is a contiguous row of the copy (Bt, b*N*K floats, caller's memory). */
struct mm_f32 { const float *A, *Bt; float *C; int64_t M, N, K, row_lo, row_hi; };
static void mm_task_f32(int tid, int nt, void *p) {
  struct mm_f32 *a = (struct mm_f32 *)p;
  int64_t lo, hi;
  split(a->row_hi - a->row_lo, tid, nt, &lo, &hi);
  for (int64_t r = a->row_lo + lo; r < a->row_lo + hi; r++) {
    const int64_t b = r / a->M;
    const float *arow = a->A + r * a->K;
    const float *bt = a->Bt + b * a->N * a->K;
    float *crow = a->C + r * a->N;
    for (int64_t j = 0; j < a->N; j++) {
      const float *bcol = bt + j * a->K;
      float acc = 0.0f;
      for (int64_t k = 0; k < a->K; k++) acc += arow[k] * bcol[k];
      crow[j] = acc;
    }
  }
}
struct tr_f32 { const float *B; float *Bt; int64_t batch, K, N; };
static void tr_task_f32(int tid, int nt, void *p) {
  struct tr_f32 *a = (struct tr_f32 *)p;
  int64_t lo, hi;
  split(a->batch * a->N, tid, nt, &lo, &hi);
  for (int64_t r = lo; r < hi; r++) {
    const int64_t b = r / a->N, j = r % a->N;
    for (int64_t k = 0; k < a->K; k++) a->Bt[r * a->K + k] = a->B[(b * a->K + k) * a->N + j];
  }
}
void mc_transpose_f32(const float *B, float *Bt, int64_t batch, int64_t K, int64_t N, int threads) {
  struct tr_f32 t = {B, Bt, batch, K, N};
  par_loop(threads, tr_task_f32, &t);
}
void mc_bmm_rows_f32(const float *A, const float *Bt, float *C, int64_t M, int64_t N, int64_t K,
                     int64_t row_lo, int64_t row_hi, int threads) {
  struct mm_f32 a = {A, Bt, C, M, N, K, row_lo, row_hi};
  par_loop(threads, mm_task_f32, &a);
}

/* The same for 16-bit inputs (f16, or bf16 when `bf16` is nonzero): A and the
 * transposed copy of B stay 16-bit in memory and every element is widened where
 * it is used, f32.f16 x * f32.f16 y summed in f32, as a program over f16 arrays
 * compiles (rts/c/half.h for the conversion; for bf16 the widening is bits << 16). */
float orc_f16_to_f32(uint16_t h);
float orc_bf16_to_f32(uint16_t h);
struct mm_16 { const uint16_t *A, *Bt; float *C; int64_t M, N, K, row_lo, row_hi; int bf16; };
static void mm_task_16(int tid, int nt, void *p) {
  struct mm_16 *a = (struct mm_16 *)p;
  int64_t lo, hi;
  split(a->row_hi - a->row_lo, tid, nt, &lo, &hi);
  for (int64_t r = a->row_lo + lo; r < a->row_lo + hi; r++) {
    const int64_t b = r / a->M;
    const uint16_t *arow = a->A + r * a->K;
    const uint16_t *bt = a->Bt + b * a->N * a->K;
    float *crow = a->C + r * a->N;
    for (int64_t j = 0; j < a->N; j++) {
      const uint16_t *bcol = bt + j * a->K;
      float acc = 0.0f;
      if (a->bf16)
        for (int64_t k = 0; k < a->K; k++) acc += orc_bf16_to_f32(arow[k]) * orc_bf16_to_f32(bcol[k]);
      else
        for (int64_t k = 0; k < a->K; k++) acc += orc_f16_to_f32(arow[k]) * orc_f16_to_f32(bcol[k]);
      crow[j] = acc;
    }
  }
}
struct tr_16 { const uint16_t *B; uint16_t *Bt; int64_t batch, K, N; };
static void tr_task_16(int tid, int nt, void *p) {
  struct tr_16 *a = (struct tr_16 *)p;
  int64_t lo, hi;
  split(a->batch * a->N, tid, nt, &lo, &hi);
  for (int64_t r = lo; r < hi; r++) {
    const int64_t b = r / a->N, j = r % a->N;
    for (int64_t k = 0; k < a->K; k++) a->Bt[r * a->K + k] = a->B[(b * a->K + k) * a->N + j];
  }
}
void mc_transpose_16(const uint16_t *B, uint16_t *Bt, int64_t batch, int64_t K, int64_t N, int threads) {
  struct tr_16 t = {B, Bt, batch, K, N};
  par_loop(threads, tr_task_16, &t);
}
void mc_bmm_rows_16(const uint16_t *A, const uint16_t *Bt, float *C, int64_t M, int64_t N, int64_t K,
                    int64_t row_lo, int64_t row_hi, int bf16, int threads) {
  struct mm_16 a = {A, Bt, C, M, N, K, row_lo, row_hi, bf16};
  par_loop(threads, mm_task_16, &a);
}

/* -------------------------------------------------------------- radix sort
 * The composition the sort is made of, per 8-bit digit from the least
 * significant one: a histogram of the digit per task, an exclusive scan of the
 * [digit][task] counts, and a scatter in which every task moves its stretch in
 * order (stable).  Keys of `kb` bytes (4 or 8) as 64-bit values; vals may be
 * NULL.  tmp buffers are the caller's (n keys, n vals). */
struct rs_arg {
  const uint64_t *k8; const uint32_t *k4; const int32_t *v;
  uint64_t *ok8; uint32_t *ok4; int32_t *ov;
  int64_t n; int shift; int64_t *counts; /* [tasks][256] */
};
static inline unsigned rs_digit(const struct rs_arg *a, int64_t i) {
  return (unsigned)(((a->k8 ? a->k8[i] : (uint64_t)a->k4[i]) >> a->shift) & 255u);
}
static void rs_count_task(int tid, int nt, void *p) {
  struct rs_arg *a = (struct rs_arg *)p;
  int64_t lo, hi;
  split(a->n, tid, nt, &lo, &hi);
  int64_t *c = a->counts + (int64_t)tid * 256;
  memset(c, 0, 256 * sizeof(int64_t));
  for (int64_t i = lo; i < hi; i++) c[rs_digit(a, i)]++;
}
static void rs_scatter_task(int tid, int nt, void *p) {
  struct rs_arg *a = (struct rs_arg *)p;
  int64_t lo, hi;
  split(a->n, tid, nt, &lo, &hi);
  int64_t *c = a->counts + (int64_t)tid * 256; /* now: first destination per digit */
  for (int64_t i = lo; i < hi; i++) {
    const int64_t d = c[rs_digit(a, i)]++;
    if (a->k8) a->ok8[d] = a->k8[i]; else a->ok4[d] = a->k4[i];
    if (a->v) a->ov[d] = a->v[i];
  }
}
void mc_radix_sort(void *keys, int32_t *vals, int64_t n, int kb, void *keys_tmp, int32_t *vals_tmp,
                   int threads) {
  int64_t *counts = (int64_t *)malloc(sizeof(int64_t) * 256 * (size_t)threads);
  void *src = keys, *dst = keys_tmp;
  int32_t *vsrc = vals, *vdst = vals_tmp;
  for (int pass = 0; pass < kb; pass++) {
    struct rs_arg a = {kb == 8 ? (const uint64_t *)src : NULL, kb == 4 ? (const uint32_t *)src : NULL,
                       vsrc, (uint64_t *)dst, (uint32_t *)dst, vdst, n, 8 * pass, counts};
    par_loop(threads, rs_count_task, &a);
    int64_t run = 0; /* exclusive scan in (digit, task) order */
    for (int d = 0; d < 256; d++)
      for (int t = 0; t < threads; t++) {
        const int64_t c = counts[(int64_t)t * 256 + d];
        counts[(int64_t)t * 256 + d] = run;
        run += c;
      }
    par_loop(threads, rs_scatter_task, &a);
    void *tk = src; src = dst; dst = tk;
    int32_t *tv = vsrc; vsrc = vdst; vdst = tv;
  }
  /* kb passes: an even number, so the result is back in `keys` / `vals` */
  free(counts);
}
