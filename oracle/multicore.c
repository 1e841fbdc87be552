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
