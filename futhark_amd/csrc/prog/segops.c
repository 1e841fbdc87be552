/*
 * segops.c -- the `segops` program: array types and entry points of the public
 * API in include/segops.h, written the way the Futhark C backends generate
 * them (array functions: src/Futhark/CodeGen/Backends/GenericC/Types.hs:177-240;
 * entry-point wrapper with lock, size checks and output packing:
 * GenericC/EntryPoints.hs:133-208), with each SegOp handed to the gfx950
 * kernel library instead of to a `gpu_kernel_*` launch wrapper.
 */
#define _POSIX_C_SOURCE 200809L
#include <stdlib.h>
#include <string.h>

#include "../rts/rts.h"
#include "futhark_amd_kernels.h"
#include "segops.h"

/* ---------------------------------------------------------- tuning params
 * Named like the reference names them, `<entry>.<description>`
 * (src/Futhark/CodeGen/ImpGen/GPU/Base.hs:118-120). */
static const char *const tuning_names[] = {
    "segops.hist_lds_bins_max",
    "segops.segred_small_threshold",
    "segops.matmul_pad_min_work",
    "segops.scan_arrival_tickets",
    "segops.sort_wide_positions",
};
static const char *const tuning_classes[] = {"shared_memory", "threshold", "threshold", "threshold",
                                             "threshold"};
static const int64_t tuning_defaults[] = {0, 0, 0, 0, 0}; /* 0: the kernel library's default */

/* The parameters choose code paths inside the kernel library (fa_tuning).
 *
 * segops.scan_arrival_tickets: how the blocks of the single-pass scan pick
 * their ticket counter (fa_tuning.scan_tickets_by_block).  0 lets the runtime
 * decide: by block index, the cheaper way, while this context is the only one
 * alive in the process and no CU mask is set in the environment (a scan of a
 * single stream then has the device to itself, as far as this process can
 * tell), by order of arrival otherwise.  1 always takes the order of arrival:
 * for a process that shares the GPU with other processes' long-running
 * kernels, or runs under a CU mask it applies by other means.
 *
 * segops.sort_wide_positions: 1 makes the radix sort use the 64-bit positions
 * it otherwise switches to at 2^32 - 1 keys (fa_tuning.sort_wide_positions). */
static void apply_tuning(struct futhark_context *ctx) {
  fa_tuning t;
  t.hist_lds_bins_max = rts_tuning_param(ctx, tuning_names[0], 0);
  t.segred_small_threshold = rts_tuning_param(ctx, tuning_names[1], 0);
  t.matmul_pad_min_work = rts_tuning_param(ctx, tuning_names[2], 0);
  t.scan_tickets_by_block =
      rts_tuning_param(ctx, tuning_names[3], 0) == 0 && rts_device_is_ours(ctx) ? 1 : 0;
  t.sort_wide_positions = rts_tuning_param(ctx, tuning_names[4], 0) != 0;
  fa_set_tuning(&t);
}

const struct rts_program futhark_program = {
    "segops", 5, tuning_names, tuning_classes, tuning_defaults, apply_tuning,
};

/* ------------------------------------------------------------------ arrays */

struct fut_array {
  struct memblock_device mem;
  int64_t shape[3];
};

static int64_t shape_elems(int rank, const int64_t *shape) {
  int64_t n = 1;
  for (int i = 0; i < rank; i++) n *= shape[i];
  return n;
}

static struct fut_array *array_new(struct futhark_context *ctx, const void *data, size_t elem,
                                   int rank, const int64_t *dims, const char *desc) {
  struct fut_array *arr = (struct fut_array *)calloc(1, sizeof(struct fut_array));
  if (arr == NULL) return NULL;
  int err = 0;
  pthread_mutex_lock(&ctx->lock);
  for (int i = 0; i < rank; i++) {
    arr->shape[i] = dims[i];
    if (dims[i] < 0) err = 1;
  }
  if (err) {
    rts_set_error(ctx, strdup("Negative array dimension.\n"));
  } else {
    const int64_t bytes = shape_elems(rank, dims) * (int64_t)elem;
    err = rts_memblock_alloc(ctx, &arr->mem, bytes, desc);
    if (err == 0) {
      err = rts_copy_h2d(ctx, arr->mem.mem, data, (size_t)bytes);
      if (err != 0) rts_memblock_unref(ctx, &arr->mem, desc);
    }
  }
  pthread_mutex_unlock(&ctx->lock);
  if (err != 0) {
    free(arr);
    return NULL;
  }
  return arr;
}

static struct fut_array *array_new_raw(struct futhark_context *ctx, void *data, size_t elem,
                                       int rank, const int64_t *dims) {
  (void)ctx;
  struct fut_array *arr = (struct fut_array *)calloc(1, sizeof(struct fut_array));
  if (arr == NULL) return NULL;
  for (int i = 0; i < rank; i++) arr->shape[i] = dims[i];
  arr->mem.references = NULL;
  arr->mem.mem = data;
  arr->mem.size = shape_elems(rank, dims) * (int64_t)elem;
  arr->mem.desc = "raw";
  return arr;
}

static int array_free(struct futhark_context *ctx, struct fut_array *arr, const char *desc) {
  pthread_mutex_lock(&ctx->lock);
  int err = rts_memblock_unref(ctx, &arr->mem, desc);
  pthread_mutex_unlock(&ctx->lock);
  free(arr);
  return err;
}

static int array_values(struct futhark_context *ctx, struct fut_array *arr, void *out,
                        size_t elem, int rank) {
  pthread_mutex_lock(&ctx->lock);
  int err =
      rts_copy_d2h(ctx, out, arr->mem.mem, (size_t)shape_elems(rank, arr->shape) * elem);
  pthread_mutex_unlock(&ctx->lock);
  return err;
}

static int array_index(struct futhark_context *ctx, void *out, struct fut_array *arr,
                       size_t elem, int rank, const int64_t *idx) {
  int64_t flat = 0;
  for (int i = 0; i < rank; i++) {
    if (idx[i] < 0 || idx[i] >= arr->shape[i]) {
      rts_set_error(ctx, strdup("Index out of bounds."));
      return 1;
    }
    flat = flat * arr->shape[i] + idx[i];
  }
  pthread_mutex_lock(&ctx->lock);
  int err = rts_copy_d2h(ctx, out, (const char *)arr->mem.mem + flat * (int64_t)elem, elem);
  pthread_mutex_unlock(&ctx->lock);
  return err;
}

#define DIMS_PARAMS_1 int64_t dim0
#define DIMS_PARAMS_2 int64_t dim0, int64_t dim1
#define DIMS_PARAMS_3 int64_t dim0, int64_t dim1, int64_t dim2
#define DIMS_ARGS_1 {dim0}
#define DIMS_ARGS_2 {dim0, dim1}
#define DIMS_ARGS_3 {dim0, dim1, dim2}
#define IDX_PARAMS_1 int64_t i0
#define IDX_PARAMS_2 int64_t i0, int64_t i1
#define IDX_PARAMS_3 int64_t i0, int64_t i1, int64_t i2
#define IDX_ARGS_1 {i0}
#define IDX_ARGS_2 {i0, i1}
#define IDX_ARGS_3 {i0, i1, i2}

#define DEFINE_ARRAY(NAME, CT, R)                                                              \
  struct futhark_##NAME##_##R##d {                                                             \
    struct fut_array a;                                                                        \
  };                                                                                           \
  struct futhark_##NAME##_##R##d *futhark_new_##NAME##_##R##d(struct futhark_context *ctx,     \
                                                              const CT *data,                  \
                                                              DIMS_PARAMS_##R) {               \
    const int64_t dims[3] = DIMS_ARGS_##R;                                                     \
    return (struct futhark_##NAME##_##R##d *)array_new(ctx, data, sizeof(CT), R, dims,         \
                                                       "arr->mem");                            \
  }                                                                                            \
  struct futhark_##NAME##_##R##d *futhark_new_raw_##NAME##_##R##d(                             \
      struct futhark_context *ctx, futhark_device_ptr data, DIMS_PARAMS_##R) {                 \
    const int64_t dims[3] = DIMS_ARGS_##R;                                                     \
    return (struct futhark_##NAME##_##R##d *)array_new_raw(ctx, data, sizeof(CT), R, dims);    \
  }                                                                                            \
  int futhark_free_##NAME##_##R##d(struct futhark_context *ctx,                                \
                                   struct futhark_##NAME##_##R##d *arr) {                      \
    return array_free(ctx, &arr->a, "arr->mem");                                               \
  }                                                                                            \
  int futhark_values_##NAME##_##R##d(struct futhark_context *ctx,                              \
                                     struct futhark_##NAME##_##R##d *arr, CT *data) {          \
    return array_values(ctx, &arr->a, data, sizeof(CT), R);                                    \
  }                                                                                            \
  int futhark_index_##NAME##_##R##d(struct futhark_context *ctx, CT *out,                      \
                                    struct futhark_##NAME##_##R##d *arr, IDX_PARAMS_##R) {     \
    const int64_t idx[3] = IDX_ARGS_##R;                                                       \
    return array_index(ctx, out, &arr->a, sizeof(CT), R, idx);                                 \
  }                                                                                            \
  futhark_device_ptr futhark_values_raw_##NAME##_##R##d(struct futhark_context *ctx,           \
                                                        struct futhark_##NAME##_##R##d *arr) { \
    (void)ctx;                                                                                 \
    return arr->a.mem.mem;                                                                     \
  }                                                                                            \
  const int64_t *futhark_shape_##NAME##_##R##d(struct futhark_context *ctx,                    \
                                               struct futhark_##NAME##_##R##d *arr) {          \
    (void)ctx;                                                                                 \
    return arr->a.shape;                                                                       \
  }

DEFINE_ARRAY(i32, int32_t, 1)
DEFINE_ARRAY(i64, int64_t, 1)
DEFINE_ARRAY(i8, int8_t, 1)
DEFINE_ARRAY(i16, int16_t, 1)
DEFINE_ARRAY(u8, uint8_t, 1)
DEFINE_ARRAY(u16, uint16_t, 1)
DEFINE_ARRAY(f16, uint16_t, 1)
DEFINE_ARRAY(u32, uint32_t, 1)
DEFINE_ARRAY(u64, uint64_t, 1)
DEFINE_ARRAY(f32, float, 1)
DEFINE_ARRAY(f64, double, 1)
DEFINE_ARRAY(i32, int32_t, 2)
DEFINE_ARRAY(i64, int64_t, 2)
DEFINE_ARRAY(f32, float, 2)
DEFINE_ARRAY(f64, double, 2)
DEFINE_ARRAY(f32, float, 3)
DEFINE_ARRAY(f16, uint16_t, 3)
DEFINE_ARRAY(u16, uint16_t, 3)

/* ------------------------------------------------------ entry-point helpers */

/* A fresh output array of `rank` dims over a new block of `bytes` bytes. */
static struct fut_array *out_array(struct futhark_context *ctx, int64_t bytes, int rank,
                                   const int64_t *dims, const char *desc) {
  struct fut_array *arr = (struct fut_array *)calloc(1, sizeof(struct fut_array));
  if (arr == NULL) return NULL;
  if (rts_memblock_alloc(ctx, &arr->mem, bytes, desc) != 0) {
    free(arr);
    return NULL;
  }
  for (int i = 0; i < rank; i++) arr->shape[i] = dims[i];
  return arr;
}

static void drop_array(struct futhark_context *ctx, struct fut_array *arr) {
  if (arr != NULL) {
    rts_memblock_unref(ctx, &arr->mem, "out");
    free(arr);
  }
}

static int bad_sizes(struct futhark_context *ctx, const char *entry) {
  rts_set_error(ctx, rts_msgprintf("Error: entry point arguments have invalid sizes.\n"
                                   "Entry point: %s\n", entry));
  return 1;
}

static const fa_dtype DT_i32 = FA_I32, DT_i64 = FA_I64, DT_f32 = FA_F32, DT_f64 = FA_F64,
                      DT_i8 = FA_I8, DT_u8 = FA_U8, DT_i16 = FA_I16, DT_u16 = FA_U16,
                      DT_u32 = FA_U32, DT_u64 = FA_U64, DT_f16 = FA_F16;
static const fa_op OP_add = FA_ADD, OP_max = FA_MAX, OP_min = FA_MIN, OP_and = FA_AND, OP_or = FA_OR,
                   OP_xor = FA_XOR;

static int do_reduce(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es, void *out,
                     const struct fut_array *in) {
  const int64_t n = in->shape[0];
  uint32_t epoch = 0;
  void *scratch = rts_scan_scratch(ctx, fa_segred_scratch_bytes(t), &epoch);
  if (scratch == NULL) return ctx->error ? FUTHARK_OUT_OF_MEMORY : 1;
  /* The kernel stores the one result into a pinned host slot of the context;
   * the caller gets it at the next futhark_context_sync. */
  void *slot = rts_scalar_slot(ctx);
  if (slot == NULL) return 1;
  struct rts_event *ev = rts_kernel_begin(
      ctx, "segred_nonseg", rts_msgprintf("{\"n\":%lld,\"bytes\":%lld}", (long long)n,
                                          (long long)(n * (int64_t)es)));
  int code = fa_segred_nonseg(ctx->stream, t, op, in->mem.mem, n, slot, scratch,
                              ctx->scan_scratch_bytes, epoch);
  int err = rts_kernel_end(ctx, ev, "segred_nonseg", code);
  if (err == 0) err = rts_take_scalar(ctx, slot, out, es);
  return err;
}

static int do_scan(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                   struct fut_array **out, const struct fut_array *flags,
                   const struct fut_array *in, int exclusive, const char *entry) {
  const int64_t n = in->shape[0];
  if (flags != NULL && flags->shape[0] != n) return bad_sizes(ctx, entry);
  const int pairs = t == FA_I32X2;  /* [n][2]i32, one (a, b) per row */
  if (pairs && in->shape[1] != 2) return bad_sizes(ctx, entry);
  uint32_t epoch = 0;
  const size_t sbytes = fa_segscan_scratch_bytes(t, n);
  void *scratch = rts_scan_scratch(ctx, sbytes, &epoch);
  if (scratch == NULL) return ctx->error ? FUTHARK_OUT_OF_MEMORY : 1;
  struct fut_array *res = out_array(ctx, n * (int64_t)es, pairs ? 2 : 1, in->shape, "scan.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct rts_event *ev = rts_kernel_begin(
      ctx, "segscan", rts_msgprintf("{\"n\":%lld,\"segmented\":%d,\"exclusive\":%d}",
                                    (long long)n, flags != NULL, exclusive));
  int code = fa_segscan(ctx->stream, t, op, in->mem.mem,
                        flags ? (const uint8_t *)flags->mem.mem : NULL, n, exclusive,
                        res->mem.mem, scratch, ctx->scan_scratch_bytes, epoch);
  int err = rts_kernel_end(ctx, ev, "segscan", code);
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

static int do_segred(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                     struct fut_array **out, const struct fut_array *offsets,
                     const struct fut_array *lens, const struct fut_array *vs,
                     const char *entry) {
  const int64_t m = offsets->shape[0], n = vs->shape[0];
  if (lens->shape[0] != m) return bad_sizes(ctx, entry);
  /* The kernels are memory-safe whatever the segments are, but their result is
     only defined for ordered, disjoint segments inside the array: anything
     else makes the next synchronisation fail, as an index out of bounds does
     in a compiled program.  The reduction's first kernel checks them. */
  struct fut_array *res = out_array(ctx, m * (int64_t)es, 1, &m, "segred.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  /* Plain workspace from the pool; not the look-back scratch of the scans,
     whose contents must stay valid descriptors. */
  struct memblock_device scratch = {0};
  int err = rts_memblock_alloc(ctx, &scratch, (int64_t)fa_segred_irregular_scratch_bytes(t, n),
                               "segred.scratch");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "segred_irregular",
        rts_msgprintf("{\"n\":%lld,\"segments\":%lld}", (long long)n, (long long)m));
    int code = fa_segred_irregular_checked(ctx->stream, t, op, vs->mem.mem, n,
                                           (const int64_t *)offsets->mem.mem,
                                           (const int64_t *)lens->mem.mem, m, res->mem.mem,
                                           scratch.mem, (size_t)scratch.size,
                                           RTS_FAILURE_WORD(ctx), RTS_FAILURE_SEGMENTS);
    err = rts_kernel_end(ctx, ev, "segred_irregular", code);
  }
  rts_memblock_unref(ctx, &scratch, "segred.scratch");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* reduce (map2 OP) (replicate k NE) xss : [k]T for xss : [n][k]T */
static int do_vecreduce(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                        struct fut_array **out, const struct fut_array *in) {
  const int64_t n = in->shape[0], k = in->shape[1];
  struct fut_array *res = out_array(ctx, k * (int64_t)es, 1, &k, "vecreduce.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct memblock_device ws = {0};
  const size_t ws_bytes = fa_segred_columns_workspace_bytes(t, n, k);
  int err = 0;
  if (ws_bytes > 0) err = rts_memblock_alloc(ctx, &ws, (int64_t)ws_bytes, "vecreduce.workspace");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "segred_columns",
        rts_msgprintf("{\"rows\":%lld,\"vector_size\":%lld}", (long long)n, (long long)k));
    int code = fa_segred_columns(ctx->stream, t, op, in->mem.mem, n, k, res->mem.mem, ws.mem,
                                 ws_bytes);
    err = rts_kernel_end(ctx, ev, "segred_columns", code);
  }
  rts_memblock_unref(ctx, &ws, "vecreduce.workspace");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

static int do_segreduce(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                        struct fut_array **out, const struct fut_array *in) {
  const int64_t m = in->shape[0], k = in->shape[1];
  struct fut_array *res = out_array(ctx, m * (int64_t)es, 1, &m, "segreduce.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct memblock_device ws = {0};
  const size_t ws_bytes = fa_segred_regular_workspace_bytes(t, m, k);
  int err = 0;
  if (ws_bytes > 0) err = rts_memblock_alloc(ctx, &ws, (int64_t)ws_bytes, "segreduce.workspace");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "segred_regular",
        rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)k));
    int code = fa_segred_regular_ws(ctx->stream, t, op, in->mem.mem, m, k, res->mem.mem, ws.mem,
                                    ws_bytes);
    err = rts_kernel_end(ctx, ev, "segred_regular", code);
  }
  rts_memblock_unref(ctx, &ws, "segreduce.workspace");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* `map (scan op ne) xss`: the scan kernel with row starts in place of flags. */
static int do_scanrows(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                       struct fut_array **out, const struct fut_array *in) {
  const int64_t m = in->shape[0], k = in->shape[1];
  uint32_t epoch = 0;
  const size_t sbytes = fa_segscan_scratch_bytes(t, m * k);
  void *scratch = rts_scan_scratch(ctx, sbytes, &epoch);
  if (scratch == NULL) return ctx->error ? FUTHARK_OUT_OF_MEMORY : 1;
  const int64_t dims[2] = {m, k};
  struct fut_array *res = out_array(ctx, m * k * (int64_t)es, 2, dims, "scanrows.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct rts_event *ev = rts_kernel_begin(
      ctx, "segscan_rows",
      rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)k));
  int code = fa_segscan_rows(ctx->stream, t, op, in->mem.mem, m, k, 0, res->mem.mem, scratch,
                             ctx->scan_scratch_bytes, epoch);
  int err = rts_kernel_end(ctx, ev, "segscan_rows", code);
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* `scan (map2 op) (replicate k ne) xss` for xss : [n][k]T: column j of the
 * result is the scan of column j.  The single-pass scan takes operators on
 * scalars (the reference's own refuses array operators too,
 * SegScan/SinglePass.hs canBeSinglePass, and falls back to two passes).  Rows
 * of whole 1 KiB strips go to fa_vecscan (fold per chunk of rows, prefixes
 * over the chunks, scan per chunk: no transposed copy); for every other shape
 * the matrix is transposed, its rows are scanned with the single-pass kernel,
 * and the result is transposed back, so that every access to HBM is a
 * coalesced one. */
static int do_vecscan(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                      struct fut_array **out, const struct fut_array *in) {
  const int64_t n = in->shape[0], k = in->shape[1];
  if (k != 0 && n > INT64_MAX / (int64_t)es / k) {
    rts_set_error(ctx, rts_msgprintf("vecscan: %lld rows of %lld elements do not fit an int64 size\n",
                                     (long long)n, (long long)k));
    return 1;
  }
  const int64_t dims[2] = {n, k};
  struct fut_array *res = out_array(ctx, n * k * (int64_t)es, 2, dims, "vecscan.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  if (n == 0 || k == 0) {
    *out = res;
    return 0;
  }
  const size_t direct_bytes = fa_vecscan_workspace_bytes(t, n, k);
  if (direct_bytes > 0) { /* rows of whole 1 KiB strips: no transposed copy */
    struct memblock_device ws = {0};
    int err = rts_memblock_alloc(ctx, &ws, (int64_t)direct_bytes, "vecscan.workspace");
    if (err == 0) {
      struct rts_event *ev = rts_kernel_begin(
          ctx, "vecscan", rts_msgprintf("{\"rows\":%lld,\"vector_size\":%lld,\"transposed\":false}",
                                        (long long)n, (long long)k));
      int code = fa_vecscan(ctx->stream, t, op, in->mem.mem, n, k, res->mem.mem, ws.mem, direct_bytes);
      err = rts_kernel_end(ctx, ev, "vecscan", code);
    }
    rts_memblock_unref(ctx, &ws, "vecscan.workspace");
    if (err != 0) {
      drop_array(ctx, res);
      return err;
    }
    *out = res;
    return 0;
  }
  uint32_t epoch = 0;
  const size_t sbytes = fa_segscan_scratch_bytes(t, n * k);
  void *scratch = rts_scan_scratch(ctx, sbytes, &epoch);
  struct memblock_device tmp = {0};
  int err = scratch == NULL ? (ctx->error ? FUTHARK_OUT_OF_MEMORY : 1) : 0;
  if (err == 0) err = rts_memblock_alloc(ctx, &tmp, n * k * (int64_t)es, "vecscan.transposed");
  if (err == 0) {
    /* res holds the transposed input first, the result at the end */
    struct rts_event *ev = rts_kernel_begin(
        ctx, "vecscan", rts_msgprintf("{\"rows\":%lld,\"vector_size\":%lld,\"transposed\":true}", (long long)n, (long long)k));
    int code = fa_map_transpose(ctx->stream, (int)es, res->mem.mem, in->mem.mem, 1, n, k);
    if (code == 0)
      code = fa_segscan_rows(ctx->stream, t, op, res->mem.mem, k, n, 0, tmp.mem, scratch,
                             ctx->scan_scratch_bytes, epoch);
    if (code == 0) code = fa_map_transpose(ctx->stream, (int)es, res->mem.mem, tmp.mem, 1, k, n);
    err = rts_kernel_end(ctx, ev, "vecscan", code);
  }
  rts_memblock_unref(ctx, &tmp, "vecscan.transposed");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* Bit pattern of the neutral element: 0 for add, or, xor; all ones for and;
 * T.lowest / T.highest for max / min (prelude/math.fut: the smallest / largest
 * integer of the type, -inf / +inf for floats). */
static uint64_t neutral_bits(fa_dtype t, fa_op op) {
  union { float f; uint32_t u; } b32;
  union { double f; uint64_t u; } b64;
  if (op == FA_ADD || op == FA_OR || op == FA_XOR) return 0;
  if (op == FA_AND) return ~0ull; /* truncated to the element size by the fill */
  const int max = op == FA_MAX;
  switch (t) {
    case FA_I8: return (uint8_t)(max ? INT8_MIN : INT8_MAX);
    case FA_I16: return (uint16_t)(max ? INT16_MIN : INT16_MAX);
    case FA_I32: return (uint32_t)(max ? INT32_MIN : INT32_MAX);
    case FA_I64: return (uint64_t)(max ? INT64_MIN : INT64_MAX);
    case FA_U8: return max ? 0 : UINT8_MAX;
    case FA_U16: return max ? 0 : UINT16_MAX;
    case FA_U32: return max ? 0 : UINT32_MAX;
    case FA_U64: return max ? 0 : UINT64_MAX;
    case FA_F16: return max ? 0xFC00u : 0x7C00u;
    case FA_F32:
      b32.f = max ? -__builtin_inff() : __builtin_inff();
      return b32.u;
    default:
      b64.f = max ? -__builtin_inf() : __builtin_inf();
      return b64.u;
  }
}

/* dest_in == NULL: histogram into a fresh array of k neutral elements. */
static int do_hist(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                   struct fut_array **out, int64_t k, const struct fut_array *dest_in,
                   const struct fut_array *is, int is64, const struct fut_array *vs,
                   const char *entry) {
  const int64_t n = is->shape[0];
  if (vs->shape[0] != n) return bad_sizes(ctx, entry);
  if (dest_in != NULL) k = dest_in->shape[0];
  if (k < 0) {
    rts_set_error(ctx, rts_msgprintf("Error: negative histogram size %lld.\n", (long long)k));
    return FUTHARK_PROGRAM_ERROR;
  }
  if (k > INT64_MAX / (int64_t)es) {
    rts_set_error(ctx, rts_msgprintf("Error: %lld bins do not fit in memory.\n", (long long)k));
    return FUTHARK_OUT_OF_MEMORY;
  }
  struct fut_array *res = out_array(ctx, k * (int64_t)es, 1, &k, "hist.dest");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  int err = 0;
  if (dest_in != NULL) {
    err = rts_copy_d2d(ctx, res->mem.mem, dest_in->mem.mem, (size_t)k * es);
  } else if (k > 0) {
    int code = fa_replicate(ctx->stream, (int)es, res->mem.mem, k, neutral_bits(t, op));
    err = rts_kernel_end(ctx, NULL, "replicate", code);
  }
  struct memblock_device scratch = {0};
  if (err == 0) {
    err = rts_memblock_alloc(ctx, &scratch, (int64_t)fa_seghist_scratch_bytes(t, is64, n, k),
                             "hist.scratch");
  }
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "seghist", rts_msgprintf("{\"n\":%lld,\"bins\":%lld}", (long long)n, (long long)k));
    int code = fa_seghist(ctx->stream, t, op, is->mem.mem, is64, vs->mem.mem, n, res->mem.mem, k,
                          scratch.mem, (size_t)scratch.size);
    err = rts_kernel_end(ctx, ev, "seghist", code);
  }
  rts_memblock_unref(ctx, &scratch, "hist.scratch");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* `map2 (hist op ne k) iss vss`: one histogram of k bins per row. */
static int do_seghist(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                      struct fut_array **out, int64_t k, const struct fut_array *iss,
                      const struct fut_array *vss, const char *entry) {
  const int64_t m = iss->shape[0], len = iss->shape[1];
  if (vss->shape[0] != m || vss->shape[1] != len) return bad_sizes(ctx, entry);
  if (k < 0) {
    rts_set_error(ctx, rts_msgprintf("Error: negative histogram size %lld.\n", (long long)k));
    return FUTHARK_PROGRAM_ERROR;
  }
  /* m * k * es must be a size that exists before anything is done with it */
  if (m > 0 && k > (INT64_MAX / (int64_t)es) / m) {
    rts_set_error(ctx, rts_msgprintf("Error: %lld histograms of %lld bins do not fit in memory.\n",
                                     (long long)m, (long long)k));
    return FUTHARK_OUT_OF_MEMORY;
  }
  const int64_t dims[2] = {m, k};
  struct fut_array *res = out_array(ctx, m * k * (int64_t)es, 2, dims, "seghist.dest");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  int err = 0;
  if (m * k > 0) {
    int code = fa_replicate(ctx->stream, (int)es, res->mem.mem, m * k, neutral_bits(t, op));
    err = rts_kernel_end(ctx, NULL, "replicate", code);
  }
  struct memblock_device scratch = {0};
  if (err == 0)
    err = rts_memblock_alloc(ctx, &scratch,
                             (int64_t)fa_seghist_segmented_scratch_bytes(t, m, len, k),
                             "seghist.scratch");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "seghist_segmented",
        rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld,\"bins\":%lld}", (long long)m,
                      (long long)len, (long long)k));
    int code = fa_seghist_segmented(ctx->stream, t, op, iss->mem.mem, 0, vss->mem.mem, m, len,
                                    res->mem.mem, k, scratch.mem, (size_t)scratch.size);
    err = rts_kernel_end(ctx, ev, "seghist_segmented", code);
  }
  rts_memblock_unref(ctx, &scratch, "seghist.scratch");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* Histograms with a shape.  js == NULL: `reduce_by_index dest (map2 op) (replicate m ne) is vss`
 * with dest : [k][m], vss : [n][m].  Otherwise `reduce_by_index_2d dest op ne (zip is js) vs`
 * with dest : [k][l], vss = vs : [n]. */
static int do_rbi_shaped(struct futhark_context *ctx, fa_dtype t, fa_op op, size_t es,
                         struct fut_array **out, const struct fut_array *dest_in,
                         const struct fut_array *is, const struct fut_array *js,
                         const struct fut_array *vss, const char *entry) {
  const int64_t n = is->shape[0];
  const int64_t H0 = dest_in->shape[0];
  const int64_t H1 = js != NULL ? dest_in->shape[1] : 1;
  const int64_t m = js != NULL ? 1 : dest_in->shape[1];
  if (vss->shape[0] != n) return bad_sizes(ctx, entry);
  if (js != NULL && js->shape[0] != n) return bad_sizes(ctx, entry);
  if (js == NULL && vss->shape[1] != m) return bad_sizes(ctx, entry);
  const int64_t cells = dest_in->shape[0] * dest_in->shape[1];
  struct fut_array *res = out_array(ctx, cells * (int64_t)es, 2, dest_in->shape, "hist.dest");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  int err = rts_copy_d2d(ctx, res->mem.mem, dest_in->mem.mem, (size_t)cells * es);
  struct memblock_device scratch = {0};
  if (err == 0)
    err = rts_memblock_alloc(ctx, &scratch,
                             (int64_t)fa_seghist_shaped_scratch_bytes(t, 1, n, H0, H1, m),
                             "hist.scratch");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "seghist_shaped",
        rts_msgprintf("{\"n\":%lld,\"bins\":[%lld,%lld],\"vector_size\":%lld}", (long long)n,
                      (long long)H0, (long long)H1, (long long)m));
    int code = fa_seghist_shaped(ctx->stream, t, op, is->mem.mem, js != NULL ? js->mem.mem : NULL,
                                 1, vss->mem.mem, n, res->mem.mem, H0, H1, m, scratch.mem,
                                 (size_t)scratch.size);
    err = rts_kernel_end(ctx, ev, "seghist_shaped", code);
  }
  rts_memblock_unref(ctx, &scratch, "hist.scratch");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

/* Every entry point runs under the context's lock and with the context's tuning
 * parameters in force for the calling thread (the kernel library keeps them per
 * thread), so contexts with different parameters can be used side by side. */
#define ENTER(ctx)                      \
  do {                                  \
    pthread_mutex_lock(&(ctx)->lock);   \
    apply_tuning(ctx);                  \
  } while (0)
#define LEAVE(ctx) pthread_mutex_unlock(&(ctx)->lock)

#define DEFINE_SEGOP_ENTRIES(OP, T, CT)                                                       \
  int futhark_entry_reduce_##OP##_##T(struct futhark_context *ctx, CT *out0,                  \
                                      const struct futhark_##T##_1d *in0) {                   \
    ENTER(ctx);                                                                               \
    int ret = do_reduce(ctx, DT_##T, OP_##OP, sizeof(CT), out0, &in0->a);                     \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_scan_##OP##_##T(struct futhark_context *ctx,                              \
                                    struct futhark_##T##_1d **out0,                           \
                                    const struct futhark_##T##_1d *in0) {                     \
    ENTER(ctx);                                                                               \
    int ret = do_scan(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, NULL,      \
                      &in0->a, 0, "scan_" #OP "_" #T);                                        \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_exscan_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_1d **out0,                         \
                                      const struct futhark_##T##_1d *in0) {                   \
    ENTER(ctx);                                                                               \
    int ret = do_scan(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, NULL,      \
                      &in0->a, 1, "exscan_" #OP "_" #T);                                      \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_segscan_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_1d **out0,                        \
                                       const struct futhark_u8_1d *in0,                       \
                                       const struct futhark_##T##_1d *in1) {                  \
    ENTER(ctx);                                                                               \
    int ret = do_scan(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a,   \
                      &in1->a, 0, "segscan_" #OP "_" #T);                                     \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_segred_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_1d **out0,                         \
                                      const struct futhark_i64_1d *in0,                       \
                                      const struct futhark_i64_1d *in1,                       \
                                      const struct futhark_##T##_1d *in2) {                   \
    ENTER(ctx);                                                                               \
    int ret = do_segred(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a, \
                        &in1->a, &in2->a, "segred_" #OP "_" #T);                              \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_segreduce_##OP##_##T(struct futhark_context *ctx,                         \
                                         struct futhark_##T##_1d **out0,                      \
                                         const struct futhark_##T##_2d *in0) {                \
    ENTER(ctx);                                                                               \
    int ret =                                                                                 \
        do_segreduce(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a);   \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_vecreduce_##OP##_##T(struct futhark_context *ctx,                         \
                                         struct futhark_##T##_1d **out0,                      \
                                         const struct futhark_##T##_2d *in0) {                \
    ENTER(ctx);                                                                               \
    int ret =                                                                                 \
        do_vecreduce(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a);   \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_scanrows_##OP##_##T(struct futhark_context *ctx,                          \
                                        struct futhark_##T##_2d **out0,                       \
                                        const struct futhark_##T##_2d *in0) {                 \
    ENTER(ctx);                                                                               \
    int ret =                                                                                 \
        do_scanrows(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a);    \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_vecscan_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0,                        \
                                       const struct futhark_##T##_2d *in0) {                  \
    ENTER(ctx);                                                                               \
    int ret =                                                                                 \
        do_vecscan(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, &in0->a);     \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_seghist_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0, const int64_t in0,     \
                                       const struct futhark_i32_2d *in1,                      \
                                       const struct futhark_##T##_2d *in2) {                  \
    ENTER(ctx);                                                                               \
    int ret = do_seghist(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, in0,    \
                         &in1->a, &in2->a, "seghist_" #OP "_" #T);                            \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_rbi_vec_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0,                        \
                                       const struct futhark_##T##_2d *in0,                    \
                                       const struct futhark_i64_1d *in1,                      \
                                       const struct futhark_##T##_2d *in2) {                  \
    ENTER(ctx);                                                                               \
    int ret = do_rbi_shaped(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0,      \
                            &in0->a, &in1->a, NULL, &in2->a, "rbi_vec_" #OP "_" #T);          \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_rbi_2d_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_2d **out0,                         \
                                      const struct futhark_##T##_2d *in0,                     \
                                      const struct futhark_i64_1d *in1,                       \
                                      const struct futhark_i64_1d *in2,                       \
                                      const struct futhark_##T##_1d *in3) {                   \
    ENTER(ctx);                                                                               \
    int ret = do_rbi_shaped(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0,      \
                            &in0->a, &in1->a, &in2->a, &in3->a, "rbi_2d_" #OP "_" #T);        \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  DEFINE_HIST_ENTRIES(OP, T, CT)

#define DEFINE_HIST_ENTRIES(OP, T, CT)                                                        \
  DEFINE_HIST_ENTRIES_IX(OP, T, CT, , i32, 0)                                                 \
  DEFINE_HIST_ENTRIES_IX(OP, T, CT, _i64, i64, 1)
/* SUFFIX: nothing for []i32 indices (widened in the fused map), _i64 for the []i64
 * indices `hist` and `reduce_by_index` are defined over (prelude/soacs.fut:132-146). */
#define DEFINE_HIST_ENTRIES_IX(OP, T, CT, SUFFIX, IT, IS64)                                   \
  int futhark_entry_hist_##OP##_##T##SUFFIX(struct futhark_context *ctx,                      \
                                            struct futhark_##T##_1d **out0, const int64_t in0, \
                                            const struct futhark_##IT##_1d *in1,              \
                                            const struct futhark_##T##_1d *in2) {             \
    ENTER(ctx);                                                                               \
    int ret = do_hist(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, in0, NULL, \
                      &in1->a, IS64, &in2->a, "hist_" #OP "_" #T #SUFFIX);                    \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }                                                                                           \
  int futhark_entry_rbi_##OP##_##T##SUFFIX(struct futhark_context *ctx,                       \
                                           struct futhark_##T##_1d **out0,                    \
                                           const struct futhark_##T##_1d *in0,                \
                                           const struct futhark_##IT##_1d *in1,               \
                                           const struct futhark_##T##_1d *in2) {              \
    ENTER(ctx);                                                                               \
    int ret = do_hist(ctx, DT_##T, OP_##OP, sizeof(CT), (struct fut_array **)out0, 0,         \
                      &in0->a, &in1->a, IS64, &in2->a, "rbi_" #OP "_" #T #SUFFIX);            \
    LEAVE(ctx);                                                                               \
    return ret;                                                                               \
  }

/* Scans of affine maps x -> a*x + b (mod 2^32) under composition: rows (a, b) of [n][2]i32. */
int futhark_entry_scan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                   const struct futhark_i32_2d *in0) {
  ENTER(ctx);
  int ret = do_scan(ctx, FA_I32X2, FA_COMPOSE, 8, (struct fut_array **)out0, NULL, &in0->a, 0,
                    "scan_compose_i32");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_exscan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                     const struct futhark_i32_2d *in0) {
  ENTER(ctx);
  int ret = do_scan(ctx, FA_I32X2, FA_COMPOSE, 8, (struct fut_array **)out0, NULL, &in0->a, 1,
                    "exscan_compose_i32");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_segscan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                      const struct futhark_u8_1d *in0,
                                      const struct futhark_i32_2d *in1) {
  ENTER(ctx);
  int ret = do_scan(ctx, FA_I32X2, FA_COMPOSE, 8, (struct fut_array **)out0, &in0->a, &in1->a, 0,
                    "segscan_compose_i32");
  LEAVE(ctx);
  return ret;
}

/* ---- SegOps with operators and fused maps of their own (per-program lambdas):
 * instantiated in csrc/kernels/custom_ops.hip from the public kernel templates. */

/* A reduction to one element; `dev_out` is where the kernel stores it. */
typedef int (*custom_reduce_fn)(fa_stream_t, const void *, int64_t, void *, void *, size_t, uint32_t);
static int do_custom_reduce(struct futhark_context *ctx, custom_reduce_fn fn, const char *name,
                            const struct fut_array *in, int64_t n, void *dev_out) {
  uint32_t epoch = 0;
  void *scratch = rts_scan_scratch(ctx, fa_segred_scratch_bytes(FA_I64), &epoch);
  if (scratch == NULL) return ctx->error ? FUTHARK_OUT_OF_MEMORY : 1;
  struct rts_event *ev = rts_kernel_begin(ctx, name, rts_msgprintf("{\"n\":%lld}", (long long)n));
  int code = fn(ctx->stream, in->mem.mem, n, dev_out, scratch, ctx->scan_scratch_bytes, epoch);
  return rts_kernel_end(ctx, ev, name, code);
}
static int reduce_argmax_fn(fa_stream_t s, const void *xs, int64_t n, void *out, void *sc, size_t sb,
                            uint32_t e) {
  return fa_reduce_argmax_i32(s, (const int32_t *)xs, n, (int32_t *)out, sc, sb, e);
}
static int reduce_compose_fn(fa_stream_t s, const void *xs, int64_t n, void *out, void *sc, size_t sb,
                             uint32_t e) {
  return fa_reduce_compose_i32(s, (const int32_t *)xs, n, (int32_t *)out, sc, sb, e);
}
static int sumsq_fn(fa_stream_t s, const void *xs, int64_t n, void *out, void *sc, size_t sb,
                    uint32_t e) {
  return fa_sumsq_f32(s, (const float *)xs, n, (float *)out, sc, sb, e);
}

/* A reduction whose result is a pair of i32, returned as a [2]i32 array. */
static int summax_fn(fa_stream_t s, const void *xs, int64_t n, void *out, void *sc, size_t sb,
                     uint32_t e) {
  return fa_reduce_summax_f32(s, (const float *)xs, n, (float *)out, sc, sb, e);
}

static int do_pair_reduce(struct futhark_context *ctx, custom_reduce_fn fn, const char *name,
                          struct fut_array **out, const struct fut_array *in) {
  const int64_t two = 2;
  struct fut_array *res = out_array(ctx, 8, 1, &two, "pair.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  int err = do_custom_reduce(ctx, fn, name, in, in->shape[0], res->mem.mem);
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

int futhark_entry_reduce_argmax_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                    const struct futhark_i32_1d *in0) {
  ENTER(ctx);
  int ret = do_pair_reduce(ctx, reduce_argmax_fn, "segred_argmax", (struct fut_array **)out0, &in0->a);
  LEAVE(ctx);
  return ret;
}

int futhark_entry_reduce_summax_f32(struct futhark_context *ctx, struct futhark_f32_1d **out0,
                                    const struct futhark_f32_1d *in0) {
  ENTER(ctx);
  int ret = do_pair_reduce(ctx, summax_fn, "segred_summax", (struct fut_array **)out0, &in0->a);
  LEAVE(ctx);
  return ret;
}

int futhark_entry_reduce_compose_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                     const struct futhark_i32_2d *in0) {
  ENTER(ctx);
  int ret = in0->a.shape[1] != 2
                ? bad_sizes(ctx, "reduce_compose_i32")
                : do_pair_reduce(ctx, reduce_compose_fn, "segred_compose", (struct fut_array **)out0,
                                 &in0->a);
  LEAVE(ctx);
  return ret;
}

int futhark_entry_sumsq_f32(struct futhark_context *ctx, float *out0, const struct futhark_f32_1d *in0) {
  ENTER(ctx);
  void *slot = rts_scalar_slot(ctx);
  int ret = slot == NULL ? 1 : do_custom_reduce(ctx, sumsq_fn, "segred_sumsq", &in0->a, in0->a.shape[0], slot);
  if (ret == 0) ret = rts_take_scalar(ctx, slot, out0, 4);
  LEAVE(ctx);
  return ret;
}

static int do_custom_scan(struct futhark_context *ctx, struct fut_array **out,
                          const struct fut_array *in, int norm, const char *entry) {
  const int64_t n = in->shape[0];
  if (!norm && in->shape[1] != 2) return bad_sizes(ctx, entry);
  uint32_t epoch = 0;
  const size_t sbytes = fa_segscan_scratch_bytes(norm ? FA_F32 : FA_I64, n);
  void *scratch = rts_scan_scratch(ctx, sbytes, &epoch);
  if (scratch == NULL) return ctx->error ? FUTHARK_OUT_OF_MEMORY : 1;
  struct fut_array *res = out_array(ctx, n * (norm ? 4 : 8), norm ? 1 : 2, in->shape, "scan.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct rts_event *ev = rts_kernel_begin(ctx, "segscan", rts_msgprintf("{\"n\":%lld}", (long long)n));
  int code = norm ? fa_scan_norm_f32(ctx->stream, (const float *)in->mem.mem, n, (float *)res->mem.mem,
                                     scratch, ctx->scan_scratch_bytes, epoch)
                  : fa_scan_argmax_i32(ctx->stream, (const int32_t *)in->mem.mem, NULL, n, 0,
                                       (int32_t *)res->mem.mem, scratch, ctx->scan_scratch_bytes, epoch);
  int err = rts_kernel_end(ctx, ev, "segscan", code);
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

int futhark_entry_scan_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                  const struct futhark_i32_2d *in0) {
  ENTER(ctx);
  int ret = do_custom_scan(ctx, (struct fut_array **)out0, &in0->a, 0, "scan_argmax_i32");
  LEAVE(ctx);
  return ret;
}

int futhark_entry_scan_norm_f32(struct futhark_context *ctx, struct futhark_f32_1d **out0,
                                const struct futhark_f32_1d *in0) {
  ENTER(ctx);
  int ret = do_custom_scan(ctx, (struct fut_array **)out0, &in0->a, 1, "scan_norm_f32");
  LEAVE(ctx);
  return ret;
}

/* The tuple and the non-commutative operator in the segmented forms. */
int futhark_entry_segreduce_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                       const struct futhark_i32_2d *in0) {
  ENTER(ctx);
  const int64_t m = in0->a.shape[0], k = in0->a.shape[1];
  const int64_t dims[2] = {m, 2};
  int ret = 0;
  struct fut_array *res = out_array(ctx, m * 8, 2, dims, "segreduce.out");
  if (res == NULL) {
    ret = FUTHARK_OUT_OF_MEMORY;
  } else {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "segred_regular",
        rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)k));
    int code = fa_segreduce_argmax_i32(ctx->stream, (const int32_t *)in0->a.mem.mem, m, k,
                                       (int32_t *)res->mem.mem);
    ret = rts_kernel_end(ctx, ev, "segred_regular", code);
    if (ret != 0) drop_array(ctx, res);
    else *out0 = (struct futhark_i32_2d *)res;
  }
  LEAVE(ctx);
  return ret;
}

/* Rows of k elements of a flat [m * k][2]i32 array; 0 on success with m in *m_out. */
static int rows_of(struct futhark_context *ctx, const struct fut_array *in, int64_t k,
                   const char *entry, int64_t *m_out) {
  const int64_t n = in->shape[0];
  if (in->shape[1] != 2 || k < 0 || (k == 0 && n != 0) || (k > 0 && n % k != 0))
    return bad_sizes(ctx, entry);
  *m_out = k == 0 ? 0 : n / k;
  return 0;
}

int futhark_entry_segreduce_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                        const int64_t in0, const struct futhark_i32_2d *in1) {
  ENTER(ctx);
  int64_t m = 0;
  int ret = rows_of(ctx, &in1->a, in0, "segreduce_compose_i32", &m);
  if (ret == 0) {
    const int64_t dims[2] = {m, 2};
    struct fut_array *res = out_array(ctx, m * 8, 2, dims, "segreduce.out");
    if (res == NULL) {
      ret = FUTHARK_OUT_OF_MEMORY;
    } else {
      struct rts_event *ev = rts_kernel_begin(
          ctx, "segred_regular",
          rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)in0));
      int code = fa_segreduce_compose_i32(ctx->stream, (const int32_t *)in1->a.mem.mem, m, in0,
                                          (int32_t *)res->mem.mem);
      ret = rts_kernel_end(ctx, ev, "segred_regular", code);
      if (ret != 0) drop_array(ctx, res);
      else *out0 = (struct futhark_i32_2d *)res;
    }
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_scanrows_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                      const int64_t in0, const struct futhark_i32_2d *in1) {
  ENTER(ctx);
  int64_t m = 0;
  int ret = rows_of(ctx, &in1->a, in0, "scanrows_argmax_i32", &m);
  if (ret == 0) {
    const int64_t n = in1->a.shape[0];
    uint32_t epoch = 0;
    void *scratch = rts_scan_scratch(ctx, fa_segscan_scratch_bytes(FA_I64, n), &epoch);
    struct fut_array *res = scratch == NULL ? NULL : out_array(ctx, n * 8, 2, in1->a.shape, "scan.out");
    if (res == NULL) {
      ret = ctx->error || scratch != NULL ? FUTHARK_OUT_OF_MEMORY : 1;
    } else {
      struct rts_event *ev = rts_kernel_begin(
          ctx, "segscan_rows",
          rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)in0));
      int code = fa_scanrows_argmax_i32(ctx->stream, (const int32_t *)in1->a.mem.mem, m, in0,
                                        (int32_t *)res->mem.mem, scratch, ctx->scan_scratch_bytes,
                                        epoch);
      ret = rts_kernel_end(ctx, ev, "segscan_rows", code);
      if (ret != 0) drop_array(ctx, res);
      else *out0 = (struct futhark_i32_2d *)res;
    }
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_segred_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                    const struct futhark_i64_1d *in0,
                                    const struct futhark_i64_1d *in1,
                                    const struct futhark_i32_2d *in2) {
  ENTER(ctx);
  const int64_t m = in0->a.shape[0], n = in2->a.shape[0];
  int ret = 0;
  if (in1->a.shape[0] != m || in2->a.shape[1] != 2) {
    ret = bad_sizes(ctx, "segred_argmax_i32");
  } else {
    const int64_t dims[2] = {m, 2};
    uint32_t epoch = 0;
    void *scratch = rts_scan_scratch(ctx, fa_segscan_scratch_bytes(FA_I64, n), &epoch);
    struct fut_array *res = scratch == NULL ? NULL : out_array(ctx, m * 8, 2, dims, "segred.out");
    struct memblock_device ws = {0};
    if (res == NULL) {
      ret = ctx->error || scratch != NULL ? FUTHARK_OUT_OF_MEMORY : 1;
    } else if ((ret = rts_memblock_alloc(ctx, &ws, (int64_t)fa_segred_argmax_workspace_bytes(n),
                                         "segred.workspace")) == 0) {
      /* The segments are checked like those of the library's own segmented
       * reduction: a violation is reported at the next synchronisation. */
      struct rts_event *ev = rts_kernel_begin(
          ctx, "segred_irregular", rts_msgprintf("{\"n\":%lld,\"segments\":%lld}", (long long)n, (long long)m));
      int code = fa_segments_check(ctx->stream, (const int64_t *)in0->a.mem.mem,
                                   (const int64_t *)in1->a.mem.mem, m, n, RTS_FAILURE_WORD(ctx),
                                   RTS_FAILURE_SEGMENTS);
      if (code == 0)
        code = fa_segred_argmax_i32(ctx->stream, (const int64_t *)in0->a.mem.mem,
                                    (const int64_t *)in1->a.mem.mem, m,
                                    (const int32_t *)in2->a.mem.mem, n, (int32_t *)res->mem.mem, ws.mem,
                                    (size_t)ws.size, scratch, ctx->scan_scratch_bytes, epoch);
      ret = rts_kernel_end(ctx, ev, "segred_irregular", code);
    }
    rts_memblock_unref(ctx, &ws, "segred.workspace");
    if (ret != 0) drop_array(ctx, res);
    else *out0 = (struct futhark_i32_2d *)res;
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_rows_fraction_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                                    const struct futhark_f32_2d *in0) {
  ENTER(ctx);
  const struct fut_array *in = &in0->a;
  const int64_t m = in->shape[0], k = in->shape[1];
  int ret = 0;
  struct fut_array *res = NULL;
  if (k != 0 && m > INT64_MAX / 4 / k) {
    rts_set_error(ctx, rts_msgprintf("rows_fraction_f32: %lld rows of %lld elements do not fit an int64 size\n",
                                     (long long)m, (long long)k));
    ret = 1;
  } else if ((res = out_array(ctx, m * k * 4, 2, in->shape, "rows_fraction.out")) == NULL) {
    ret = FUTHARK_OUT_OF_MEMORY;
  } else {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "intrablock_rows",
        rts_msgprintf("{\"segments\":%lld,\"segment_size\":%lld}", (long long)m, (long long)k));
    int code = fa_rows_fraction_f32(ctx->stream, (const float *)in->mem.mem, m, k, (float *)res->mem.mem);
    ret = rts_kernel_end(ctx, ev, "intrablock_rows", code);
    if (ret != 0)
      drop_array(ctx, res);
    else
      *out0 = (struct futhark_f32_2d *)res;
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_hist_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                  const int64_t in0, const struct futhark_i32_1d *in1,
                                  const struct futhark_i32_1d *in2) {
  ENTER(ctx);
  int ret = 0;
  const int64_t k = in0, n = in1->a.shape[0];
  if (in2->a.shape[0] != n) {
    ret = bad_sizes(ctx, "hist_argmax_i32");
  } else if (k < 0 || k > fa_hist_argmax_max_bins()) {
    rts_set_error(ctx, rts_msgprintf("hist_argmax_i32: between 0 and %lld bins, got %lld\n",
                                     (long long)fa_hist_argmax_max_bins(), (long long)k));
    ret = FUTHARK_PROGRAM_ERROR;
  } else {
    const int64_t shape[2] = {k, 2};
    struct fut_array *res = out_array(ctx, k * 8, 2, shape, "hist.out");
    if (res == NULL) {
      ret = FUTHARK_OUT_OF_MEMORY;
    } else {
      /* every bin starts as the neutral pair (i32.lowest, i32.highest) */
      const uint64_t ne = ((uint64_t)(uint32_t)INT32_MAX << 32) | (uint32_t)INT32_MIN;
      struct memblock_device ws = {0};
      ret = rts_memblock_alloc(ctx, &ws, (int64_t)fa_hist_argmax_workspace_bytes(k), "hist.workspace");
      if (ret == 0) {
        struct rts_event *ev = rts_kernel_begin(
            ctx, "seghist_locked", rts_msgprintf("{\"n\":%lld,\"bins\":%lld}", (long long)n, (long long)k));
        int code = fa_replicate(ctx->stream, 8, res->mem.mem, k, ne);
        if (code == 0)
          code = fa_hist_argmax_i32(ctx->stream, (const int32_t *)in1->a.mem.mem,
                                    (const int32_t *)in2->a.mem.mem, n, (int32_t *)res->mem.mem, k,
                                    ws.mem, (size_t)ws.size);
        ret = rts_kernel_end(ctx, ev, "seghist_locked", code);
        rts_memblock_unref(ctx, &ws, "hist.workspace");
      }
      if (ret != 0) drop_array(ctx, res);
      else *out0 = (struct futhark_i32_2d *)res;
    }
  }
  LEAVE(ctx);
  return ret;
}

#define DEFINE_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_OP(DEFINE_SEGOP_ENTRIES, T, CT)
FUTHARK_FOR_EACH_NUM_TYPE(DEFINE_FOR_TYPE)
#define DEFINE_BITOPS_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_BITOP(DEFINE_SEGOP_ENTRIES, T, CT)
FUTHARK_FOR_EACH_INT_TYPE(DEFINE_BITOPS_FOR_TYPE)
#define DEFINE_HIST_ONLY_INT(T, CT)                  \
  FUTHARK_FOR_EACH_OP(DEFINE_HIST_ENTRIES, T, CT)    \
  FUTHARK_FOR_EACH_BITOP(DEFINE_HIST_ENTRIES, T, CT)
FUTHARK_FOR_EACH_HIST_ONLY_INT_TYPE(DEFINE_HIST_ONLY_INT)
FUTHARK_FOR_EACH_OP(DEFINE_HIST_ENTRIES, f16, uint16_t)

/* ------------------------------------------------------------------ matmul */

static int do_bmm(struct futhark_context *ctx, fa_dtype in_t, struct fut_array **out, int rank,
                  const struct fut_array *A, const struct fut_array *B, const char *entry) {
  int64_t b = 1, M, K, K2, N;
  if (rank == 3) {
    b = A->shape[0];
    M = A->shape[1];
    K = A->shape[2];
    K2 = B->shape[1];
    N = B->shape[2];
    if (B->shape[0] != b) return bad_sizes(ctx, entry);
  } else {
    M = A->shape[0];
    K = A->shape[1];
    K2 = B->shape[0];
    N = B->shape[1];
  }
  if (K != K2) return bad_sizes(ctx, entry);
  const int64_t dims3[3] = {b, M, N}, dims2[2] = {M, N};
  struct fut_array *res =
      out_array(ctx, b * M * N * 4, rank, rank == 3 ? dims3 : dims2, "bmm.out");
  if (res == NULL) return FUTHARK_OUT_OF_MEMORY;
  struct memblock_device ws = {0};
  const size_t ws_bytes = fa_matmul_workspace_bytes(in_t, b, M, N, K);
  int err = 0;
  if (ws_bytes > 0) err = rts_memblock_alloc(ctx, &ws, (int64_t)ws_bytes, "bmm.workspace");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "segmap_matmul",
        rts_msgprintf("{\"batch\":%lld,\"M\":%lld,\"N\":%lld,\"K\":%lld,\"flop\":%lld,"
                      "\"padded\":%s}",
                      (long long)b, (long long)M, (long long)N, (long long)K,
                      (long long)(2 * b * M * N * K), ws_bytes > 0 ? "true" : "false"));
    int code = fa_matmul_ws(ctx->stream, in_t, A->mem.mem, B->mem.mem, (float *)res->mem.mem, b,
                            M, N, K, ws.mem, ws_bytes);
    err = rts_kernel_end(ctx, ev, "segmap_matmul", code);
  }
  rts_memblock_unref(ctx, &ws, "bmm.workspace");
  if (err != 0) {
    drop_array(ctx, res);
    return err;
  }
  *out = res;
  return 0;
}

int futhark_entry_bmm_f32(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                          const struct futhark_f32_3d *in0, const struct futhark_f32_3d *in1) {
  ENTER(ctx);
  int ret = do_bmm(ctx, FA_F32, (struct fut_array **)out0, 3, &in0->a, &in1->a, "bmm_f32");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_bmm_f16(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                          const struct futhark_f16_3d *in0, const struct futhark_f16_3d *in1) {
  ENTER(ctx);
  int ret = do_bmm(ctx, FA_F16, (struct fut_array **)out0, 3, &in0->a, &in1->a, "bmm_f16");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_bmm_bf16(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                           const struct futhark_u16_3d *in0, const struct futhark_u16_3d *in1) {
  ENTER(ctx);
  int ret = do_bmm(ctx, FA_BF16, (struct fut_array **)out0, 3, &in0->a, &in1->a, "bmm_bf16");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_matmul_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                             const struct futhark_f32_2d *in0, const struct futhark_f32_2d *in1) {
  ENTER(ctx);
  int ret = do_bmm(ctx, FA_F32, (struct fut_array **)out0, 2, &in0->a, &in1->a, "matmul_f32");
  LEAVE(ctx);
  return ret;
}

/* -------------------------------------------------------------- radix sort */

static int do_sort(struct futhark_context *ctx, int key_bytes, int val_bytes,
                   struct fut_array **out_keys, struct fut_array **out_vals,
                   const struct fut_array *keys, const struct fut_array *vals,
                   const char *entry) {
  const int64_t n = keys->shape[0];
  if (vals != NULL && vals->shape[0] != n) return bad_sizes(ctx, entry);
  struct fut_array *rk = out_array(ctx, n * key_bytes, 1, &n, "sort.keys");
  struct fut_array *rv = vals ? out_array(ctx, n * val_bytes, 1, &n, "sort.vals") : NULL;
  struct memblock_device tk = {0}, tv = {0}, scratch = {0};
  int err = (rk == NULL || (vals && rv == NULL)) ? FUTHARK_OUT_OF_MEMORY : 0;
  if (err == 0) err = rts_memblock_alloc(ctx, &tk, n * key_bytes, "sort.keys_tmp");
  if (err == 0 && vals) err = rts_memblock_alloc(ctx, &tv, n * val_bytes, "sort.vals_tmp");
  if (err == 0)
    err = rts_memblock_alloc(ctx, &scratch, (int64_t)fa_radix_sort_scratch_bytes(n),
                             "sort.scratch");
  if (err == 0) {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "radix_sort", rts_msgprintf("{\"n\":%lld,\"key_bytes\":%d,\"val_bytes\":%d}",
                                         (long long)n, key_bytes, val_bytes));
    int code = fa_radix_sort(ctx->stream, key_bytes, val_bytes, keys->mem.mem, rk->mem.mem,
                             tk.mem, vals ? vals->mem.mem : NULL, rv ? rv->mem.mem : NULL,
                             vals ? tv.mem : NULL, n, 0, key_bytes * 8, scratch.mem,
                             (size_t)scratch.size);
    err = rts_kernel_end(ctx, ev, "radix_sort", code);
  }
  rts_memblock_unref(ctx, &tk, "sort.keys_tmp");
  rts_memblock_unref(ctx, &tv, "sort.vals_tmp");
  rts_memblock_unref(ctx, &scratch, "sort.scratch");
  if (err != 0) {
    drop_array(ctx, rk);
    drop_array(ctx, rv);
    return err;
  }
  *out_keys = rk;
  if (out_vals) *out_vals = rv;
  return 0;
}

int futhark_entry_radix_sort_u32(struct futhark_context *ctx, struct futhark_u32_1d **out0,
                                 const struct futhark_u32_1d *in0) {
  ENTER(ctx);
  int ret = do_sort(ctx, 4, 0, (struct fut_array **)out0, NULL, &in0->a, NULL, "radix_sort_u32");
  LEAVE(ctx);
  return ret;
}
int futhark_entry_radix_sort_u64(struct futhark_context *ctx, struct futhark_u64_1d **out0,
                                 const struct futhark_u64_1d *in0) {
  ENTER(ctx);
  int ret = do_sort(ctx, 8, 0, (struct fut_array **)out0, NULL, &in0->a, NULL, "radix_sort_u64");
  LEAVE(ctx);
  return ret;
}
/* ------------------------------------------------- tuples of two arrays
 * An entry point has one result; a tuple result is an opaque record
 * (docs/c-api.rst:318-432) named after its type by
 * src/Futhark/CodeGen/Backends/SimpleRep.hs:144-186: ([]u32, []i32) is
 * futhark_opaque_tup2_arr1d_u32_arr1d_i32.  Components are held as array
 * values of their own (fields v0, v1); new and project hand out aliases with
 * their own lifetime (GenericC/Types.hs:280-446); store writes the components
 * one after the other in the binary data format and restore reads them back
 * (GenericC/Types.hs:1063-1135). */
static struct fut_array *array_alias(struct futhark_context *ctx, const struct fut_array *src) {
  struct fut_array *a = (struct fut_array *)malloc(sizeof(struct fut_array));
  if (a == NULL) return NULL;
  memcpy(a, src, sizeof(*a));
  pthread_mutex_lock(&ctx->lock);
  if (a->mem.references != NULL) (*a->mem.references)++;
  pthread_mutex_unlock(&ctx->lock);
  return a;
}

#define VALUE_HEADER_BYTES 7 /* 'b', version, rank, four type characters */
static unsigned char *put_header_1d(unsigned char *out, const char *tag, int64_t dim0) {
  *out++ = 'b';
  *out++ = 2;
  *out++ = 1;
  memcpy(out, tag, 4);
  out += 4;
  memcpy(out, &dim0, sizeof(int64_t));
  return out + sizeof(int64_t);
}
static const unsigned char *get_header_1d(const unsigned char *src, const char *tag,
                                          int64_t *dim0, int *err) {
  *err |= (src[0] != 'b') | (src[1] != 2) | (src[2] != 1) | (memcmp(src + 3, tag, 4) != 0);
  if (*err == 0) memcpy(dim0, src + VALUE_HEADER_BYTES, sizeof(int64_t));
  return src + VALUE_HEADER_BYTES + sizeof(int64_t);
}

#define DEFINE_TUP2(NAME, T0, CT0, TAG0, T1, CT1, TAG1)                                         \
  struct futhark_opaque_##NAME {                                                                \
    struct futhark_##T0##_1d *v0;                                                               \
    struct futhark_##T1##_1d *v1;                                                               \
  };                                                                                            \
  int futhark_free_opaque_##NAME(struct futhark_context *ctx,                                   \
                                 struct futhark_opaque_##NAME *obj) {                           \
    int ret = 0, tmp;                                                                           \
    if (obj->v0 != NULL && (tmp = futhark_free_##T0##_1d(ctx, obj->v0)) != 0) ret = tmp;        \
    if (obj->v1 != NULL && (tmp = futhark_free_##T1##_1d(ctx, obj->v1)) != 0) ret = tmp;        \
    free(obj);                                                                                  \
    return ret;                                                                                 \
  }                                                                                             \
  int futhark_store_opaque_##NAME(struct futhark_context *ctx,                                  \
                                  const struct futhark_opaque_##NAME *obj, void **p,            \
                                  size_t *n) {                                                  \
    int ret = 0;                                                                                \
    const int64_t n0 = obj->v0->a.shape[0], n1 = obj->v1->a.shape[0];                           \
    const int64_t size_0 = VALUE_HEADER_BYTES + 8 + n0 * (int64_t)sizeof(CT0);                  \
    const int64_t size_1 = VALUE_HEADER_BYTES + 8 + n1 * (int64_t)sizeof(CT1);                  \
    *n = (size_t)(size_0 + size_1);                                                             \
    if (p != NULL && *p == NULL) *p = malloc(*n);                                               \
    if (p != NULL) {                                                                            \
      unsigned char *out = (unsigned char *)*p;                                                 \
      if (out == NULL) return FUTHARK_OUT_OF_MEMORY;                                            \
      out = put_header_1d(out, TAG0, n0);                                                       \
      ret |= futhark_values_##T0##_1d(ctx, obj->v0, (CT0 *)(void *)out);                        \
      out += n0 * (int64_t)sizeof(CT0);                                                         \
      out = put_header_1d(out, TAG1, n1);                                                       \
      ret |= futhark_values_##T1##_1d(ctx, obj->v1, (CT1 *)(void *)out);                        \
    }                                                                                           \
    return ret;                                                                                 \
  }                                                                                             \
  struct futhark_opaque_##NAME *futhark_restore_opaque_##NAME(struct futhark_context *ctx,      \
                                                              const void *p) {                  \
    int err = 0;                                                                                \
    const unsigned char *src = (const unsigned char *)p;                                        \
    struct futhark_opaque_##NAME *obj = malloc(sizeof(*obj));                                   \
    if (obj == NULL) return NULL;                                                               \
    obj->v0 = NULL;                                                                             \
    obj->v1 = NULL;                                                                             \
    int64_t n0 = 0, n1 = 0;                                                                     \
    const unsigned char *data_0 = get_header_1d(src, TAG0, &n0, &err);                          \
    const unsigned char *data_1 = NULL;                                                         \
    if (err == 0 && n0 < 0) err = 1;                                                            \
    if (err == 0) data_1 = get_header_1d(data_0 + n0 * (int64_t)sizeof(CT0), TAG1, &n1, &err);  \
    if (err == 0 && n1 < 0) err = 1;                                                            \
    if (err == 0) {                                                                             \
      /* the bytes need not be aligned for CT0 / CT1: the copy is byte-wise */                  \
      obj->v0 = futhark_new_##T0##_1d(ctx, (const CT0 *)(const void *)data_0, n0);              \
      if (obj->v0 == NULL) err = 1;                                                             \
      obj->v1 = futhark_new_##T1##_1d(ctx, (const CT1 *)(const void *)data_1, n1);              \
      if (obj->v1 == NULL) err = 1;                                                             \
    }                                                                                           \
    if (err != 0) {                                                                             \
      futhark_free_opaque_##NAME(ctx, obj);                                                     \
      obj = NULL;                                                                               \
    }                                                                                           \
    return obj;                                                                                 \
  }                                                                                             \
  int futhark_new_opaque_##NAME(struct futhark_context *ctx, struct futhark_opaque_##NAME **out, \
                                const struct futhark_##T0##_1d *f_0,                            \
                                const struct futhark_##T1##_1d *f_1) {                          \
    struct futhark_opaque_##NAME *v = malloc(sizeof(*v));                                       \
    if (v == NULL) return FUTHARK_OUT_OF_MEMORY;                                                \
    v->v0 = (struct futhark_##T0##_1d *)array_alias(ctx, &f_0->a);                              \
    v->v1 = (struct futhark_##T1##_1d *)array_alias(ctx, &f_1->a);                              \
    if (v->v0 == NULL || v->v1 == NULL) {                                                       \
      futhark_free_opaque_##NAME(ctx, v);                                                       \
      return FUTHARK_OUT_OF_MEMORY;                                                             \
    }                                                                                           \
    *out = v;                                                                                   \
    return FUTHARK_SUCCESS;                                                                     \
  }                                                                                             \
  int futhark_project_opaque_##NAME##_0(struct futhark_context *ctx,                            \
                                        struct futhark_##T0##_1d **out,                         \
                                        const struct futhark_opaque_##NAME *obj) {              \
    struct fut_array *v = array_alias(ctx, &obj->v0->a);                                        \
    if (v == NULL) return FUTHARK_OUT_OF_MEMORY;                                                \
    *out = (struct futhark_##T0##_1d *)v;                                                       \
    return 0;                                                                                   \
  }                                                                                             \
  int futhark_project_opaque_##NAME##_1(struct futhark_context *ctx,                            \
                                        struct futhark_##T1##_1d **out,                         \
                                        const struct futhark_opaque_##NAME *obj) {              \
    struct fut_array *v = array_alias(ctx, &obj->v1->a);                                        \
    if (v == NULL) return FUTHARK_OUT_OF_MEMORY;                                                \
    *out = (struct futhark_##T1##_1d *)v;                                                       \
    return 0;                                                                                   \
  }                                                                                             \
  int futhark_entry_radix_sort_pairs_##T0##_##T1(struct futhark_context *ctx,                   \
                                                 struct futhark_opaque_##NAME **out0,           \
                                                 const struct futhark_##T0##_1d *in0,           \
                                                 const struct futhark_##T1##_1d *in1) {         \
    struct futhark_opaque_##NAME *v = malloc(sizeof(*v));                                       \
    if (v == NULL) return FUTHARK_OUT_OF_MEMORY;                                                \
    ENTER(ctx);                                                                                 \
    int ret = do_sort(ctx, (int)sizeof(CT0), (int)sizeof(CT1), (struct fut_array **)&v->v0,     \
                      (struct fut_array **)&v->v1, &in0->a, &in1->a,                            \
                      "radix_sort_pairs_" #T0 "_" #T1);                                         \
    LEAVE(ctx);                                                                                 \
    if (ret != 0) {                                                                             \
      free(v); /* on error the out-parameter is not touched */                                  \
      return ret;                                                                               \
    }                                                                                           \
    *out0 = v;                                                                                  \
    return 0;                                                                                   \
  }

DEFINE_TUP2(tup2_arr1d_u32_arr1d_i32, u32, uint32_t, " u32", i32, int32_t, " i32")
DEFINE_TUP2(tup2_arr1d_u64_arr1d_i32, u64, uint64_t, " u64", i32, int32_t, " i32")

int futhark_entry_transpose_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                                const struct futhark_f32_2d *in0) {
  ENTER(ctx);
  const int64_t rows = in0->a.shape[0], cols = in0->a.shape[1];
  const int64_t dims[2] = {cols, rows};
  int ret = 0;
  struct fut_array *res = out_array(ctx, rows * cols * 4, 2, dims, "transpose.out");
  if (res == NULL) {
    ret = FUTHARK_OUT_OF_MEMORY;
  } else {
    struct rts_event *ev = rts_kernel_begin(
        ctx, "map_transpose_4b",
        rts_msgprintf("{\"rows\":%lld,\"cols\":%lld}", (long long)rows, (long long)cols));
    int code = fa_map_transpose(ctx->stream, 4, res->mem.mem, in0->a.mem.mem, 1, rows, cols);
    ret = rts_kernel_end(ctx, ev, "map_transpose_4b", code);
    if (ret != 0) drop_array(ctx, res);
    else *out0 = (struct futhark_f32_2d *)res;
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_iota_i64(struct futhark_context *ctx, struct futhark_i64_1d **out0,
                           const int64_t in0) {
  ENTER(ctx);
  int ret = 0;
  if (in0 < 0) {
    rts_set_error(ctx, rts_msgprintf("Error: Range 0..<%lld is invalid.\n", (long long)in0));
    ret = FUTHARK_PROGRAM_ERROR;
  } else {
    struct fut_array *res = out_array(ctx, in0 * 8, 1, &in0, "iota.out");
    if (res == NULL) {
      ret = FUTHARK_OUT_OF_MEMORY;
    } else {
      int code = fa_iota(ctx->stream, FA_I64, res->mem.mem, in0, 0, 1);
      ret = rts_kernel_end(ctx, NULL, "iota_i64", code);
      if (ret != 0) drop_array(ctx, res);
      else *out0 = (struct futhark_i64_1d *)res;
    }
  }
  LEAVE(ctx);
  return ret;
}

int futhark_entry_replicate_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                const int64_t in0, const int32_t in1) {
  ENTER(ctx);
  int ret = 0;
  if (in0 < 0) {
    rts_set_error(ctx, rts_msgprintf("Error: negative size %lld.\n", (long long)in0));
    ret = FUTHARK_PROGRAM_ERROR;
  } else {
    struct fut_array *res = out_array(ctx, in0 * 4, 1, &in0, "replicate.out");
    if (res == NULL) {
      ret = FUTHARK_OUT_OF_MEMORY;
    } else {
      int code = fa_replicate(ctx->stream, 4, res->mem.mem, in0, (uint32_t)in1);
      ret = rts_kernel_end(ctx, NULL, "replicate_i32", code);
      if (ret != 0) drop_array(ctx, res);
      else *out0 = (struct futhark_i32_1d *)res;
    }
  }
  LEAVE(ctx);
  return ret;
}

void *futhark_context_get_stream(struct futhark_context *ctx) { return ctx->stream; }
