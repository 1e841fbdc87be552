/* The `segops` program as the executables see it: its types with uniform
 * shims over the per-type array API, and its entry points with their argument
 * types, consumption and tuning parameters -- the information
 * src/Futhark/CodeGen/Backends/GenericC/{Server,CLI}.hs take from the manifest
 * when they generate the server and the command-line executable.  Included by
 * server.c and cli.c; everything here is static. */
#ifndef SEGOPS_PROGRAM_TABLE_H
#define SEGOPS_PROGRAM_TABLE_H

#include <stdint.h>
#include <string.h>

#include "segops.h"

/* ------------------------------------------------------------------ types */

enum kind { K_PRIMITIVE, K_ARRAY, K_RECORD };

struct stype;
typedef void *(*arr_new_fn)(struct futhark_context *, const void *, const int64_t *);
typedef int (*arr_free_fn)(struct futhark_context *, void *);
typedef int (*arr_values_fn)(struct futhark_context *, void *, void *);
typedef const int64_t *(*arr_shape_fn)(struct futhark_context *, void *);
typedef int (*arr_index_fn)(struct futhark_context *, void *, void *, const int64_t *);

struct stype {
  const char *name; /* Futhark syntax without sizes: "f32", "[]f32", "([]u32, []i32)" */
  enum kind kind;
  const char *prim; /* element (or scalar) type name for values.c */
  int rank;
  arr_new_fn arr_new;
  arr_free_fn arr_free;
  arr_values_fn arr_values;
  arr_shape_fn arr_shape;
  arr_index_fn arr_index;
  int num_fields; /* records */
  const char *field_names[2];
  const char *field_types[2];
};

/* Uniform-signature shims over the per-type array API. */
#define ARRAY_SHIMS_1D(N, CT)                                                                \
  static void *new_##N##_1d(struct futhark_context *c, const void *d, const int64_t *s) {    \
    return futhark_new_##N##_1d(c, (const CT *)d, s[0]);                                     \
  }                                                                                          \
  static int index_##N##_1d(struct futhark_context *c, void *o, void *a, const int64_t *i) { \
    return futhark_index_##N##_1d(c, (CT *)o, a, i[0]);                                      \
  }
#define ARRAY_SHIMS_2D(N, CT)                                                                \
  static void *new_##N##_2d(struct futhark_context *c, const void *d, const int64_t *s) {    \
    return futhark_new_##N##_2d(c, (const CT *)d, s[0], s[1]);                               \
  }                                                                                          \
  static int index_##N##_2d(struct futhark_context *c, void *o, void *a, const int64_t *i) { \
    return futhark_index_##N##_2d(c, (CT *)o, a, i[0], i[1]);                                \
  }
#define ARRAY_SHIMS_3D(N, CT)                                                                \
  static void *new_##N##_3d(struct futhark_context *c, const void *d, const int64_t *s) {    \
    return futhark_new_##N##_3d(c, (const CT *)d, s[0], s[1], s[2]);                         \
  }                                                                                          \
  static int index_##N##_3d(struct futhark_context *c, void *o, void *a, const int64_t *i) { \
    return futhark_index_##N##_3d(c, (CT *)o, a, i[0], i[1], i[2]);                          \
  }
#define ARRAY_SHIMS_COMMON(N, R)                                                             \
  static int free_##N##_##R(struct futhark_context *c, void *a) {                            \
    return futhark_free_##N##_##R(c, a);                                                     \
  }                                                                                          \
  static int values_##N##_##R(struct futhark_context *c, void *a, void *o) {                 \
    return futhark_values_##N##_##R(c, a, o);                                                \
  }                                                                                          \
  static const int64_t *shape_##N##_##R(struct futhark_context *c, void *a) {                \
    return futhark_shape_##N##_##R(c, a);                                                    \
  }
#define A1(N, CT) ARRAY_SHIMS_1D(N, CT) ARRAY_SHIMS_COMMON(N, 1d)
#define A2(N, CT) ARRAY_SHIMS_2D(N, CT) ARRAY_SHIMS_COMMON(N, 2d)
#define A3(N, CT) ARRAY_SHIMS_3D(N, CT) ARRAY_SHIMS_COMMON(N, 3d)
A1(i32, int32_t) A1(i64, int64_t) A1(u8, uint8_t) A1(u32, uint32_t) A1(u64, uint64_t)
A1(f32, float) A1(f64, double)
A1(i8, int8_t) A1(i16, int16_t) A1(u16, uint16_t) A1(f16, uint16_t)
A2(i32, int32_t) A2(i64, int64_t) A2(f32, float) A2(f64, double)
A3(f32, float) A3(f16, uint16_t) A3(u16, uint16_t)

#define PRIM(N) {N, K_PRIMITIVE, N, 0, NULL, NULL, NULL, NULL, NULL, 0, {0}, {0}}
#define ARR(NAME, P, R, N, S) \
  {NAME, K_ARRAY, P, R, new_##N##_##S, free_##N##_##S, values_##N##_##S, shape_##N##_##S, \
   index_##N##_##S, 0, {0}, {0}}
#define PAIR(NAME, T0, T1) \
  {NAME, K_RECORD, NULL, 0, NULL, NULL, NULL, NULL, NULL, 2, {"0", "1"}, {T0, T1}}

static const struct stype types[] = {
    PRIM("i32"), PRIM("i64"), PRIM("f32"), PRIM("f64"),
    ARR("[]i32", "i32", 1, i32, 1d), ARR("[]i64", "i64", 1, i64, 1d),
    ARR("[]u8", "u8", 1, u8, 1d), ARR("[]u32", "u32", 1, u32, 1d),
    ARR("[]u64", "u64", 1, u64, 1d), ARR("[]f32", "f32", 1, f32, 1d),
    ARR("[]f64", "f64", 1, f64, 1d),
    ARR("[]i8", "i8", 1, i8, 1d), ARR("[]i16", "i16", 1, i16, 1d),
    ARR("[]u16", "u16", 1, u16, 1d), ARR("[]f16", "f16", 1, f16, 1d),
    ARR("[][]i32", "i32", 2, i32, 2d), ARR("[][]i64", "i64", 2, i64, 2d),
    ARR("[][]f32", "f32", 2, f32, 2d), ARR("[][]f64", "f64", 2, f64, 2d),
    ARR("[][][]f32", "f32", 3, f32, 3d), ARR("[][][]f16", "f16", 3, f16, 3d),
    ARR("[][][]u16", "u16", 3, u16, 3d),
    PAIR("([]u32, []i32)", "[]u32", "[]i32"), PAIR("([]u64, []i32)", "[]u64", "[]i32"),
};
#define NUM_TYPES ((int)(sizeof(types) / sizeof(types[0])))

static const struct stype *find_type(const char *name) {
  for (int i = 0; i < NUM_TYPES; i++)
    if (strcmp(types[i].name, name) == 0) return &types[i];
  return NULL;
}

/* ----------------------------------------------------------------- values */

struct variable;
struct value {
  const struct stype *type;
  union {
    int32_t i32;
    int64_t i64;
    float f32;
    double f64;
    unsigned char bytes[8];
    void *arr;
    struct variable *fields[2]; /* records own anonymous variables */
  } u;
};

struct variable {
  char *name; /* NULL for the anonymous fields of a record */
  struct value value;
  struct variable *next;
};

/* ------------------------------------------------------------ entry points */

typedef int (*entry_fn)(struct futhark_context *, struct value *out, struct value **ins);

#define ENTRY_MAX_INPUTS 4 /* most inputs any entry point of the program takes */

struct entry {
  const char *name;
  entry_fn f;
  const char *out_type;
  int out_unique;
  int num_ins;
  const char *in_types[ENTRY_MAX_INPUTS];
  int in_consumed[ENTRY_MAX_INPUTS];
  const char *tuning_params[3]; /* NULL terminated */
};

#define ARRP(v) ((v)->u.arr)
#define SEGOP_ENTRY_FNS(OP, T, CT)                                                             \
  static int e_reduce_##OP##_##T(struct futhark_context *c, struct value *o,                   \
                                 struct value **i) {                                           \
    return futhark_entry_reduce_##OP##_##T(c, (CT *)o->u.bytes, ARRP(i[0]));                   \
  }                                                                                            \
  static int e_scan_##OP##_##T(struct futhark_context *c, struct value *o, struct value **i) { \
    return futhark_entry_scan_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,             \
                                         ARRP(i[0]));                                          \
  }                                                                                            \
  static int e_exscan_##OP##_##T(struct futhark_context *c, struct value *o,                   \
                                 struct value **i) {                                           \
    return futhark_entry_exscan_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,           \
                                           ARRP(i[0]));                                        \
  }                                                                                            \
  static int e_segscan_##OP##_##T(struct futhark_context *c, struct value *o,                  \
                                  struct value **i) {                                          \
    return futhark_entry_segscan_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,          \
                                            ARRP(i[0]), ARRP(i[1]));                           \
  }                                                                                            \
  static int e_segred_##OP##_##T(struct futhark_context *c, struct value *o,                   \
                                 struct value **i) {                                           \
    return futhark_entry_segred_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,           \
                                           ARRP(i[0]), ARRP(i[1]), ARRP(i[2]));                \
  }                                                                                            \
  static int e_segreduce_##OP##_##T(struct futhark_context *c, struct value *o,                \
                                    struct value **i) {                                        \
    return futhark_entry_segreduce_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,        \
                                              ARRP(i[0]));                                     \
  }                                                                                            \
  static int e_vecreduce_##OP##_##T(struct futhark_context *c, struct value *o,                \
                                    struct value **i) {                                        \
    return futhark_entry_vecreduce_##OP##_##T(c, (struct futhark_##T##_1d **)&o->u.arr,        \
                                              ARRP(i[0]));                                     \
  }                                                                                            \
  static int e_scanrows_##OP##_##T(struct futhark_context *c, struct value *o,                 \
                                   struct value **i) {                                         \
    return futhark_entry_scanrows_##OP##_##T(c, (struct futhark_##T##_2d **)&o->u.arr,         \
                                             ARRP(i[0]));                                      \
  }                                                                                            \
  static int e_vecscan_##OP##_##T(struct futhark_context *c, struct value *o,                  \
                                  struct value **i) {                                          \
    return futhark_entry_vecscan_##OP##_##T(c, (struct futhark_##T##_2d **)&o->u.arr,          \
                                            ARRP(i[0]));                                       \
  }                                                                                            \
  static int e_seghist_##OP##_##T(struct futhark_context *c, struct value *o,                  \
                                  struct value **i) {                                          \
    return futhark_entry_seghist_##OP##_##T(c, (struct futhark_##T##_2d **)&o->u.arr,          \
                                            i[0]->u.i64, ARRP(i[1]), ARRP(i[2]));              \
  }                                                                                            \
  static int e_rbi_vec_##OP##_##T(struct futhark_context *c, struct value *o,                  \
                                  struct value **i) {                                          \
    return futhark_entry_rbi_vec_##OP##_##T(c, (struct futhark_##T##_2d **)&o->u.arr,          \
                                            ARRP(i[0]), ARRP(i[1]), ARRP(i[2]));               \
  }                                                                                            \
  static int e_rbi_2d_##OP##_##T(struct futhark_context *c, struct value *o,                   \
                                 struct value **i) {                                           \
    return futhark_entry_rbi_2d_##OP##_##T(c, (struct futhark_##T##_2d **)&o->u.arr,           \
                                           ARRP(i[0]), ARRP(i[1]), ARRP(i[2]), ARRP(i[3]));    \
  }                                                                                            \
  HIST_ENTRY_FNS(OP, T, CT)
#define HIST_ENTRY_FNS(OP, T, CT) HIST_ENTRY_FNS_IX(OP, T, CT, ) HIST_ENTRY_FNS_IX(OP, T, CT, _i64)
#define HIST_ENTRY_FNS_IX(OP, T, CT, SUFFIX)                                                   \
  static int e_hist_##OP##_##T##SUFFIX(struct futhark_context *c, struct value *o,             \
                                       struct value **i) {                                     \
    return futhark_entry_hist_##OP##_##T##SUFFIX(c, (struct futhark_##T##_1d **)&o->u.arr,     \
                                                 i[0]->u.i64, ARRP(i[1]), ARRP(i[2]));         \
  }                                                                                            \
  static int e_rbi_##OP##_##T##SUFFIX(struct futhark_context *c, struct value *o,              \
                                      struct value **i) {                                      \
    return futhark_entry_rbi_##OP##_##T##SUFFIX(c, (struct futhark_##T##_1d **)&o->u.arr,      \
                                                ARRP(i[0]), ARRP(i[1]), ARRP(i[2]));           \
  }
#define SEGOP_ENTRY_FNS_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_OP(SEGOP_ENTRY_FNS, T, CT)
FUTHARK_FOR_EACH_NUM_TYPE(SEGOP_ENTRY_FNS_FOR_TYPE)
#define SEGOP_BITOP_FNS_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_BITOP(SEGOP_ENTRY_FNS, T, CT)
FUTHARK_FOR_EACH_INT_TYPE(SEGOP_BITOP_FNS_FOR_TYPE)
#define HIST_ONLY_INT_FNS(T, CT) \
  FUTHARK_FOR_EACH_OP(HIST_ENTRY_FNS, T, CT) FUTHARK_FOR_EACH_BITOP(HIST_ENTRY_FNS, T, CT)
FUTHARK_FOR_EACH_HIST_ONLY_INT_TYPE(HIST_ONLY_INT_FNS)
FUTHARK_FOR_EACH_OP(HIST_ENTRY_FNS, f16, uint16_t)

static int e_bmm_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_bmm_f32(c, (struct futhark_f32_3d **)&o->u.arr, ARRP(i[0]), ARRP(i[1]));
}
static int e_bmm_f16(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_bmm_f16(c, (struct futhark_f32_3d **)&o->u.arr, ARRP(i[0]), ARRP(i[1]));
}
static int e_scan_compose_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_scan_compose_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_exscan_compose_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_exscan_compose_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_reduce_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_reduce_argmax_i32(c, (struct futhark_i32_1d **)&o->u.arr, ARRP(i[0]));
}
static int e_scan_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_scan_argmax_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_hist_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_hist_argmax_i32(c, (struct futhark_i32_2d **)&o->u.arr, i[0]->u.i64,
                                       ARRP(i[1]), ARRP(i[2]));
}
static int e_reduce_compose_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_reduce_compose_i32(c, (struct futhark_i32_1d **)&o->u.arr, ARRP(i[0]));
}
static int e_sumsq_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_sumsq_f32(c, &o->u.f32, ARRP(i[0]));
}
static int e_segreduce_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_segreduce_argmax_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_segreduce_compose_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_segreduce_compose_i32(c, (struct futhark_i32_2d **)&o->u.arr, i[0]->u.i64,
                                             ARRP(i[1]));
}
static int e_scanrows_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_scanrows_argmax_i32(c, (struct futhark_i32_2d **)&o->u.arr, i[0]->u.i64,
                                           ARRP(i[1]));
}
static int e_segred_argmax_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_segred_argmax_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]),
                                         ARRP(i[1]), ARRP(i[2]));
}
static int e_rows_fraction_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_rows_fraction_f32(c, (struct futhark_f32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_reduce_summax_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_reduce_summax_f32(c, (struct futhark_f32_1d **)&o->u.arr, ARRP(i[0]));
}
static int e_scan_norm_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_scan_norm_f32(c, (struct futhark_f32_1d **)&o->u.arr, ARRP(i[0]));
}
static int e_segscan_compose_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_segscan_compose_i32(c, (struct futhark_i32_2d **)&o->u.arr, ARRP(i[0]),
                                           ARRP(i[1]));
}
static int e_bmm_bf16(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_bmm_bf16(c, (struct futhark_f32_3d **)&o->u.arr, ARRP(i[0]), ARRP(i[1]));
}
static int e_matmul_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_matmul_f32(c, (struct futhark_f32_2d **)&o->u.arr, ARRP(i[0]),
                                  ARRP(i[1]));
}
static int e_radix_sort_u32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_radix_sort_u32(c, (struct futhark_u32_1d **)&o->u.arr, ARRP(i[0]));
}
static int e_radix_sort_u64(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_radix_sort_u64(c, (struct futhark_u64_1d **)&o->u.arr, ARRP(i[0]));
}
/* The tuple result arrives as one opaque value; the server keeps records as
 * their fields, so it projects both and lets the tuple go. */
#define SORT_PAIRS_ENTRY_FN(NAME, K, V)                                                         \
  static int e_radix_sort_pairs_##K##_##V(struct futhark_context *c, struct value *o,           \
                                          struct value **i) {                                   \
    struct futhark_opaque_##NAME *t = NULL;                                                     \
    int ret = futhark_entry_radix_sort_pairs_##K##_##V(c, &t, ARRP(i[0]), ARRP(i[1]));          \
    if (ret != 0) return ret;                                                                   \
    ret = futhark_project_opaque_##NAME##_0(                                                    \
        c, (struct futhark_##K##_1d **)&o->u.fields[0]->value.u.arr, t);                        \
    if (ret == 0)                                                                               \
      ret = futhark_project_opaque_##NAME##_1(                                                  \
          c, (struct futhark_##V##_1d **)&o->u.fields[1]->value.u.arr, t);                      \
    int tmp = futhark_free_opaque_##NAME(c, t);                                                 \
    return ret != 0 ? ret : tmp;                                                                \
  }
SORT_PAIRS_ENTRY_FN(tup2_arr1d_u32_arr1d_i32, u32, i32)
SORT_PAIRS_ENTRY_FN(tup2_arr1d_u64_arr1d_i32, u64, i32)
static int e_transpose_f32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_transpose_f32(c, (struct futhark_f32_2d **)&o->u.arr, ARRP(i[0]));
}
static int e_iota_i64(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_iota_i64(c, (struct futhark_i64_1d **)&o->u.arr, i[0]->u.i64);
}
static int e_replicate_i32(struct futhark_context *c, struct value *o, struct value **i) {
  return futhark_entry_replicate_i32(c, (struct futhark_i32_1d **)&o->u.arr, i[0]->u.i64,
                                     i[1]->u.i32);
}

#define HIST_PARAM "segops.hist_lds_bins_max"
#define SEGRED_PARAM "segops.segred_small_threshold"
#define MATMUL_PARAM "segops.matmul_pad_min_work"
#define SCAN_PARAM "segops.scan_arrival_tickets"
#define SORT_PARAM "segops.sort_wide_positions"
#define SEGOP_ENTRY_ROWS(OP, T, CT)                                                             \
  {"reduce_" #OP "_" #T, e_reduce_##OP##_##T, #T, 0, 1, {"[]" #T}, {0}, {NULL}},                \
  {"scan_" #OP "_" #T, e_scan_##OP##_##T, "[]" #T, 1, 1, {"[]" #T}, {0}, {SCAN_PARAM, NULL}},   \
  {"exscan_" #OP "_" #T, e_exscan_##OP##_##T, "[]" #T, 1, 1, {"[]" #T}, {0},                    \
   {SCAN_PARAM, NULL}},                                                                         \
  {"segscan_" #OP "_" #T, e_segscan_##OP##_##T, "[]" #T, 1, 2, {"[]u8", "[]" #T}, {0},          \
   {SCAN_PARAM, NULL}},                                                                         \
  {"segred_" #OP "_" #T, e_segred_##OP##_##T, "[]" #T, 1, 3, {"[]i64", "[]i64", "[]" #T},       \
   {0}, {NULL}},                                                                                \
  {"segreduce_" #OP "_" #T, e_segreduce_##OP##_##T, "[]" #T, 1, 1, {"[][]" #T}, {0},            \
   {SEGRED_PARAM, NULL}},                                                                       \
  {"vecreduce_" #OP "_" #T, e_vecreduce_##OP##_##T, "[]" #T, 1, 1, {"[][]" #T}, {0}, {NULL}},   \
  {"scanrows_" #OP "_" #T, e_scanrows_##OP##_##T, "[][]" #T, 1, 1, {"[][]" #T}, {0},            \
   {SCAN_PARAM, NULL}},                                                                         \
  {"vecscan_" #OP "_" #T, e_vecscan_##OP##_##T, "[][]" #T, 1, 1, {"[][]" #T}, {0}, {NULL}},     \
  {"seghist_" #OP "_" #T, e_seghist_##OP##_##T, "[][]" #T, 1, 3,                                \
   {"i64", "[][]i32", "[][]" #T}, {0}, {HIST_PARAM, NULL}},                                     \
  {"rbi_vec_" #OP "_" #T, e_rbi_vec_##OP##_##T, "[][]" #T, 1, 3,                                \
   {"[][]" #T, "[]i64", "[][]" #T}, {1, 0, 0}, {HIST_PARAM, NULL}},                             \
  {"rbi_2d_" #OP "_" #T, e_rbi_2d_##OP##_##T, "[][]" #T, 1, 4,                                  \
   {"[][]" #T, "[]i64", "[]i64", "[]" #T}, {1, 0, 0, 0}, {HIST_PARAM, NULL}},                   \
  HIST_ENTRY_ROWS(OP, T, CT)
#define HIST_ENTRY_ROWS(OP, T, CT) \
  HIST_ENTRY_ROWS_IX(OP, T, CT, , "[]i32") HIST_ENTRY_ROWS_IX(OP, T, CT, _i64, "[]i64")
#define HIST_ENTRY_ROWS_IX(OP, T, CT, SUFFIX, IXT)                                              \
  {"hist_" #OP "_" #T #SUFFIX, e_hist_##OP##_##T##SUFFIX, "[]" #T, 1, 3,                        \
   {"i64", IXT, "[]" #T}, {0}, {HIST_PARAM, NULL}},                                             \
  {"rbi_" #OP "_" #T #SUFFIX, e_rbi_##OP##_##T##SUFFIX, "[]" #T, 1, 3,                          \
   {"[]" #T, IXT, "[]" #T}, {1, 0, 0}, {HIST_PARAM, NULL}},
#define SEGOP_ENTRY_ROWS_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_OP(SEGOP_ENTRY_ROWS, T, CT)
#define SEGOP_BITOP_ROWS_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_BITOP(SEGOP_ENTRY_ROWS, T, CT)
#define HIST_ONLY_INT_ROWS(T, CT) \
  FUTHARK_FOR_EACH_OP(HIST_ENTRY_ROWS, T, CT) FUTHARK_FOR_EACH_BITOP(HIST_ENTRY_ROWS, T, CT)

static const struct entry entries[] = {
    FUTHARK_FOR_EACH_NUM_TYPE(SEGOP_ENTRY_ROWS_FOR_TYPE)
    FUTHARK_FOR_EACH_INT_TYPE(SEGOP_BITOP_ROWS_FOR_TYPE)
    FUTHARK_FOR_EACH_HIST_ONLY_INT_TYPE(HIST_ONLY_INT_ROWS)
    FUTHARK_FOR_EACH_OP(HIST_ENTRY_ROWS, f16, uint16_t)
    {"bmm_f32", e_bmm_f32, "[][][]f32", 1, 2, {"[][][]f32", "[][][]f32"}, {0}, {MATMUL_PARAM, NULL}},
    {"bmm_f16", e_bmm_f16, "[][][]f32", 1, 2, {"[][][]f16", "[][][]f16"}, {0}, {MATMUL_PARAM, NULL}},
    {"scan_compose_i32", e_scan_compose_i32, "[][]i32", 1, 1, {"[][]i32"}, {0}, {SCAN_PARAM, NULL}},
    {"exscan_compose_i32", e_exscan_compose_i32, "[][]i32", 1, 1, {"[][]i32"}, {0},
     {SCAN_PARAM, NULL}},
    {"segscan_compose_i32", e_segscan_compose_i32, "[][]i32", 1, 2, {"[]u8", "[][]i32"}, {0},
     {SCAN_PARAM, NULL}},
    {"reduce_argmax_i32", e_reduce_argmax_i32, "[]i32", 1, 1, {"[]i32"}, {0}, {NULL}},
    {"scan_argmax_i32", e_scan_argmax_i32, "[][]i32", 1, 1, {"[][]i32"}, {0}, {NULL}},
    {"hist_argmax_i32", e_hist_argmax_i32, "[][]i32", 1, 3, {"i64", "[]i32", "[]i32"}, {0}, {NULL}},
    {"reduce_compose_i32", e_reduce_compose_i32, "[]i32", 1, 1, {"[][]i32"}, {0}, {NULL}},
    {"sumsq_f32", e_sumsq_f32, "f32", 0, 1, {"[]f32"}, {0}, {NULL}},
    {"scan_norm_f32", e_scan_norm_f32, "[]f32", 1, 1, {"[]f32"}, {0}, {NULL}},
    {"reduce_summax_f32", e_reduce_summax_f32, "[]f32", 1, 1, {"[]f32"}, {0}, {NULL}},
    {"rows_fraction_f32", e_rows_fraction_f32, "[][]f32", 1, 1, {"[][]f32"}, {0}, {NULL}},
    {"segreduce_argmax_i32", e_segreduce_argmax_i32, "[][]i32", 1, 1, {"[][]i32"}, {0}, {NULL}},
    {"segreduce_compose_i32", e_segreduce_compose_i32, "[][]i32", 1, 2, {"i64", "[][]i32"}, {0},
     {NULL}},
    {"scanrows_argmax_i32", e_scanrows_argmax_i32, "[][]i32", 1, 2, {"i64", "[][]i32"}, {0}, {NULL}},
    {"segred_argmax_i32", e_segred_argmax_i32, "[][]i32", 1, 3, {"[]i64", "[]i64", "[][]i32"}, {0},
     {NULL}},
    {"bmm_bf16", e_bmm_bf16, "[][][]f32", 1, 2, {"[][][]u16", "[][][]u16"}, {0}, {MATMUL_PARAM, NULL}},
    {"matmul_f32", e_matmul_f32, "[][]f32", 1, 2, {"[][]f32", "[][]f32"}, {0}, {MATMUL_PARAM, NULL}},
    {"radix_sort_u32", e_radix_sort_u32, "[]u32", 1, 1, {"[]u32"}, {0}, {SORT_PARAM, NULL}},
    {"radix_sort_u64", e_radix_sort_u64, "[]u64", 1, 1, {"[]u64"}, {0}, {SORT_PARAM, NULL}},
    {"radix_sort_pairs_u32_i32", e_radix_sort_pairs_u32_i32, "([]u32, []i32)", 1, 2,
     {"[]u32", "[]i32"}, {0}, {SORT_PARAM, NULL}},
    {"radix_sort_pairs_u64_i32", e_radix_sort_pairs_u64_i32, "([]u64, []i32)", 1, 2,
     {"[]u64", "[]i32"}, {0}, {SORT_PARAM, NULL}},
    {"transpose_f32", e_transpose_f32, "[][]f32", 1, 1, {"[][]f32"}, {0}, {NULL}},
    {"iota_i64", e_iota_i64, "[]i64", 1, 1, {"i64"}, {0}, {NULL}},
    {"replicate_i32", e_replicate_i32, "[]i32", 1, 2, {"i64", "i32"}, {0}, {NULL}},
};
#define NUM_ENTRIES ((int)(sizeof(entries) / sizeof(entries[0])))

static const struct entry *find_entry(const char *name) {
  for (int i = 0; i < NUM_ENTRIES; i++)
    if (strcmp(entries[i].name, name) == 0) return &entries[i];
  return NULL;
}

#endif
