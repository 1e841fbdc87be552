/*
 * segops.h -- public C API of the `segops` program library (libsegops.so), in
 * the shape `futhark hip --library` gives every compiled program
 * (docs/c-api.rst; header layout src/Futhark/CodeGen/Backends/GenericC.hs:390-424;
 * array functions GenericC/Types.hs:159-240; entry points
 * GenericC/EntryPoints.hs:133-208).  A C caller written against a Futhark
 * library with these entry points links against this one unchanged.
 *
 * The Futhark source each entry point stands for:
 *
 *   entry reduce_OP_T  (xs: []T) : T           = reduce OP NE xs
 *   entry scan_OP_T    (xs: []T) : []T         = scan OP NE xs
 *   entry exscan_OP_T  (xs: []T) : []T         -- prelude/soacs.fut:212-215
 *   entry segscan_OP_T (flags: []u8) (vs: []T) : []T =
 *     (unzip (scan (\(fx,x) (fy,y) -> (fx || fy, if fy then y else x `OP` y))
 *                  (false,NE) (zip (map (!=0) flags) vs))).1
 *                                   -- Pass/Flatten/Builtins.hs:374-401
 *   entry segred_OP_T [m] (offsets: [m]i64) (lens: [m]i64) (vs: []T) : [m]T =
 *     let flags = scatter (replicate n false) offsets (replicate m true)
 *     let s = segscan OP NE flags vs
 *     in map2 (\o l -> if l == 0 then NE else s[o+l-1]) offsets lens
 *                                   -- Builtins.hs:570-602
 *   entry segreduce_OP_T (xss: [][]T) : []T    = map (reduce OP NE) xss
 *   entry vecreduce_OP_T (xss: [n][k]T) : [k]T = reduce (map2 OP) (replicate k NE) xss
 *   entry scanrows_OP_T (xss: [][]T) : [][]T   = map (scan OP NE) xss
 *   entry vecscan_OP_T (xss: [n][k]T) : [n][k]T = scan (map2 OP) (replicate k NE) xss
 *   entry hist_OP_T (k: i64) (is: []i32) (vs: []T) : [k]T =
 *     hist OP NE k (map i64.i32 is) vs           -- prelude/soacs.fut:132-146
 *   entry seghist_OP_T (k: i64) (iss: [][]i32) (vss: [][]T) : [][]T =
 *     map2 (\is vs -> hist OP NE k (map i64.i32 is) vs) iss vss
 *                                   -- tests/hist/segmented.fut
 *   entry rbi_OP_T (dest: *[]T) (is: []i32) (vs: []T) : []T =
 *     reduce_by_index dest OP NE (map i64.i32 is) vs
 *   entry hist_OP_T_i64 (k: i64) (is: []i64) (vs: []T) : [k]T = hist OP NE k is vs
 *   entry rbi_OP_T_i64 (dest: *[]T) (is: []i64) (vs: []T) : []T =
 *     reduce_by_index dest OP NE is vs           -- the index type of the prelude
 *   entry rbi_vec_OP_T [m] (dest: *[][m]T) (is: []i64) (vss: [][m]T) : [][m]T =
 *     reduce_by_index dest (map2 OP) (replicate m NE) is vss
 *   entry rbi_2d_OP_T (dest: *[][]T) (is: []i64) (js: []i64) (vs: []T) : [][]T =
 *     reduce_by_index_2d dest OP NE (zip is js) vs
 *   entry bmm_f32 (A: [][][]f32) (B: [][][]f32) : [][][]f32 =
 *     map2 (\a b -> map (\ar -> map (\bc -> reduce (+) 0 (map2 (*) ar bc))
 *                                   (transpose b)) a) A B
 *                                   -- tests/reg-tiling/mmm.fut:17-21, batched
 *   entry bmm_f16: the same with f16 inputs, products and sums in f32
 *   entry bmm_bf16: [][][]u16 inputs, x -> f32.from_bits (u32.u16 x << 16)
 *   entry radix_sort_T (keys: []T) : []T       -- 8-bit LSD passes, stable
 *   entry radix_sort_pairs_K_V (keys: []K) (vals: []V) : ([]K, []V)
 *                                  -- one opaque result, see "Opaque" below
 *   entry transpose_f32 (xss: [][]f32) : [][]f32 = transpose xss
 *
 * OP in {add, max, min}; NE = 0, T.lowest, T.highest; T in {i32, i64, f32, f64};
 * for T in {i32, i64} also OP in {and, or, xor} with NE = -1, 0, 0
 * (tests/hist/{and,or,xor}.fut).
 * hist_OP_T, rbi_OP_T and their _i64 forms exist in addition for T in {i8, u8, i16, u16, u32,
 * u64} with all six operators and for f16 with add, max, min: the element types
 * whose updates the reference emulates with compare-and-swap, and the unsigned
 * comparisons (tests/hist/{i8,i16,and8,and16,max8,max16,max,f16}.fut ...).
 */
#ifndef SEGOPS_H
#define SEGOPS_H

#include <stdint.h>
#include <stddef.h>
#include <stdbool.h>
#include <stdio.h>
#include <float.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FUTHARK_BACKEND_hip
#define FUTHARK_SUCCESS 0
#define FUTHARK_PROGRAM_ERROR 2
#define FUTHARK_OUT_OF_MEMORY 3

/* Device pointers cross the raw-array functions as this type. */
typedef void *futhark_device_ptr;

/* --------------------------------------------------------- Initialisation */
struct futhark_context_config;
struct futhark_context_config *futhark_context_config_new(void);
void futhark_context_config_free(struct futhark_context_config *cfg);
int futhark_context_config_set_tuning_param(struct futhark_context_config *cfg,
                                            const char *param_name, size_t new_value);
void futhark_context_config_set_debugging(struct futhark_context_config *cfg, int flag);
void futhark_context_config_set_profiling(struct futhark_context_config *cfg, int flag);
void futhark_context_config_set_logging(struct futhark_context_config *cfg, int flag);
void futhark_context_config_set_cache_file(struct futhark_context_config *cfg, const char *f);
int futhark_get_tuning_param_count(void);
const char *futhark_get_tuning_param_name(int i);
const char *futhark_get_tuning_param_class(int i);
/* GPU backends (docs/c-api.rst:609-669) */
void futhark_context_config_set_device(struct futhark_context_config *cfg, const char *s);
void futhark_context_config_set_unified_memory(struct futhark_context_config *cfg, int flag);
void futhark_context_config_set_default_thread_block_size(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_group_size(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_grid_size(struct futhark_context_config *cfg, int num);
void futhark_context_config_set_default_num_groups(struct futhark_context_config *cfg, int num);
void futhark_context_config_set_default_tile_size(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_reg_tile_size(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_cache(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_registers(struct futhark_context_config *cfg, int size);
void futhark_context_config_set_default_threshold(struct futhark_context_config *cfg, int size);
void futhark_context_config_add_build_option(struct futhark_context_config *cfg, const char *opt);
const char *futhark_context_config_get_program(struct futhark_context_config *cfg);
void futhark_context_config_set_program(struct futhark_context_config *cfg, const char *s);

struct futhark_context;
struct futhark_context *futhark_context_new(struct futhark_context_config *cfg);
void futhark_context_free(struct futhark_context *ctx);

/* ----------------------------------------------------------------- Arrays
 * For every array type futhark_T_Rd:
 *   new      copies `data` (row-major, host) to the device, asynchronously
 *   new_raw  wraps caller-owned device memory; never freed by the library
 *   free     drops one reference
 *   values   asynchronous copy to host; sync before reading
 *   index    one element to host; 1 + "Index out of bounds." if outside
 *   values_raw, shape
 */
#define FUTHARK_DECLARE_ARRAY_1D(NAME, CT)                                                     \
  struct futhark_##NAME##_1d;                                                                  \
  struct futhark_##NAME##_1d *futhark_new_##NAME##_1d(struct futhark_context *ctx,             \
                                                      const CT *data, int64_t dim0);           \
  struct futhark_##NAME##_1d *futhark_new_raw_##NAME##_1d(struct futhark_context *ctx,         \
                                                          futhark_device_ptr data,             \
                                                          int64_t dim0);                       \
  int futhark_free_##NAME##_1d(struct futhark_context *ctx, struct futhark_##NAME##_1d *arr);  \
  int futhark_values_##NAME##_1d(struct futhark_context *ctx, struct futhark_##NAME##_1d *arr, \
                                 CT *data);                                                    \
  int futhark_index_##NAME##_1d(struct futhark_context *ctx, CT *out,                          \
                                struct futhark_##NAME##_1d *arr, int64_t i0);                  \
  futhark_device_ptr futhark_values_raw_##NAME##_1d(struct futhark_context *ctx,               \
                                                    struct futhark_##NAME##_1d *arr);          \
  const int64_t *futhark_shape_##NAME##_1d(struct futhark_context *ctx,                        \
                                           struct futhark_##NAME##_1d *arr);

#define FUTHARK_DECLARE_ARRAY_2D(NAME, CT)                                                     \
  struct futhark_##NAME##_2d;                                                                  \
  struct futhark_##NAME##_2d *futhark_new_##NAME##_2d(struct futhark_context *ctx,             \
                                                      const CT *data, int64_t dim0,            \
                                                      int64_t dim1);                           \
  struct futhark_##NAME##_2d *futhark_new_raw_##NAME##_2d(struct futhark_context *ctx,         \
                                                          futhark_device_ptr data,             \
                                                          int64_t dim0, int64_t dim1);         \
  int futhark_free_##NAME##_2d(struct futhark_context *ctx, struct futhark_##NAME##_2d *arr);  \
  int futhark_values_##NAME##_2d(struct futhark_context *ctx, struct futhark_##NAME##_2d *arr, \
                                 CT *data);                                                    \
  int futhark_index_##NAME##_2d(struct futhark_context *ctx, CT *out,                          \
                                struct futhark_##NAME##_2d *arr, int64_t i0, int64_t i1);      \
  futhark_device_ptr futhark_values_raw_##NAME##_2d(struct futhark_context *ctx,               \
                                                    struct futhark_##NAME##_2d *arr);          \
  const int64_t *futhark_shape_##NAME##_2d(struct futhark_context *ctx,                        \
                                           struct futhark_##NAME##_2d *arr);

#define FUTHARK_DECLARE_ARRAY_3D(NAME, CT)                                                     \
  struct futhark_##NAME##_3d;                                                                  \
  struct futhark_##NAME##_3d *futhark_new_##NAME##_3d(struct futhark_context *ctx,             \
                                                      const CT *data, int64_t dim0,            \
                                                      int64_t dim1, int64_t dim2);             \
  struct futhark_##NAME##_3d *futhark_new_raw_##NAME##_3d(struct futhark_context *ctx,         \
                                                          futhark_device_ptr data,             \
                                                          int64_t dim0, int64_t dim1,          \
                                                          int64_t dim2);                       \
  int futhark_free_##NAME##_3d(struct futhark_context *ctx, struct futhark_##NAME##_3d *arr);  \
  int futhark_values_##NAME##_3d(struct futhark_context *ctx, struct futhark_##NAME##_3d *arr, \
                                 CT *data);                                                    \
  int futhark_index_##NAME##_3d(struct futhark_context *ctx, CT *out,                          \
                                struct futhark_##NAME##_3d *arr, int64_t i0, int64_t i1,       \
                                int64_t i2);                                                   \
  futhark_device_ptr futhark_values_raw_##NAME##_3d(struct futhark_context *ctx,               \
                                                    struct futhark_##NAME##_3d *arr);          \
  const int64_t *futhark_shape_##NAME##_3d(struct futhark_context *ctx,                        \
                                           struct futhark_##NAME##_3d *arr);

FUTHARK_DECLARE_ARRAY_1D(i32, int32_t)
FUTHARK_DECLARE_ARRAY_1D(i64, int64_t)
FUTHARK_DECLARE_ARRAY_1D(i8, int8_t)
FUTHARK_DECLARE_ARRAY_1D(i16, int16_t)
FUTHARK_DECLARE_ARRAY_1D(u8, uint8_t)
FUTHARK_DECLARE_ARRAY_1D(u16, uint16_t)
FUTHARK_DECLARE_ARRAY_1D(f16, uint16_t) /* f16 crosses the API as its bits */
FUTHARK_DECLARE_ARRAY_1D(u32, uint32_t)
FUTHARK_DECLARE_ARRAY_1D(u64, uint64_t)
FUTHARK_DECLARE_ARRAY_1D(f32, float)
FUTHARK_DECLARE_ARRAY_1D(f64, double)
FUTHARK_DECLARE_ARRAY_2D(i32, int32_t)
FUTHARK_DECLARE_ARRAY_2D(i64, int64_t)
FUTHARK_DECLARE_ARRAY_2D(f32, float)
FUTHARK_DECLARE_ARRAY_2D(f64, double)
FUTHARK_DECLARE_ARRAY_3D(f32, float)
FUTHARK_DECLARE_ARRAY_3D(f16, uint16_t) /* f16 crosses the API as its bits */
FUTHARK_DECLARE_ARRAY_3D(u16, uint16_t)

/* ---------------------------------------------------------------- Opaque
 * A tuple result is one opaque value (docs/c-api.rst:318-432); the type
 * ([]K, []V) is named futhark_opaque_tup2_arr1d_K_arr1d_V
 * (src/Futhark/CodeGen/Backends/SimpleRep.hs:144-186).
 *   free     drops the value (its components have their own references)
 *   store    serialises to *p (malloc'd if *p is NULL; p == NULL only sets *n);
 *            the components follow each other in the binary data format
 *   restore  the inverse; NULL on malformed input
 *   new      a tuple aliasing the given arrays, with its own lifetime
 *   project  component 0 / 1 as an array value the caller frees */
#define FUTHARK_DECLARE_SORT_PAIRS(NAME, K, V)                                                 \
  struct futhark_opaque_##NAME;                                                                \
  int futhark_free_opaque_##NAME(struct futhark_context *ctx,                                  \
                                 struct futhark_opaque_##NAME *obj);                           \
  int futhark_store_opaque_##NAME(struct futhark_context *ctx,                                 \
                                  const struct futhark_opaque_##NAME *obj, void **p,           \
                                  size_t *n);                                                  \
  struct futhark_opaque_##NAME *futhark_restore_opaque_##NAME(struct futhark_context *ctx,     \
                                                              const void *p);                  \
  int futhark_new_opaque_##NAME(struct futhark_context *ctx,                                   \
                                struct futhark_opaque_##NAME **out,                            \
                                const struct futhark_##K##_1d *f_0,                            \
                                const struct futhark_##V##_1d *f_1);                           \
  int futhark_project_opaque_##NAME##_0(struct futhark_context *ctx,                           \
                                        struct futhark_##K##_1d **out,                         \
                                        const struct futhark_opaque_##NAME *obj);              \
  int futhark_project_opaque_##NAME##_1(struct futhark_context *ctx,                           \
                                        struct futhark_##V##_1d **out,                         \
                                        const struct futhark_opaque_##NAME *obj);              \
  int futhark_entry_radix_sort_pairs_##K##_##V(struct futhark_context *ctx,                    \
                                               struct futhark_opaque_##NAME **out0,            \
                                               const struct futhark_##K##_1d *in0,             \
                                               const struct futhark_##V##_1d *in1);

/* ----------------------------------------------------------- Entry points
 * int futhark_entry_NAME(ctx, outputs..., inputs...): 0 on success; scalar
 * outputs are valid after futhark_context_sync; array outputs are new values
 * the caller frees. */
#define FUTHARK_FOR_EACH_NUM_TYPE(X) X(i32, int32_t) X(i64, int64_t) X(f32, float) X(f64, double)
#define FUTHARK_FOR_EACH_OP(X, T, CT) X(add, T, CT) X(max, T, CT) X(min, T, CT)

#define FUTHARK_DECLARE_SEGOP_ENTRIES(OP, T, CT)                                              \
  int futhark_entry_reduce_##OP##_##T(struct futhark_context *ctx, CT *out0,                  \
                                      const struct futhark_##T##_1d *in0);                    \
  int futhark_entry_scan_##OP##_##T(struct futhark_context *ctx,                              \
                                    struct futhark_##T##_1d **out0,                           \
                                    const struct futhark_##T##_1d *in0);                      \
  int futhark_entry_exscan_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_1d **out0,                         \
                                      const struct futhark_##T##_1d *in0);                    \
  int futhark_entry_segscan_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_1d **out0,                        \
                                       const struct futhark_u8_1d *in0,                       \
                                       const struct futhark_##T##_1d *in1);                   \
  int futhark_entry_segred_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_1d **out0,                         \
                                      const struct futhark_i64_1d *in0,                       \
                                      const struct futhark_i64_1d *in1,                       \
                                      const struct futhark_##T##_1d *in2);                    \
  int futhark_entry_segreduce_##OP##_##T(struct futhark_context *ctx,                         \
                                         struct futhark_##T##_1d **out0,                      \
                                         const struct futhark_##T##_2d *in0);                 \
  int futhark_entry_vecreduce_##OP##_##T(struct futhark_context *ctx,                         \
                                         struct futhark_##T##_1d **out0,                      \
                                         const struct futhark_##T##_2d *in0);                 \
  int futhark_entry_scanrows_##OP##_##T(struct futhark_context *ctx,                          \
                                        struct futhark_##T##_2d **out0,                       \
                                        const struct futhark_##T##_2d *in0);                  \
  int futhark_entry_vecscan_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0,                        \
                                       const struct futhark_##T##_2d *in0);                   \
  int futhark_entry_seghist_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0, const int64_t in0,     \
                                       const struct futhark_i32_2d *in1,                      \
                                       const struct futhark_##T##_2d *in2);                   \
  int futhark_entry_rbi_vec_##OP##_##T(struct futhark_context *ctx,                           \
                                       struct futhark_##T##_2d **out0,                        \
                                       const struct futhark_##T##_2d *in0,                    \
                                       const struct futhark_i64_1d *in1,                      \
                                       const struct futhark_##T##_2d *in2);                   \
  int futhark_entry_rbi_2d_##OP##_##T(struct futhark_context *ctx,                            \
                                      struct futhark_##T##_2d **out0,                         \
                                      const struct futhark_##T##_2d *in0,                     \
                                      const struct futhark_i64_1d *in1,                       \
                                      const struct futhark_i64_1d *in2,                       \
                                      const struct futhark_##T##_1d *in3);                    \
  FUTHARK_DECLARE_HIST_ENTRIES(OP, T, CT)

#define FUTHARK_DECLARE_HIST_ENTRIES(OP, T, CT)                                               \
  FUTHARK_DECLARE_HIST_ENTRIES_IX(OP, T, CT, , i32)                                           \
  FUTHARK_DECLARE_HIST_ENTRIES_IX(OP, T, CT, _i64, i64)
#define FUTHARK_DECLARE_HIST_ENTRIES_IX(OP, T, CT, SUFFIX, IT)                                \
  int futhark_entry_hist_##OP##_##T##SUFFIX(struct futhark_context *ctx,                      \
                                            struct futhark_##T##_1d **out0, const int64_t in0, \
                                            const struct futhark_##IT##_1d *in1,              \
                                            const struct futhark_##T##_1d *in2);              \
  int futhark_entry_rbi_##OP##_##T##SUFFIX(struct futhark_context *ctx,                       \
                                           struct futhark_##T##_1d **out0,                    \
                                           const struct futhark_##T##_1d *in0,                \
                                           const struct futhark_##IT##_1d *in1,               \
                                           const struct futhark_##T##_1d *in2);

#define FUTHARK_DECLARE_FOR_TYPE(T, CT) FUTHARK_FOR_EACH_OP(FUTHARK_DECLARE_SEGOP_ENTRIES, T, CT)
FUTHARK_FOR_EACH_NUM_TYPE(FUTHARK_DECLARE_FOR_TYPE)

/* The same eight entry points for the bitwise operators on the integer types. */
#define FUTHARK_FOR_EACH_INT_TYPE(X) X(i32, int32_t) X(i64, int64_t)
#define FUTHARK_FOR_EACH_BITOP(X, T, CT) X(and, T, CT) X(or, T, CT) X(xor, T, CT)
#define FUTHARK_DECLARE_BITOPS_FOR_TYPE(T, CT) \
  FUTHARK_FOR_EACH_BITOP(FUTHARK_DECLARE_SEGOP_ENTRIES, T, CT)
FUTHARK_FOR_EACH_INT_TYPE(FUTHARK_DECLARE_BITOPS_FOR_TYPE)

/* hist_OP_T and rbi_OP_T alone for the remaining integer types and f16. */
#define FUTHARK_FOR_EACH_HIST_ONLY_INT_TYPE(X) \
  X(i8, int8_t) X(u8, uint8_t) X(i16, int16_t) X(u16, uint16_t) X(u32, uint32_t) X(u64, uint64_t)
#define FUTHARK_DECLARE_HIST_ONLY_INT(T, CT)                  \
  FUTHARK_FOR_EACH_OP(FUTHARK_DECLARE_HIST_ENTRIES, T, CT)    \
  FUTHARK_FOR_EACH_BITOP(FUTHARK_DECLARE_HIST_ENTRIES, T, CT)
FUTHARK_FOR_EACH_HIST_ONLY_INT_TYPE(FUTHARK_DECLARE_HIST_ONLY_INT)
FUTHARK_FOR_EACH_OP(FUTHARK_DECLARE_HIST_ENTRIES, f16, uint16_t)

int futhark_entry_bmm_f32(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                          const struct futhark_f32_3d *in0, const struct futhark_f32_3d *in1);
int futhark_entry_bmm_f16(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                          const struct futhark_f16_3d *in0, const struct futhark_f16_3d *in1);
/* Scans with a non-commutative operator: composition of affine maps modulo 2^32,
 *   def compose (a1: i32, b1: i32) (a2: i32, b2: i32) = (a1 * a2, a2 * b1 + b2)
 *   entry scan_compose_i32 (abs: [][2]i32) : [][2]i32 =
 *     scan compose (1, 0) (map (\r -> (r[0], r[1])) abs) |> map (\(a, b) -> [a, b])
 * exscan_compose_i32 and segscan_compose_i32 (flags: []u8) likewise. */
int futhark_entry_scan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                   const struct futhark_i32_2d *in0);
int futhark_entry_exscan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                     const struct futhark_i32_2d *in0);
int futhark_entry_segscan_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                      const struct futhark_u8_1d *in0,
                                      const struct futhark_i32_2d *in1);

/* SegOps whose operator or fused maps are the program's own (kernels
 * instantiated from include/futhark_amd_segops.hpp):
 *   def argmax (v1: i32, i1: i32) (v2: i32, i2: i32) =
 *     if v1 > v2 || (v1 == v2 && i1 < i2) then (v1, i1) else (v2, i2)
 *   entry reduce_argmax_i32 [n] (xs: [n]i32) : [2]i32 =
 *     let (v, i) = reduce_comm argmax (i32.lowest, i32.highest) (zip xs (map i32.i64 (iota n)))
 *     in [v, i]
 *   entry scan_argmax_i32 (vis: [][2]i32) : [][2]i32 =     -- rows (value, index)
 *     scan argmax (i32.lowest, i32.highest) (map (\r -> (r[0], r[1])) vis) |> map (\(v, i) -> [v, i])
 *   entry hist_argmax_i32 (k: i64) (is: []i32) (xs: []i32) : [k][2]i32 =
 *     hist argmax (i32.lowest, i32.highest) k (map i64.i32 is) (zip xs (map i32.i64 (indices xs)))
 *     |> map (\(v, i) -> [v, i])
 *   entry reduce_compose_i32 (abs: [][2]i32) : [2]i32 =    -- compose as above; does not commute
 *     let (a, b) = reduce compose (1, 0) (map (\r -> (r[0], r[1])) abs) in [a, b]
 *   entry sumsq_f32 (xs: []f32) : f32 = reduce (+) 0 (map (\x -> x * x) xs)
 *   entry reduce_summax_f32 (xs: []f32) : [2]f32 =
 *     let (s, m) = reduce (\(a,b) (c,d) -> (a + c, f32.max b d)) (0, -f32.inf) (zip xs xs) in [s, m]
 *                                   -- two operators in one SegRed, SegRed.hs:157-199
 *   entry scan_norm_f32 (xs: []f32) : []f32 = map f32.sqrt (scan (+) 0 (map (\x -> x * x) xs))
 *   entry rows_fraction_f32 (xss: [][]f32) : [][]f32 =
 *     map (\r -> let t = reduce (+) 0 r in map (/ t) (scan (+) 0 r)) xss
 *                                   -- SegOps at block level, ImpGen/GPU/Block.hs:357-615
 * The same operators in the segmented forms (SegRed.hs:396-636,
 * SegScan/SinglePass.hs:327-361, Pass/Flatten/Builtins.hs:570-602):
 *   entry segreduce_argmax_i32 [m][k] (xss: [m][k]i32) : [m][2]i32 =
 *     map (\row -> reduce_comm argmax (i32.lowest, i32.highest) (zip row (map i32.i64 (iota k)))) xss
 *     |> map (\(v, i) -> [v, i])
 *   entry segreduce_compose_i32 (k: i64) (abs: [][2]i32) : [][2]i32 =   -- rows of k maps each
 *     map (reduce compose (1, 0)) (unflatten (map (\r -> (r[0], r[1])) abs)) |> map (\(a, b) -> [a, b])
 *   entry scanrows_argmax_i32 (k: i64) (vis: [][2]i32) : [][2]i32 =     -- rows of k pairs each
 *     map (scan argmax (i32.lowest, i32.highest)) (unflatten ...) |> flatten
 *   entry segred_argmax_i32 [m] (offsets: [m]i64) (lens: [m]i64) (vis: [][2]i32) : [m][2]i32
 *     -- segred_OP_T above with argmax over the pairs */
int futhark_entry_reduce_argmax_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                    const struct futhark_i32_1d *in0);
int futhark_entry_scan_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                  const struct futhark_i32_2d *in0);
int futhark_entry_hist_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                  const int64_t in0, const struct futhark_i32_1d *in1,
                                  const struct futhark_i32_1d *in2);
int futhark_entry_reduce_compose_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                     const struct futhark_i32_2d *in0);
int futhark_entry_sumsq_f32(struct futhark_context *ctx, float *out0,
                            const struct futhark_f32_1d *in0);
int futhark_entry_reduce_summax_f32(struct futhark_context *ctx, struct futhark_f32_1d **out0,
                                    const struct futhark_f32_1d *in0);
int futhark_entry_scan_norm_f32(struct futhark_context *ctx, struct futhark_f32_1d **out0,
                                const struct futhark_f32_1d *in0);
int futhark_entry_rows_fraction_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                                    const struct futhark_f32_2d *in0);
int futhark_entry_segreduce_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                       const struct futhark_i32_2d *in0);
int futhark_entry_segreduce_compose_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                        const int64_t in0, const struct futhark_i32_2d *in1);
int futhark_entry_scanrows_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                      const int64_t in0, const struct futhark_i32_2d *in1);
int futhark_entry_segred_argmax_i32(struct futhark_context *ctx, struct futhark_i32_2d **out0,
                                    const struct futhark_i64_1d *in0,
                                    const struct futhark_i64_1d *in1,
                                    const struct futhark_i32_2d *in2);
int futhark_entry_bmm_bf16(struct futhark_context *ctx, struct futhark_f32_3d **out0,
                           const struct futhark_u16_3d *in0, const struct futhark_u16_3d *in1);
int futhark_entry_matmul_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                             const struct futhark_f32_2d *in0, const struct futhark_f32_2d *in1);

int futhark_entry_radix_sort_u32(struct futhark_context *ctx, struct futhark_u32_1d **out0,
                                 const struct futhark_u32_1d *in0);
int futhark_entry_radix_sort_u64(struct futhark_context *ctx, struct futhark_u64_1d **out0,
                                 const struct futhark_u64_1d *in0);
FUTHARK_DECLARE_SORT_PAIRS(tup2_arr1d_u32_arr1d_i32, u32, i32)
FUTHARK_DECLARE_SORT_PAIRS(tup2_arr1d_u64_arr1d_i32, u64, i32)

int futhark_entry_transpose_f32(struct futhark_context *ctx, struct futhark_f32_2d **out0,
                                const struct futhark_f32_2d *in0);
int futhark_entry_iota_i64(struct futhark_context *ctx, struct futhark_i64_1d **out0,
                           const int64_t in0);
int futhark_entry_replicate_i32(struct futhark_context *ctx, struct futhark_i32_1d **out0,
                                const int64_t in0, const int32_t in1);

/* ---------------------------------------------------------- Miscellaneous */
int futhark_context_sync(struct futhark_context *ctx);
char *futhark_context_get_error(struct futhark_context *ctx); /* caller frees */
void futhark_context_set_logging_file(struct futhark_context *ctx, FILE *f);
void futhark_context_pause_profiling(struct futhark_context *ctx);
void futhark_context_unpause_profiling(struct futhark_context *ctx);
char *futhark_context_report(struct futhark_context *ctx); /* JSON; caller frees */
int futhark_context_clear_caches(struct futhark_context *ctx);

/* Not part of the reference API: the HIP stream all work of this context is
 * queued on, for callers that time kernels with their own events. */
void *futhark_context_get_stream(struct futhark_context *ctx);

#ifdef __cplusplus
}
#endif
#endif /* SEGOPS_H */
