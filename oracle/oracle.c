/*
 * oracle.c -- CPU restatement of what `futhark c` computes for the SegOp path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships may call into this file: only
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg load
 * liboracle.so, and only as the checker / the timed CPU baseline.
 *
 * `futhark c` sequentialises every SOAC with
 * src/Futhark/Transform/FirstOrderTransform.hs:
 *   reduce/scan   acc = ne; for i < n: acc = op(acc, x[i])      (:613-656)
 *   hist          in-order read-modify-write, out-of-range bins skipped (:505-560)
 * and scalar operators mean what rts/c/scalar.h says: add wraps in two's
 * complement (:29-30), smax/smin (:488-503), fmax/fmin = fmaxf/fminf (:931-934).
 * Functions named *_lit follow that evaluation order literally in the element
 * type.  Functions named *_f64acc accumulate floating-point sums in double
 * and round once per output; they are the yardstick for the 1e-5 tolerance,
 * because any parallel schedule reassociates and the literal f32 fold is itself
 * far from the exact sum at these sizes.
 *
 * Pinning (tests/test_oracle_golden.py): every function here is checked
 * against the golden vectors the reference's own tests hold (tests/golden/),
 * and against numpy closed forms / library routines on seeded inputs.
 * bf16 matmul has no Futhark program to compare with (no such type in the
 * reference): parity unpinned for orc_bmm_bf16 beyond its definition
 * (bits << 16, then the f32 path).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ----------------------------------------------------------- scalar ops */
#define OPS_INT(T, U, S)                                                        \
  static inline T add_##S(T a, T b) { return (T)((U)a + (U)b); }                \
  static inline T max_##S(T a, T b) { return a < b ? b : a; }                   \
  static inline T min_##S(T a, T b) { return a < b ? a : b; }                   \
  static inline T and_##S(T a, T b) { return a & b; }                           \
  static inline T or_##S(T a, T b) { return a | b; }                            \
  static inline T xor_##S(T a, T b) { return a ^ b; }
OPS_INT(int32_t, uint32_t, i32)
OPS_INT(int64_t, uint64_t, i64)
/* the remaining integer types: element types of histograms only
 * (tests/hist/{i8,i16,and8,and16,max8,max16,min8,min16,or8,or16,xor8,xor16}.fut) */
OPS_INT(int8_t, uint8_t, i8)
OPS_INT(uint8_t, uint8_t, u8)
OPS_INT(int16_t, uint16_t, i16)
OPS_INT(uint16_t, uint16_t, u16)
OPS_INT(uint32_t, uint32_t, u32)
OPS_INT(uint64_t, uint64_t, u64)
static inline float add_f32(float a, float b) { return a + b; }
static inline float max_f32(float a, float b) { return fmaxf(a, b); }
static inline float min_f32(float a, float b) { return fminf(a, b); }
static inline double add_f64(double a, double b) { return a + b; }
static inline double max_f64(double a, double b) { return fmax(a, b); }
static inline double min_f64(double a, double b) { return fmin(a, b); }

/* neutral elements: 0, T.lowest, T.highest (prelude/math.fut:555-556,633-634,1077-1078) */
#define NE_add_i32 0
#define NE_max_i32 INT32_MIN
#define NE_min_i32 INT32_MAX
#define NE_add_i64 0
#define NE_max_i64 INT64_MIN
#define NE_min_i64 INT64_MAX
/* bitwise operators: -1, 0, 0 (tests/hist/and.fut:32, or.fut:32, xor.fut:32) */
#define NE_and_i32 (-1)
#define NE_or_i32 0
#define NE_xor_i32 0
#define NE_and_i64 (-1)
#define NE_or_i64 0
#define NE_xor_i64 0
#define NE_add_f32 0.0f
#define NE_max_f32 (-INFINITY)
#define NE_min_f32 (INFINITY)
#define NE_add_f64 0.0
#define NE_max_f64 (-(double)INFINITY)
#define NE_min_f64 ((double)INFINITY)

/* ------------------------------------- reduce / scan / segmented, literal
 * FirstOrderTransform.hs:613-656; flag-tuple operator
 * src/Futhark/Pass/Flatten/Builtins.hs:374-393; exclusive scan
 * prelude/soacs.fut:212-215; irregular segmented reduce Builtins.hs:570-602. */
#define DEFINE_LIT(OP, S, T)                                                                   \
  T orc_reduce_##OP##_##S##_lit(const T *xs, int64_t n) {                                      \
    T acc = NE_##OP##_##S;                                                                     \
    for (int64_t i = 0; i < n; i++) acc = OP##_##S(acc, xs[i]);                                \
    return acc;                                                                                \
  }                                                                                            \
  void orc_scan_##OP##_##S##_lit(const T *xs, int64_t n, T *out) {                             \
    T acc = NE_##OP##_##S;                                                                     \
    for (int64_t i = 0; i < n; i++) {                                                          \
      acc = OP##_##S(acc, xs[i]);                                                              \
      out[i] = acc;                                                                            \
    }                                                                                          \
  }                                                                                            \
  void orc_exscan_##OP##_##S##_lit(const T *xs, int64_t n, T *out) {                           \
    T acc = NE_##OP##_##S;                                                                     \
    for (int64_t i = 0; i < n; i++) {                                                          \
      out[i] = acc;                                                                            \
      acc = OP##_##S(acc, xs[i]);                                                              \
    }                                                                                          \
  }                                                                                            \
  void orc_segscan_##OP##_##S##_lit(const uint8_t *flags, const T *xs, int64_t n, T *out) {    \
    int af = 0;                                                                                \
    T av = NE_##OP##_##S;                                                                      \
    for (int64_t i = 0; i < n; i++) {                                                          \
      const int yf = flags[i] != 0;                                                            \
      av = yf ? xs[i] : OP##_##S(av, xs[i]);                                                   \
      af = af || yf;                                                                           \
      out[i] = av;                                                                             \
    }                                                                                          \
    (void)af;                                                                                  \
  }                                                                                            \
  /* returns 0, or 1 if an offset lies outside [0,n) for a non-empty segment */                \
  int orc_segred_##OP##_##S##_lit(const int64_t *offsets, const int64_t *lens, int64_t m,      \
                                  const T *xs, int64_t n, T *out) {                            \
    uint8_t *flags = (uint8_t *)calloc((size_t)(n > 0 ? n : 1), 1);                            \
    T *s = (T *)malloc(sizeof(T) * (size_t)(n > 0 ? n : 1));                                   \
    for (int64_t i = 0; i < m; i++)                                                            \
      if (offsets[i] >= 0 && offsets[i] < n) flags[offsets[i]] = 1; /* scatter drops OOB */    \
    orc_segscan_##OP##_##S##_lit(flags, xs, n, s);                                             \
    int bad = 0;                                                                               \
    for (int64_t i = 0; i < m; i++) {                                                          \
      if (lens[i] == 0) out[i] = NE_##OP##_##S;                                                \
      else {                                                                                   \
        const int64_t p = offsets[i] + lens[i] - 1;                                            \
        if (p < 0 || p >= n) { bad = 1; out[i] = NE_##OP##_##S; }                              \
        else out[i] = s[p];                                                                    \
      }                                                                                        \
    }                                                                                          \
    free(flags);                                                                               \
    free(s);                                                                                   \
    return bad;                                                                                \
  }                                                                                            \
  void orc_segreduce_##OP##_##S##_lit(const T *xss, int64_t m, int64_t k, T *out) {            \
    for (int64_t i = 0; i < m; i++) out[i] = orc_reduce_##OP##_##S##_lit(xss + i * k, k);      \
  }                                                                                            \
  /* reduce_by_index dest (map2 OP) (replicate m NE) is vss: dest [H][m], vss [n][m]; the     \
   * same in-order read-modify-write, a whole vector per update */                             \
  void orc_rbi_vec_##OP##_##S##_lit(T *dest, int64_t H, int64_t m, const int64_t *is,          \
                                    const T *vss, int64_t n) {                                 \
    for (int64_t i = 0; i < n; i++) {                                                          \
      const int64_t b = is[i];                                                                 \
      if (b < 0 || b >= H) continue;                                                           \
      for (int64_t c = 0; c < m; c++) dest[b * m + c] = OP##_##S(dest[b * m + c], vss[i * m + c]); \
    }                                                                                          \
  }                                                                                            \
  /* reduce_by_index_2d dest OP NE (zip is js) vs (prelude/soacs.fut:149-150): an update     \
   * is dropped unless both coordinates are in range */                                        \
  void orc_rbi_2d_##OP##_##S##_lit(T *dest, int64_t H0, int64_t H1, const int64_t *is,         \
                                   const int64_t *js, const T *vs, int64_t n) {                \
    for (int64_t i = 0; i < n; i++) {                                                          \
      if (is[i] < 0 || is[i] >= H0 || js[i] < 0 || js[i] >= H1) continue;                      \
      T *cell = dest + is[i] * H1 + js[i];                                                     \
      *cell = OP##_##S(*cell, vs[i]);                                                          \
    }                                                                                          \
  }                                                                                            \
  /* reduce (map2 OP) (replicate k NE) xss, rows folded in order */                            \
  void orc_vecreduce_##OP##_##S##_lit(const T *xss, int64_t n, int64_t k, T *out) {            \
    for (int64_t j = 0; j < k; j++) out[j] = NE_##OP##_##S;                                    \
    for (int64_t i = 0; i < n; i++)                                                            \
      for (int64_t j = 0; j < k; j++) out[j] = OP##_##S(out[j], xss[i * k + j]);               \
  }                                                                                            \
  /* hist / reduce_by_index: FirstOrderTransform.hs:505-560 */                                 \
  void orc_rbi_##OP##_##S##_lit(T *dest, int64_t H, const int32_t *is, const T *vs,            \
                                int64_t n) {                                                   \
    for (int64_t i = 0; i < n; i++) {                                                          \
      const int64_t b = (int64_t)is[i];                                                        \
      if (b >= 0 && b < H) dest[b] = OP##_##S(dest[b], vs[i]);                                 \
    }                                                                                          \
  }

#define DEFINE_LIT_ALL_OPS(S, T) DEFINE_LIT(add, S, T) DEFINE_LIT(max, S, T) DEFINE_LIT(min, S, T)
DEFINE_LIT_ALL_OPS(i32, int32_t)
DEFINE_LIT_ALL_OPS(i64, int64_t)
#define DEFINE_LIT_BITOPS(S, T) DEFINE_LIT(and, S, T) DEFINE_LIT(or, S, T) DEFINE_LIT(xor, S, T)
DEFINE_LIT_BITOPS(i32, int32_t)
DEFINE_LIT_BITOPS(i64, int64_t)
DEFINE_LIT_ALL_OPS(f32, float)
DEFINE_LIT_ALL_OPS(f64, double)

/* Scans of affine maps x -> a*x + b modulo 2^32 under composition,
 *   (a1, b1) then (a2, b2) = (a1*a2, a2*b1 + b2), neutral (1, 0):
 * an associative operator that does not commute.  abs and out are [n][2].
 * The same left-to-right loops as the scans above (FirstOrderTransform.hs:613-656;
 * flag operator Pass/Flatten/Builtins.hs:374-393). */
void orc_scan_compose_i32_lit(const uint8_t *flags, const int32_t *abs, int64_t n, int exclusive,
                              int32_t *out) {
  uint32_t a = 1, b = 0;
  for (int64_t i = 0; i < n; i++) {
    const uint32_t xa = (uint32_t)abs[2 * i], xb = (uint32_t)abs[2 * i + 1];
    if (flags != NULL && flags[i] != 0) { a = 1; b = 0; }
    if (exclusive) { out[2 * i] = (int32_t)a; out[2 * i + 1] = (int32_t)b; }
    const uint32_t na = a * xa, nb = xa * b + xb;
    a = na; b = nb;
    if (!exclusive) { out[2 * i] = (int32_t)a; out[2 * i + 1] = (int32_t)b; }
  }
}

/* The argmax operator on (value, index) pairs of i32: the larger value wins,
 * among equal values the smaller index; neutral (INT32_MIN, INT32_MAX).  Scan,
 * reduce and reduce_by_index with it are the same left-to-right loops as above
 * (FirstOrderTransform.hs:505-560 for hist, :613-656 for scan); a tuple is just
 * two accumulators (the loops carry one variable per component). */
static void argmax_i32(int32_t *v, int32_t *i, int32_t v2, int32_t i2) {
  if (!(*v > v2 || (*v == v2 && *i < i2))) { *v = v2; *i = i2; }
}
void orc_scan_argmax_i32_lit(const uint8_t *flags, const int32_t *vis, int64_t n, int exclusive,
                             int32_t *out) {
  int32_t v = INT32_MIN, ix = INT32_MAX;
  for (int64_t i = 0; i < n; i++) {
    if (flags != NULL && flags[i] != 0) { v = INT32_MIN; ix = INT32_MAX; }
    if (exclusive) { out[2 * i] = v; out[2 * i + 1] = ix; }
    argmax_i32(&v, &ix, vis[2 * i], vis[2 * i + 1]);
    if (!exclusive) { out[2 * i] = v; out[2 * i + 1] = ix; }
  }
}
void orc_hist_argmax_i32_lit(int32_t *dest /* [H][2] */, int64_t H, const int32_t *is,
                             const int32_t *xs, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    const int64_t b = (int64_t)is[i];
    if (b >= 0 && b < H) argmax_i32(&dest[2 * b], &dest[2 * b + 1], xs[i], (int32_t)i);
  }
}

/* hist / reduce_by_index alone for the other integer types */
#define DEFINE_RBI(OP, S, T)                                                                   \
  void orc_rbi_##OP##_##S##_lit(T *dest, int64_t H, const int32_t *is, const T *vs,            \
                                int64_t n) {                                                   \
    for (int64_t i = 0; i < n; i++) {                                                          \
      const int64_t b = (int64_t)is[i];                                                        \
      if (b >= 0 && b < H) dest[b] = OP##_##S(dest[b], vs[i]);                                 \
    }                                                                                          \
  }
#define DEFINE_RBI_ALL_OPS(S, T)                                                   \
  DEFINE_RBI(add, S, T) DEFINE_RBI(max, S, T) DEFINE_RBI(min, S, T) DEFINE_RBI(and, S, T) \
  DEFINE_RBI(or, S, T) DEFINE_RBI(xor, S, T)
DEFINE_RBI_ALL_OPS(i8, int8_t)
DEFINE_RBI_ALL_OPS(u8, uint8_t)
DEFINE_RBI_ALL_OPS(i16, int16_t)
DEFINE_RBI_ALL_OPS(u16, uint16_t)
DEFINE_RBI_ALL_OPS(u32, uint32_t)
DEFINE_RBI_ALL_OPS(u64, uint64_t)

/* ------------------------------- f32 sums accumulated in double (yardstick) */
float orc_reduce_add_f32_f64acc(const float *xs, int64_t n) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; i++) acc += (double)xs[i];
  return (float)acc;
}
void orc_scan_add_f32_f64acc(const float *xs, int64_t n, float *out) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; i++) {
    acc += (double)xs[i];
    out[i] = (float)acc;
  }
}
void orc_exscan_add_f32_f64acc(const float *xs, int64_t n, float *out) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; i++) {
    out[i] = (float)acc;
    acc += (double)xs[i];
  }
}
void orc_segscan_add_f32_f64acc(const uint8_t *flags, const float *xs, int64_t n, float *out) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; i++) {
    acc = flags[i] ? (double)xs[i] : acc + (double)xs[i];
    out[i] = (float)acc;
  }
}
void orc_segred_add_f32_f64acc(const int64_t *offsets, const int64_t *lens, int64_t m,
                               const float *xs, int64_t n, float *out) {
  /* Segments that tile the array: the sum of a segment is the scanned value at
   * its last element. */
  for (int64_t i = 0; i < m; i++) {
    double acc = 0.0;
    for (int64_t j = offsets[i]; j < offsets[i] + lens[i] && j < n; j++) acc += (double)xs[j];
    out[i] = (float)acc;
  }
}
void orc_rbi_add_f32_f64acc(float *dest, int64_t H, const int32_t *is, const float *vs,
                            int64_t n) {
  double *acc = (double *)malloc(sizeof(double) * (size_t)(H > 0 ? H : 1));
  for (int64_t b = 0; b < H; b++) acc[b] = (double)dest[b];
  for (int64_t i = 0; i < n; i++) {
    const int64_t b = (int64_t)is[i];
    if (b >= 0 && b < H) acc[b] += (double)vs[i];
  }
  for (int64_t b = 0; b < H; b++) dest[b] = (float)acc[b];
  free(acc);
}

/* ------------------------------------------------------------------ matmul
 * tests/reg-tiling/mmm.fut:17-21: C[i][j] = reduce (+) 0 (map2 (*) A[i,:] B[:,j]),
 * batched with an outer map2.  `lit` keeps products and the running sum in f32
 * in k order; `f64acc` accumulates in double. */
void orc_bmm_f32_lit(const float *A, const float *B, float *C, int64_t b, int64_t M, int64_t N,
                     int64_t K) {
  for (int64_t q = 0; q < b; q++)
    for (int64_t i = 0; i < M; i++)
      for (int64_t j = 0; j < N; j++) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; k++)
          acc = acc + A[(q * M + i) * K + k] * B[(q * K + k) * N + j];
        C[(q * M + i) * N + j] = acc;
      }
}
void orc_bmm_f32_f64acc(const float *A, const float *B, float *C, int64_t b, int64_t M,
                        int64_t N, int64_t K) {
  double *row = (double *)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
  for (int64_t q = 0; q < b; q++)
    for (int64_t i = 0; i < M; i++) {
      for (int64_t j = 0; j < N; j++) row[j] = 0.0;
      for (int64_t k = 0; k < K; k++) {
        const double a = (double)A[(q * M + i) * K + k];
        const float *brow = B + (q * K + k) * N;
        for (int64_t j = 0; j < N; j++) row[j] += a * (double)brow[j];
      }
      for (int64_t j = 0; j < N; j++) C[(q * M + i) * N + j] = (float)row[j];
    }
  free(row);
}

/* f16 -> f32, exact (every binary16 value is a binary32 value); what
 * rts/c/half.h:220-236 computes with tables. */
float orc_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  const uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ff;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {
      /* subnormal: value = man * 2^-24 */
      float f = (float)man * 5.9604644775390625e-08f;
      memcpy(&bits, &f, 4);
      bits |= sign;
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112) << 23) | (man << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
/* f32 -> f16, round to nearest even: what the `half` type of the GPU backends
 * does on conversion (rts/c/scalar_f16.h:11-60 computes f16 operators in float
 * and converts back; the table-driven float2halfbits of rts/c/half.h:220-228,
 * used where there is no native half type, truncates instead). */
uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu)); /* NaN */
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* 65520 and above, inf: to inf */
  if (x < 0x33000001u) return (uint16_t)sign; /* <= 2^-25: to zero (the tie goes to even) */
  if (x < 0x38800000u) {                      /* below 2^-14: subnormal result, units of 2^-24 */
    const int shift = 126 - (int)(x >> 23);   /* 14 .. 24 */
    const uint32_t man = (x & 0x7fffffu) | 0x800000u;
    uint32_t r = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
  }
  uint32_t r = (((x >> 23) - 112u) << 10) | ((x >> 13) & 0x3ffu);
  const uint32_t rem = x & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++; /* a carry runs into the exponent */
  return (uint16_t)(sign | r);
}
void orc_narrow_f16(const float *in, uint16_t *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(in[i]);
}
/* f16 histograms: operator in float on the widened operands, result stored as
 * f16 after every update (`lit`); sums accumulated in double and rounded once
 * per bin (`f64acc`). */
#define DEFINE_RBI_F16(OP)                                                                  \
  void orc_rbi_##OP##_f16_lit(uint16_t *dest, int64_t H, const int32_t *is,                 \
                              const uint16_t *vs, int64_t n) {                              \
    for (int64_t i = 0; i < n; i++) {                                                       \
      const int64_t b = (int64_t)is[i];                                                     \
      if (b >= 0 && b < H)                                                                  \
        dest[b] = orc_f32_to_f16(OP##_f32(orc_f16_to_f32(dest[b]), orc_f16_to_f32(vs[i]))); \
    }                                                                                       \
  }
DEFINE_RBI_F16(add)
DEFINE_RBI_F16(max)
DEFINE_RBI_F16(min)
void orc_rbi_add_f16_f64acc(uint16_t *dest, int64_t H, const int32_t *is, const uint16_t *vs,
                            int64_t n) {
  double *acc = (double *)malloc(sizeof(double) * (size_t)(H > 0 ? H : 1));
  for (int64_t b = 0; b < H; b++) acc[b] = (double)orc_f16_to_f32(dest[b]);
  for (int64_t i = 0; i < n; i++) {
    const int64_t b = (int64_t)is[i];
    if (b >= 0 && b < H) acc[b] += (double)orc_f16_to_f32(vs[i]);
  }
  for (int64_t b = 0; b < H; b++) dest[b] = orc_f32_to_f16((float)acc[b]);
  free(acc);
}

float orc_bf16_to_f32(uint16_t h) {
  const uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
/* 16-bit inputs widened to f32, then the f32 matmul: products f32.f16 x * f32.f16 y
 * summed in f32 (for bf16 the widening is bits << 16). */
void orc_widen_f16(const uint16_t *in, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(in[i]);
}
void orc_widen_bf16(const uint16_t *in, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = orc_bf16_to_f32(in[i]);
}

/* -------------------------------------------------------------- radix sort
 * Stable LSD radix sort, 8-bit digits: per pass a histogram of the digit, an
 * exclusive scan of the 256 counts, and an in-order scatter (the composition of
 * tests/issue2234.fut:10-44 with 8-bit instead of 2-bit digits).  Keys compare
 * as unsigned; vals may be NULL. */
static void radix_pass(const uint8_t *kin, uint8_t *kout, const uint8_t *vin, uint8_t *vout,
                       int64_t n, int kb, int vb, int shift) {
  int64_t count[256] = {0}, start[256];
  for (int64_t i = 0; i < n; i++) {
    uint64_t k = 0;
    memcpy(&k, kin + i * kb, (size_t)kb);
    count[(k >> shift) & 0xff]++;
  }
  int64_t acc = 0;
  for (int d = 0; d < 256; d++) {
    start[d] = acc;
    acc += count[d];
  }
  for (int64_t i = 0; i < n; i++) {
    uint64_t k = 0;
    memcpy(&k, kin + i * kb, (size_t)kb);
    const int64_t p = start[(k >> shift) & 0xff]++;
    memcpy(kout + p * kb, kin + i * kb, (size_t)kb);
    if (vin) memcpy(vout + p * vb, vin + i * vb, (size_t)vb);
  }
}
void orc_radix_sort(const void *keys, void *keys_out, const void *vals, void *vals_out,
                    int64_t n, int key_bytes, int val_bytes) {
  const size_t kbytes = (size_t)(n > 0 ? n : 1) * (size_t)key_bytes;
  const size_t vbytes = (size_t)(n > 0 ? n : 1) * (size_t)(val_bytes > 0 ? val_bytes : 1);
  uint8_t *ka = (uint8_t *)malloc(kbytes), *kb2 = (uint8_t *)malloc(kbytes);
  uint8_t *va = vals ? (uint8_t *)malloc(vbytes) : NULL, *vb2 = vals ? (uint8_t *)malloc(vbytes) : NULL;
  memcpy(ka, keys, (size_t)n * (size_t)key_bytes);
  if (vals) memcpy(va, vals, (size_t)n * (size_t)val_bytes);
  for (int pass = 0; pass < key_bytes; pass++) {
    radix_pass(ka, kb2, va, vb2, n, key_bytes, val_bytes, 8 * pass);
    uint8_t *t = ka; ka = kb2; kb2 = t;
    t = va; va = vb2; vb2 = t;
  }
  memcpy(keys_out, ka, (size_t)n * (size_t)key_bytes);
  if (vals) memcpy(vals_out, va, (size_t)n * (size_t)val_bytes);
  free(ka); free(kb2); free(va); free(vb2);
}

/* --------------------------------------------------------- data movement */
/* LMAD copy, element by element in row-major index order: what the reference's
 * generic copy does (rts/c/copy.h:35-53, lmad_copy_elements), for elements of
 * any size.  Offsets and strides count elements. */
static void orc_lmad_rec(int r, uint8_t *dst, const int64_t *dst_strides, const uint8_t *src,
                         const int64_t *src_strides, const int64_t *shape, int64_t es) {
  if (r == 0) {
    memcpy(dst, src, (size_t)es);
    return;
  }
  for (int64_t i = 0; i < shape[0]; i++)
    orc_lmad_rec(r - 1, dst + i * dst_strides[0] * es, dst_strides + 1,
                 src + i * src_strides[0] * es, src_strides + 1, shape + 1, es);
}

void orc_lmad_copy(int elem_bytes, void *dst, int64_t dst_offset, const int64_t *dst_strides,
                   const void *src, int64_t src_offset, const int64_t *src_strides,
                   const int64_t *shape, int rank) {
  for (int i = 0; i < rank; i++)
    if (shape[i] == 0) return;
  orc_lmad_rec(rank, (uint8_t *)dst + dst_offset * elem_bytes, dst_strides,
               (const uint8_t *)src + src_offset * elem_bytes, src_strides, shape, elem_bytes);
}

void orc_transpose_f32(const float *in, float *out, int64_t rows, int64_t cols) {
  for (int64_t i = 0; i < rows; i++)
    for (int64_t j = 0; j < cols; j++) out[j * rows + i] = in[i * cols + j];
}
