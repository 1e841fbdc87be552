/* libfuthark_amd_values.so -- reading and writing Futhark values: the binary
 * data format (docs/binary-data-format.rst; the reference's reader/writer is
 * rts/c/values.h:498-812, pasted into every generated executable) and the
 * textual syntax in both directions (rts/c/values.h:14-491,724-768).  Host memory
 * only.  The server executable and Python tools (futhark_amd/values.py) use it. */
#ifndef FUTHARK_AMD_VALUES_H
#define FUTHARK_AMD_VALUES_H

#include <stdint.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif

struct fv_primtype {
  const char *name;  /* "i32", "bool", ... as Futhark spells the type */
  char binname[5];   /* the four-character tag of the binary format */
  int size;          /* bytes per element */
};

/* NULL if `name` is not one of i8 i16 i32 i64 u8 u16 u32 u64 f16 f32 f64 bool. */
const struct fv_primtype *fv_primtype(const char *name);
/* The same, by the four-character tag ("  i8", " f32", "bool"). */
const struct fv_primtype *fv_primtype_by_tag(const char tag[4]);

#define FV_MAX_RANK 8

/* Reads one value in the binary format.  The value must have element type
 * `expect` and `rank` dimensions (0 = scalar).  On success returns 0, stores the
 * dimensions in shape[0..rank) and a malloc'ed buffer of the elements (row
 * major, host byte order; at least one byte even if empty) in *data.  Returns
 * nonzero and writes a message to `err` (if not NULL, `errlen` bytes) when the
 * input is not binary, has another version, type or rank, or is truncated. */
int fv_read_binary(FILE *f, const struct fv_primtype *expect, int rank, int64_t *shape,
                   void **data, char *err, size_t errlen);

/* Writes one value in the binary format (version 2, little endian). */
int fv_write_binary(FILE *f, const struct fv_primtype *t, int rank, const int64_t *shape,
                    const void *data);

/* Writes one value in Futhark's textual syntax, e.g. [[1i32, 2i32], [3i32, 4i32]],
 * `empty([0][3]i32)` for empty arrays, f32.nan / f32.inf for non-finite floats. */
int fv_write_text(FILE *f, const struct fv_primtype *t, int rank, const int64_t *shape,
                  const void *data);

/* Reads one value in the textual syntax (rts/c/values.h:14-398): nested
 * brackets with rows of equal length, empty([0][3]i32), numbers with optional
 * type suffix and underscores, hexadecimal integers, T.nan / T.inf / -T.inf,
 * true / false, `--` comments.  Results as for fv_read_binary.  f16 literals are
 * narrowed from float by cutting the mantissa, as the reference's reader does. */
int fv_read_text(FILE *f, const struct fv_primtype *expect, int rank, int64_t *shape,
                 void **data, char *err, size_t errlen);

/* Reads one value in either form: binary if the next non-blank character is
 * 'b', else textual (read_array / read_scalar, rts/c/values.h:705-712,814-829). */
int fv_read_value(FILE *f, const struct fv_primtype *expect, int rank, int64_t *shape,
                  void **data, char *err, size_t errlen);

/* 0 if only blanks and `--` comments remain before end of file; otherwise
 * nonzero, and the next value can still be read. */
int fv_end_of_input(FILE *f);

#ifdef __cplusplus
}
#endif
#endif
