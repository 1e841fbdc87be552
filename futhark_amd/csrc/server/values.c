/* Binary data format and textual output of Futhark values; see include/futhark_amd_values.h. */
#include "futhark_amd_values.h"

#include <ctype.h>
#include <inttypes.h>
#include <math.h>
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#define FV_BINARY_VERSION 2 /* rts/c/values.h:498 */

static const struct fv_primtype fv_types[] = {
    {"i8", "  i8", 1},  {"i16", " i16", 2}, {"i32", " i32", 4}, {"i64", " i64", 8},
    {"u8", "  u8", 1},  {"u16", " u16", 2}, {"u32", " u32", 4}, {"u64", " u64", 8},
    {"f16", " f16", 2}, {"f32", " f32", 4}, {"f64", " f64", 8}, {"bool", "bool", 1},
};
#define FV_NUM_TYPES ((int)(sizeof(fv_types) / sizeof(fv_types[0])))

const struct fv_primtype *fv_primtype(const char *name) {
  for (int i = 0; i < FV_NUM_TYPES; i++)
    if (strcmp(fv_types[i].name, name) == 0) return &fv_types[i];
  return NULL;
}

const struct fv_primtype *fv_primtype_by_tag(const char tag[4]) {
  for (int i = 0; i < FV_NUM_TYPES; i++)
    if (memcmp(fv_types[i].binname, tag, 4) == 0) return &fv_types[i];
  return NULL;
}

static int host_is_big_endian(void) {
  const uint16_t one = 1;
  return *(const unsigned char *)&one == 0;
}

static void swap_elements(unsigned char *p, size_t count, int size) {
  if (size == 1) return;
  for (size_t i = 0; i < count; i++, p += size)
    for (int a = 0, b = size - 1; a < b; a++, b--) {
      unsigned char t = p[a];
      p[a] = p[b];
      p[b] = t;
    }
}

static int fail(char *err, size_t errlen, const char *fmt, ...) {
  if (err != NULL && errlen > 0) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err, errlen, fmt, ap);
    va_end(ap);
  }
  return 1;
}

int fv_read_binary(FILE *f, const struct fv_primtype *expect, int rank, int64_t *shape,
                   void **data, char *err, size_t errlen) {
  int c;
  do {
    c = getc(f);
  } while (c != EOF && isspace(c));
  if (c != 'b') {
    if (c != EOF) ungetc(c, f);
    return fail(err, errlen, "input is not in the binary format (no leading 'b')");
  }
  const int version = getc(f);
  if (version != FV_BINARY_VERSION)
    return fail(err, errlen, "binary format version %d, expected %d", version, FV_BINARY_VERSION);
  const int dims = getc(f);
  if (dims == EOF) return fail(err, errlen, "truncated header");
  char tag[4];
  if (fread(tag, 1, 4, f) != 4) return fail(err, errlen, "truncated header");
  const struct fv_primtype *t = fv_primtype_by_tag(tag);
  if (t == NULL) return fail(err, errlen, "unknown element type '%.4s'", tag);
  if (t != expect)
    return fail(err, errlen, "expected element type %s, got %s", expect->name, t->name);
  if (dims != rank) return fail(err, errlen, "expected %d dimensions, got %d", rank, dims);
  if (rank > FV_MAX_RANK) return fail(err, errlen, "rank %d not supported", rank);

  uint64_t count = 1;
  for (int i = 0; i < rank; i++) {
    unsigned char b[8];
    if (fread(b, 1, 8, f) != 8) return fail(err, errlen, "truncated shape");
    uint64_t d = 0;
    for (int k = 7; k >= 0; k--) d = (d << 8) | b[k];
    if (d > (uint64_t)INT64_MAX) return fail(err, errlen, "dimension %d too large", i);
    shape[i] = (int64_t)d;
    if (d != 0 && count > UINT64_MAX / d) return fail(err, errlen, "array too large");
    count *= d;
  }
  if (count > SIZE_MAX / (size_t)t->size) return fail(err, errlen, "array too large");
  const size_t bytes = (size_t)count * (size_t)t->size;
  unsigned char *buf = malloc(bytes > 0 ? bytes : 1);
  if (buf == NULL) return fail(err, errlen, "out of memory (%zu bytes)", bytes);
  if (bytes > 0 && fread(buf, 1, bytes, f) != bytes) {
    free(buf);
    return fail(err, errlen, "truncated data: expected %zu bytes of elements", bytes);
  }
  if (host_is_big_endian()) swap_elements(buf, (size_t)count, t->size);
  *data = buf;
  return 0;
}

int fv_write_binary(FILE *f, const struct fv_primtype *t, int rank, const int64_t *shape,
                    const void *data) {
  if (rank < 0 || rank > FV_MAX_RANK) return 1;
  putc('b', f);
  putc(FV_BINARY_VERSION, f);
  putc(rank, f);
  fwrite(t->binname, 1, 4, f);
  size_t count = 1;
  for (int i = 0; i < rank; i++) {
    uint64_t d = (uint64_t)shape[i];
    unsigned char b[8];
    for (int k = 0; k < 8; k++, d >>= 8) b[k] = (unsigned char)(d & 0xff);
    fwrite(b, 1, 8, f);
    count *= (size_t)shape[i];
  }
  if (count > 0) {
    if (host_is_big_endian()) {
      unsigned char *tmp = malloc(count * (size_t)t->size);
      if (tmp == NULL) return 1;
      memcpy(tmp, data, count * (size_t)t->size);
      swap_elements(tmp, count, t->size);
      fwrite(tmp, (size_t)t->size, count, f);
      free(tmp);
    } else {
      fwrite(data, (size_t)t->size, count, f);
    }
  }
  return ferror(f) ? 1 : 0;
}

/* binary16 -> float, for printing only. */
static float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31;
  const int exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0x1f) {
    bits = sign | 0x7f800000u | (man << 13);
  } else if (exp != 0) {
    bits = sign | ((uint32_t)(exp - 15 + 127) << 23) | (man << 13);
  } else if (man == 0) {
    bits = sign;
  } else {
    int e = -1;
    do {
      man <<= 1;
      e++;
    } while ((man & 0x400u) == 0);
    bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
  }
  float out;
  memcpy(&out, &bits, 4);
  return out;
}

/* Shortest-round-trip digit counts as the reference prints them
 * (rts/c/values.h:448-485): 9 significant digits for f16/f32, 17 for f64. */
static void write_float(FILE *f, double v, const char *suffix, int digits) {
  if (isnan(v)) fprintf(f, "%s.nan", suffix);
  else if (isinf(v)) fprintf(f, "%s%s.inf", v < 0 ? "-" : "", suffix);
  else fprintf(f, "%.*g%s", digits, v, suffix);
}

static void write_elem(FILE *f, const struct fv_primtype *t, const unsigned char *p) {
  const char *n = t->name;
  if (strcmp(n, "bool") == 0) {
    fputs(*p ? "true" : "false", f);
  } else if (n[0] == 'f') {
    if (t->size == 2) {
      uint16_t h;
      memcpy(&h, p, 2);
      write_float(f, half_bits_to_float(h), "f16", 9);
    } else if (t->size == 4) {
      float v;
      memcpy(&v, p, 4);
      write_float(f, v, "f32", 9);
    } else {
      double v;
      memcpy(&v, p, 8);
      write_float(f, v, "f64", 17);
    }
  } else {
    const int is_signed = n[0] == 'i';
    int64_t sv = 0;
    uint64_t uv = 0;
    switch (t->size) {
      case 1: sv = *(const int8_t *)p; uv = *p; break;
      case 2: { int16_t a; uint16_t b; memcpy(&a, p, 2); memcpy(&b, p, 2); sv = a; uv = b; } break;
      case 4: { int32_t a; uint32_t b; memcpy(&a, p, 4); memcpy(&b, p, 4); sv = a; uv = b; } break;
      default: memcpy(&sv, p, 8); memcpy(&uv, p, 8); break;
    }
    if (is_signed) fprintf(f, "%" PRId64 "%s", sv, n);
    else fprintf(f, "%" PRIu64 "%s", uv, n);
  }
}

static const unsigned char *write_text_rec(FILE *f, const struct fv_primtype *t, int rank,
                                           const int64_t *shape, const unsigned char *p) {
  if (rank == 0) {
    write_elem(f, t, p);
    return p + t->size;
  }
  putc('[', f);
  for (int64_t i = 0; i < shape[0]; i++) {
    if (i > 0) fputs(", ", f);
    p = write_text_rec(f, t, rank - 1, shape + 1, p);
  }
  putc(']', f);
  return p;
}

int fv_write_text(FILE *f, const struct fv_primtype *t, int rank, const int64_t *shape,
                  const void *data) {
  int empty = 0;
  for (int i = 0; i < rank; i++) empty |= shape[i] == 0;
  if (rank > 0 && empty) {
    fputs("empty(", f);
    for (int i = 0; i < rank; i++) fprintf(f, "[%" PRId64 "]", shape[i]);
    fprintf(f, "%s)", t->name);
  } else {
    write_text_rec(f, t, rank, shape, data);
  }
  return ferror(f) ? 1 : 0;
}

int fv_end_of_input(FILE *f) {
  int c;
  do {
    c = getc(f);
  } while (c != EOF && isspace(c));
  if (c == EOF) return 0;
  ungetc(c, f);
  return 1;
}
