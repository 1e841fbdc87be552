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

/* ------------------------------------------------------------ textual input
 * The syntax rts/c/values.h:14-398 accepts.  Tokens are maximal runs of
 * letters, digits and . - + _, or single other characters; `--` starts a
 * comment that runs to the end of the line.  A value of rank r is r levels of
 * [ ... , ... ] with rows of equal length, or empty([d0]...[dr-1]T) with some
 * dimension 0.  Numbers may contain underscores and may carry their type as a
 * suffix; integers also come in hexadecimal and octal (C's %i); u64 is decimal
 * only; floats have T.nan, T.inf, -T.inf; bool is true / false. */
struct text_parser {
  FILE *f;
  char tok[128];
  int have; /* tok holds a token that was peeked at but not consumed */
};

static int is_constituent(int c) {
  return isalnum(c) || c == '.' || c == '-' || c == '+' || c == '_';
}

/* An empty token means end of input. */
static const char *peek_token(struct text_parser *p) {
  if (p->have) return p->tok;
  p->have = 1;
  int c, n = 0;
  for (;;) {
    do {
      c = getc(p->f);
    } while (c != EOF && isspace(c));
    if (c != '-') break;
    const int d = getc(p->f);
    if (d != '-') {
      if (d != EOF) ungetc(d, p->f);
      break;
    }
    while (c != '\n' && c != EOF) c = getc(p->f);
  }
  if (c == EOF) {
    p->tok[0] = 0;
    return p->tok;
  }
  p->tok[n++] = (char)c;
  if (is_constituent(c)) {
    while ((c = getc(p->f)) != EOF && is_constituent(c))
      if (n < (int)sizeof(p->tok) - 1) p->tok[n++] = (char)c;
    if (c != EOF) ungetc(c, p->f);
  }
  p->tok[n] = 0;
  return p->tok;
}

static const char *next_token(struct text_parser *p) {
  const char *t = peek_token(p);
  p->have = 0;
  return t;
}

static int accept_token(struct text_parser *p, const char *want) {
  if (strcmp(peek_token(p), want) != 0) return 0;
  p->have = 0;
  return 1;
}

/* float -> binary16 the way the reference's reader narrows (float2halfbits,
 * rts/c/half.h:220-228, tables after van der Zijp): the mantissa is cut, not
 * rounded; too small goes to zero, too large to infinity. */
static uint16_t float_to_half_bits_truncating(float v) {
  uint32_t x;
  memcpy(&x, &v, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const int e = (int)((x >> 23) & 0xff);
  const uint32_t man = x & 0x7fffffu;
  if (e < 103) return sign;
  if (e < 113) return (uint16_t)(sign | ((0x0400u >> (113 - e)) + (man >> (126 - e))));
  if (e < 143) return (uint16_t)(sign | ((uint32_t)(e - 112) << 10) | (man >> 13));
  if (e < 255) return (uint16_t)(sign | 0x7c00u);
  return (uint16_t)(sign | 0x7c00u | (man >> 13));
}

/* The rest of a number token must be empty or the type's name. */
static int suffix_ok(const char *rest, const char *name) {
  return *rest == 0 || strcmp(rest, name) == 0;
}

static int parse_scalar(const char *token, const struct fv_primtype *t, unsigned char *dst) {
  char buf[128];
  size_t n = 0;
  for (const char *r = token; *r && n < sizeof(buf) - 1; r++)
    if (*r != '_') buf[n++] = *r;
  buf[n] = 0;
  const char *name = t->name;
  if (strcmp(name, "bool") == 0) {
    if (strcmp(token, "true") == 0) *dst = 1;
    else if (strcmp(token, "false") == 0) *dst = 0;
    else return 1;
    return 0;
  }
  if (name[0] == 'f') {
    char special[16];
    double v;
    int sign = 1;
    const char *b = buf;
    snprintf(special, sizeof special, "%s.nan", name);
    if (strcmp(b, special) == 0) {
      v = (double)NAN;
    } else {
      snprintf(special, sizeof special, "%s.inf", name);
      if (b[0] == '-' && strcmp(b + 1, special) == 0) sign = -1, b++;
      if (strcmp(b, special) == 0) {
        v = sign * (double)INFINITY;
      } else {
        char *end;
        if (t->size == 8) v = strtod(buf, &end);
        else v = (double)strtof(buf, &end);
        if (end == buf || !suffix_ok(end, name)) return 1;
      }
    }
    if (t->size == 8) {
      memcpy(dst, &v, 8);
    } else if (t->size == 4) {
      const float f = (float)v;
      memcpy(dst, &f, 4);
    } else {
      const uint16_t h = float_to_half_bits_truncating((float)v);
      memcpy(dst, &h, 2);
    }
    return 0;
  }
  /* integers: the digits the way scanf's %i reads them (sign, 0x, leading 0),
   * u64 the way %u does; narrower types keep the low bits */
  char *end;
  if (strcmp(name, "u64") == 0) {
    const char *d = buf;
    if (*d == '+') d++;
    if (!isdigit((unsigned char)*d)) return 1;
    const uint64_t v = strtoull(d, &end, 10);
    if (!suffix_ok(end, name)) return 1;
    memcpy(dst, &v, 8);
    return 0;
  }
  const char *d = buf;
  if (*d == '-' || *d == '+') d++;
  if (!isdigit((unsigned char)*d)) return 1;
  const long long v = strtoll(buf, &end, 0);
  if (end == buf || !suffix_ok(end, name)) return 1;
  switch (t->size) {
    case 1: { const int8_t x = (int8_t)v; memcpy(dst, &x, 1); } break;
    case 2: { const int16_t x = (int16_t)v; memcpy(dst, &x, 2); } break;
    case 4: { const int32_t x = (int32_t)v; memcpy(dst, &x, 4); } break;
    default: { const int64_t x = (int64_t)v; memcpy(dst, &x, 8); } break;
  }
  return 0;
}

struct text_array {
  const struct fv_primtype *t;
  int rank;
  int64_t *shape;
  char known[FV_MAX_RANK];
  unsigned char *elems;
  size_t used, space; /* in elements */
};

static int parse_level(struct text_parser *p, struct text_array *a, int level) {
  if (!accept_token(p, "[")) return 1;
  int64_t count = 0;
  while (strcmp(peek_token(p), "]") != 0) {
    if (level == a->rank - 1) {
      if (a->used == a->space) {
        a->space *= 2;
        unsigned char *grown = realloc(a->elems, a->space * (size_t)a->t->size);
        if (grown == NULL) return 1;
        a->elems = grown;
      }
      const char *tok = next_token(p);
      if (*tok == 0 || parse_scalar(tok, a->t, a->elems + a->used * (size_t)a->t->size) != 0)
        return 1;
      a->used++;
    } else if (parse_level(p, a, level + 1) != 0) {
      return 1;
    }
    count++;
    if (!accept_token(p, ",")) break; /* a comma may also precede the closing bracket */
  }
  if (!accept_token(p, "]")) return 1;
  if (a->known[level]) return a->shape[level] != count;
  a->known[level] = 1;
  a->shape[level] = count;
  return 0;
}

static int parse_empty(struct text_parser *p, const struct fv_primtype *t, int rank,
                       int64_t *shape) {
  if (!accept_token(p, "empty") || !accept_token(p, "(")) return 1;
  int some_zero = 0;
  for (int i = 0; i < rank; i++) {
    if (!accept_token(p, "[")) return 1;
    const char *tok = next_token(p);
    char *end;
    if (!isdigit((unsigned char)*tok)) return 1;
    shape[i] = (int64_t)strtoull(tok, &end, 10);
    if (*end != 0 || !accept_token(p, "]")) return 1;
    some_zero |= shape[i] == 0;
  }
  if (!accept_token(p, t->name) || !accept_token(p, ")")) return 1;
  return !some_zero;
}

int fv_read_text(FILE *f, const struct fv_primtype *t, int rank, int64_t *shape, void **data,
                 char *err, size_t errlen) {
  if (rank < 0 || rank > FV_MAX_RANK) return fail(err, errlen, "rank %d not supported", rank);
  struct text_parser p = {f, {0}, 0};
  if (*peek_token(&p) == 0) return fail(err, errlen, "end of input where a value was expected");
  if (rank == 0) {
    unsigned char *buf = malloc(8);
    if (buf == NULL) return fail(err, errlen, "out of memory");
    if (parse_scalar(next_token(&p), t, buf) != 0) {
      free(buf);
      return fail(err, errlen, "not a value of type %s: %s", t->name, p.tok);
    }
    *data = buf;
    return 0;
  }
  if (strcmp(peek_token(&p), "empty") == 0) {
    if (parse_empty(&p, t, rank, shape) != 0)
      return fail(err, errlen, "malformed empty(...) for an array of %s of rank %d", t->name, rank);
    *data = malloc(1);
    return *data == NULL;
  }
  struct text_array a = {t, rank, shape, {0}, malloc(16 * (size_t)t->size), 0, 16};
  if (a.elems == NULL) return fail(err, errlen, "out of memory");
  if (parse_level(&p, &a, 0) != 0) {
    free(a.elems);
    return fail(err, errlen, "malformed array of %s of rank %d near '%s'", t->name, rank, p.tok);
  }
  /* dimensions inside an empty outer dimension were never seen */
  for (int i = 0; i < rank; i++)
    if (!a.known[i]) shape[i] = 0;
  *data = a.elems;
  return 0;
}

int fv_read_value(FILE *f, const struct fv_primtype *t, int rank, int64_t *shape, void **data,
                  char *err, size_t errlen) {
  int c;
  do {
    c = getc(f);
  } while (c != EOF && isspace(c));
  if (c != EOF) ungetc(c, f);
  /* no textual value starts with the letter b (rts/c/values.h:590-610) */
  if (c == 'b') return fv_read_binary(f, t, rank, shape, data, err, errlen);
  return fv_read_text(f, t, rank, shape, data, err, errlen);
}

int fv_end_of_input(FILE *f) {
  /* blanks and `--` comments may follow the last value (end_of_input,
   * rts/c/values.h:713-722); whatever else is found stays in the stream.  A `-`
   * that does not open a comment takes two characters to recognise, and ISO C
   * promises only one character of push-back: on a stream that can seek, the
   * position before the `-` is restored instead; on a pipe the second push-back
   * is left to the C library (glibc keeps it), and should it be refused the
   * answer is still right, only the `-` is gone from the stream. */
  for (;;) {
    fpos_t before;
    const int can_seek = fgetpos(f, &before) == 0;
    int c = getc(f);
    if (c == EOF) return 0;
    if (isspace(c)) continue;
    if (c == '-') {
      int c2 = getc(f);
      if (c2 == '-') {
        while (c2 != EOF && c2 != '\n') c2 = getc(f);
        continue;
      }
      if (can_seek && fsetpos(f, &before) == 0) return 1;
      if (c2 != EOF) ungetc(c2, f);
    }
    ungetc(c, f);
    return 1;
  }
}
