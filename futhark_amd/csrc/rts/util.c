/* Small host utilities of the runtime: formatted strings, fatal errors, wall
 * clock and a growable string used for the profiling report
 * (counterparts: rts/c/util.h, rts/c/timing.h). */
#define _POSIX_C_SOURCE 200809L
#include "rts.h"

#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

char *rts_msgprintf(const char *fmt, ...) {
  va_list vl;
  va_start(vl, fmt);
  int needed = vsnprintf(NULL, 0, fmt, vl);
  va_end(vl);
  if (needed < 0) return NULL;
  char *buf = (char *)malloc((size_t)needed + 1);
  if (buf == NULL) return NULL;
  va_start(vl, fmt);
  vsnprintf(buf, (size_t)needed + 1, fmt, vl);
  va_end(vl);
  return buf;
}

void rts_panic(int eval, const char *fmt, ...) {
  va_list vl;
  va_start(vl, fmt);
  fprintf(stderr, "futhark-amd runtime: ");
  vfprintf(stderr, fmt, vl);
  va_end(vl);
  exit(eval);
}

int64_t rts_wall_time_us(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000 + ts.tv_nsec / 1000;
}

void str_builder_init(struct str_builder *b) {
  b->capacity = 256;
  b->used = 0;
  b->str = (char *)malloc(b->capacity);
  b->str[0] = 0;
}

static void str_builder_reserve(struct str_builder *b, size_t extra) {
  while (b->used + extra + 1 > b->capacity) {
    b->capacity *= 2;
    b->str = (char *)realloc(b->str, b->capacity);
  }
}

void str_builder_printf(struct str_builder *b, const char *fmt, ...) {
  va_list vl;
  va_start(vl, fmt);
  int needed = vsnprintf(NULL, 0, fmt, vl);
  va_end(vl);
  if (needed < 0) return;
  str_builder_reserve(b, (size_t)needed);
  va_start(vl, fmt);
  vsnprintf(b->str + b->used, (size_t)needed + 1, fmt, vl);
  va_end(vl);
  b->used += (size_t)needed;
}

void str_builder_json_str(struct str_builder *b, const char *s) {
  str_builder_printf(b, "\"");
  for (; *s; s++) {
    unsigned char c = (unsigned char)*s;
    if (c == '"' || c == '\\') str_builder_printf(b, "\\%c", c);
    else if (c == '\n') str_builder_printf(b, "\\n");
    else if (c < 0x20) str_builder_printf(b, "\\u%04x", c);
    else str_builder_printf(b, "%c", c);
  }
  str_builder_printf(b, "\"");
}
