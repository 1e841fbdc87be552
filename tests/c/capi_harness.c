/* A C program written against include/segops.h the way the reference's own C
 * harnesses are written against a generated header (tests_lib/c/test_c.c:
 * repeated context creation; test_index.c: index errors; test_raw.c: raw
 * arrays; test_f.c: use from another thread; test_e.c: errors are not sticky;
 * test_g.c: size constraints between arguments).  Built into
 * futhark_amd/bin/capi-harness; exits 0 and prints one "ok NAME" line per
 * section.  With --no-device it checks instead that a context without a device
 * reports an error through futhark_context_get_error and can be freed. */
#include <assert.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "segops.h"

#define CHECK(cond)                                                           \
  do {                                                                        \
    if (!(cond)) {                                                            \
      fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
      exit(1);                                                                \
    }                                                                         \
  } while (0)

static void section_lifecycle(void) {
  /* Contexts must clean up after themselves: twenty rounds of 1 GiB each. */
  for (int i = 0; i < 20; i++) {
    struct futhark_context_config *cfg = futhark_context_config_new();
    struct futhark_context *ctx = futhark_context_new(cfg);
    CHECK(futhark_context_get_error(ctx) == NULL);
    struct futhark_i64_1d *arr;
    CHECK(futhark_entry_iota_i64(ctx, &arr, (1 << 30) / 8) == 0);
    CHECK(futhark_context_sync(ctx) == 0);
    CHECK(futhark_free_i64_1d(ctx, arr) == 0);
    futhark_context_free(ctx);
    futhark_context_config_free(cfg);
  }
  puts("ok lifecycle");
}

static void section_index(struct futhark_context *ctx) {
  char *err;
  struct futhark_i64_1d *a;
  CHECK(futhark_entry_iota_i64(ctx, &a, 10) == 0);
  CHECK(futhark_index_i64_1d(ctx, NULL, a, 100) == 1); /* too high */
  CHECK((err = futhark_context_get_error(ctx)) != NULL);
  CHECK(strstr(err, "Index out of bounds") != NULL);
  free(err);
  CHECK(futhark_context_get_error(ctx) == NULL); /* reading the error clears it */
  CHECK(futhark_index_i64_1d(ctx, NULL, a, -1) == 1); /* negative */
  CHECK((err = futhark_context_get_error(ctx)) != NULL);
  free(err);
  int64_t x = -1;
  CHECK(futhark_index_i64_1d(ctx, &x, a, 5) == 0);
  CHECK(futhark_context_sync(ctx) == 0);
  CHECK(x == 5);
  CHECK(futhark_shape_i64_1d(ctx, a)[0] == 10);
  CHECK(futhark_free_i64_1d(ctx, a) == 0);

  float host[12];
  for (int i = 0; i < 12; i++) host[i] = (float)(i / 4 + i % 4); /* b[i][j] = i + j */
  struct futhark_f32_2d *b = futhark_new_f32_2d(ctx, host, 3, 4);
  CHECK(b != NULL);
  CHECK(futhark_index_f32_2d(ctx, NULL, b, 0, 4) == 1); /* one dimension out of range */
  CHECK((err = futhark_context_get_error(ctx)) != NULL);
  free(err);
  float y = 0;
  CHECK(futhark_index_f32_2d(ctx, &y, b, 2, 3) == 0);
  CHECK(futhark_context_sync(ctx) == 0);
  CHECK(y == 5.0f);
  CHECK(futhark_free_f32_2d(ctx, b) == 0);
  puts("ok index");
}

static void section_raw(struct futhark_context *ctx) {
  /* Device memory owned by the caller (here: borrowed from another array)
   * wrapped as an array, used as input, and left alone when freed. */
  int32_t data[3] = {1, 2, 3};
  struct futhark_i32_1d *owner = futhark_new_i32_1d(ctx, data, 3);
  CHECK(owner != NULL);
  futhark_device_ptr p = futhark_values_raw_i32_1d(ctx, owner);
  CHECK(p != NULL);
  struct futhark_i32_1d *in = futhark_new_raw_i32_1d(ctx, p, 3);
  CHECK(in != NULL);
  struct futhark_i32_1d *out;
  CHECK(futhark_entry_scan_add_i32(ctx, &out, in) == FUTHARK_SUCCESS);
  int32_t got[3];
  CHECK(futhark_values_i32_1d(ctx, out, got) == 0);
  CHECK(futhark_context_sync(ctx) == FUTHARK_SUCCESS);
  CHECK(got[0] == 1 && got[1] == 3 && got[2] == 6);
  CHECK(futhark_free_i32_1d(ctx, in) == 0);
  /* the memory is still the owner's */
  int32_t again[3];
  CHECK(futhark_values_i32_1d(ctx, owner, again) == 0);
  CHECK(futhark_context_sync(ctx) == 0);
  CHECK(memcmp(again, data, sizeof data) == 0);
  CHECK(futhark_free_i32_1d(ctx, out) == 0);
  CHECK(futhark_free_i32_1d(ctx, owner) == 0);
  puts("ok raw");
}

struct thread_args {
  struct futhark_context *ctx;
  struct futhark_i32_1d *xs;
  int n;
};

static void *thread_fn(void *arg) {
  struct thread_args *a = arg;
  struct futhark_i32_1d *out = NULL;
  CHECK(futhark_entry_exscan_add_i32(a->ctx, &out, a->xs) == 0);
  int32_t *host = malloc(sizeof(int32_t) * (size_t)a->n);
  CHECK(futhark_values_i32_1d(a->ctx, out, host) == 0);
  CHECK(futhark_context_sync(a->ctx) == 0);
  for (int i = 0; i < a->n; i++) CHECK(host[i] == i * (i - 1) / 2);
  free(host);
  CHECK(futhark_free_i32_1d(a->ctx, out) == 0);
  CHECK(futhark_free_i32_1d(a->ctx, a->xs) == 0);
  return NULL;
}

static void section_threads(struct futhark_context *ctx) {
  enum { N = 5000 };
  static int32_t xs[N];
  for (int i = 0; i < N; i++) xs[i] = i;
  struct thread_args args = {ctx, futhark_new_i32_1d(ctx, xs, N), N};
  CHECK(args.xs != NULL);
  pthread_t tid;
  CHECK(pthread_create(&tid, NULL, thread_fn, &args) == 0);
  CHECK(pthread_join(tid, NULL) == 0);
  puts("ok threads");
}

static void section_errors_are_not_sticky(struct futhark_context *ctx) {
  uint8_t flags[4] = {1, 0, 1, 0};
  float vs3[3] = {1, 2, 3}, vs4[4] = {1, 2, 3, 4};
  struct futhark_u8_1d *f = futhark_new_u8_1d(ctx, flags, 4);
  struct futhark_f32_1d *v3 = futhark_new_f32_1d(ctx, vs3, 3);
  struct futhark_f32_1d *v4 = futhark_new_f32_1d(ctx, vs4, 4);
  struct futhark_f32_1d *out = NULL;
  /* sizes that must agree do not: nonzero, a message, outputs untouched */
  CHECK(futhark_entry_segscan_add_f32(ctx, &out, f, v3) != 0);
  CHECK(out == NULL);
  char *err = futhark_context_get_error(ctx);
  CHECK(err != NULL && strstr(err, "invalid sizes") != NULL);
  free(err);
  /* the next call is unaffected */
  CHECK(futhark_entry_segscan_add_f32(ctx, &out, f, v4) == 0);
  float got[4];
  CHECK(futhark_values_f32_1d(ctx, out, got) == 0);
  CHECK(futhark_context_sync(ctx) == 0);
  CHECK(got[0] == 1 && got[1] == 3 && got[2] == 3 && got[3] == 7);
  CHECK(futhark_free_f32_1d(ctx, out) == 0);
  CHECK(futhark_free_f32_1d(ctx, v3) == 0 && futhark_free_f32_1d(ctx, v4) == 0);
  CHECK(futhark_free_u8_1d(ctx, f) == 0);
  puts("ok errors_are_not_sticky");
}

static void section_two_results_and_report(struct futhark_context *ctx) {
  uint32_t keys[6] = {5, 1, 5, 0, 1, 9};
  int32_t vals[6] = {0, 1, 2, 3, 4, 5};
  struct futhark_u32_1d *k = futhark_new_u32_1d(ctx, keys, 6), *ko;
  struct futhark_i32_1d *v = futhark_new_i32_1d(ctx, vals, 6), *vo;
  struct futhark_opaque_tup2_arr1d_u32_arr1d_i32 *sorted;
  futhark_context_unpause_profiling(ctx);
  CHECK(futhark_entry_radix_sort_pairs_u32_i32(ctx, &sorted, k, v) == 0);
  /* a tuple result is one opaque value; its fields are projected out
   * (tests_lib/c/test_b.c) and outlive it */
  CHECK(futhark_project_opaque_tup2_arr1d_u32_arr1d_i32_0(ctx, &ko, sorted) == 0);
  CHECK(futhark_project_opaque_tup2_arr1d_u32_arr1d_i32_1(ctx, &vo, sorted) == 0);
  CHECK(futhark_free_opaque_tup2_arr1d_u32_arr1d_i32(ctx, sorted) == 0);
  uint32_t kh[6];
  int32_t vh[6];
  CHECK(futhark_values_u32_1d(ctx, ko, kh) == 0 && futhark_values_i32_1d(ctx, vo, vh) == 0);
  CHECK(futhark_context_sync(ctx) == 0);
  const uint32_t kw[6] = {0, 1, 1, 5, 5, 9};
  const int32_t vw[6] = {3, 1, 4, 0, 2, 5}; /* stable */
  CHECK(memcmp(kh, kw, sizeof kw) == 0 && memcmp(vh, vw, sizeof vw) == 0);
  char *report = futhark_context_report(ctx);
  CHECK(report != NULL && strstr(report, "\"events\"") != NULL && strstr(report, "radix_sort") != NULL);
  free(report);
  futhark_context_pause_profiling(ctx);
  CHECK(futhark_free_u32_1d(ctx, k) == 0 && futhark_free_u32_1d(ctx, ko) == 0);
  CHECK(futhark_free_i32_1d(ctx, v) == 0 && futhark_free_i32_1d(ctx, vo) == 0);
  CHECK(futhark_context_clear_caches(ctx) == 0);
  puts("ok two_results_and_report");
}

int main(int argc, char **argv) {
  if (argc > 1 && strcmp(argv[1], "--no-device") == 0) {
    struct futhark_context_config *cfg = futhark_context_config_new();
    struct futhark_context *ctx = futhark_context_new(cfg);
    CHECK(ctx != NULL);
    char *err = futhark_context_get_error(ctx);
    CHECK(err != NULL);
    printf("ok no_device: %s", err);
    free(err);
    futhark_context_free(ctx);
    futhark_context_config_free(cfg);
    return 0;
  }
  section_lifecycle();
  struct futhark_context_config *cfg = futhark_context_config_new();
  futhark_context_config_set_profiling(cfg, 1);
  CHECK(futhark_context_config_set_tuning_param(cfg, "no.such.parameter", 1) == 1);
  CHECK(futhark_context_config_set_tuning_param(cfg, futhark_get_tuning_param_name(0), 4096) == 0);
  struct futhark_context *ctx = futhark_context_new(cfg);
  CHECK(futhark_context_get_error(ctx) == NULL);
  futhark_context_pause_profiling(ctx);
  section_index(ctx);
  section_raw(ctx);
  section_threads(ctx);
  section_errors_are_not_sticky(ctx);
  section_two_results_and_report(ctx);
  futhark_context_free(ctx);
  futhark_context_config_free(cfg);
  puts("ok all");
  return 0;
}
