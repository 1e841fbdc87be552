/*
 * context.c -- configuration and context objects of the generated-library API,
 * and the HIP backend under them.
 *
 * Public functions and their behaviour follow docs/c-api.rst:74-200,609-669 and
 * the reference implementations in rts/c/context.h:89-211, rts/c/gpu.h:54-135
 * and rts/c/backends/hip.h:96-160,579-703.  Differences that a caller can see:
 *   - kernels are prebuilt for gfx950, so nothing is compiled at context
 *     creation; build options, the program text and the cache file are stored
 *     but have no effect;
 *   - when no usable device exists, futhark_context_new reports it through
 *     futhark_context_get_error instead of terminating the process.
 */
#define _POSIX_C_SOURCE 200809L
#include "rts.h"

#include <assert.h>
#include <ctype.h>
#include <stdlib.h>
#include <string.h>

#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

/* ---------------------------------------------------------------- errors */

void rts_set_error(struct futhark_context *ctx, char *msg) {
  pthread_mutex_lock(&ctx->error_lock);
  if (ctx->error == NULL) ctx->error = msg;
  else free(msg);
  pthread_mutex_unlock(&ctx->error_lock);
}

/* Turns a HIP status into a runtime status, recording a message. */
static int hip_check(struct futhark_context *ctx, hipError_t e, const char *what) {
  if (e == hipSuccess) return FUTHARK_SUCCESS;
  rts_set_error(ctx, rts_msgprintf("%s failed with error code %d (%s)\n", what, (int)e,
                                   hipGetErrorString(e)));
  return e == hipErrorOutOfMemory ? FUTHARK_OUT_OF_MEMORY : 1;
}

char *futhark_context_get_error(struct futhark_context *ctx) {
  pthread_mutex_lock(&ctx->error_lock);
  char *e = ctx->error;
  ctx->error = NULL;
  pthread_mutex_unlock(&ctx->error_lock);
  return e;
}

/* ---------------------------------------------------------------- config */

struct futhark_context_config *futhark_context_config_new(void) {
  struct futhark_context_config *cfg =
      (struct futhark_context_config *)calloc(1, sizeof(struct futhark_context_config));
  if (cfg == NULL) return NULL;
  const struct rts_program *p = &futhark_program;
  cfg->num_tuning_params = p->num_tuning_params;
  cfg->tuning_params = (struct tuning_param *)calloc((size_t)p->num_tuning_params + 1,
                                                     sizeof(struct tuning_param));
  for (int i = 0; i < p->num_tuning_params; i++) {
    cfg->tuning_params[i].name = p->tuning_param_names[i];
    cfg->tuning_params[i].param_class = p->tuning_param_classes[i];
    cfg->tuning_params[i].default_value = p->tuning_param_defaults[i];
    cfg->tuning_params[i].val = p->tuning_param_defaults[i];
    cfg->tuning_params[i].set = false;
  }
  cfg->preferred_device = strdup("");
  cfg->preferred_device_num = 0;
  cfg->unified_memory = 0;
  cfg->default_block_size = 256;
  cfg->default_tile_size = 32;
  cfg->default_reg_tile_size = 2;
  cfg->default_threshold = 32 * 1024;
  cfg->program_text = strdup("");
  cfg->build_opts = (char **)calloc(1, sizeof(char *));
  return cfg;
}

void futhark_context_config_free(struct futhark_context_config *cfg) {
  assert(!cfg->in_use);
  for (int i = 0; i < cfg->num_build_opts; i++) free(cfg->build_opts[i]);
  free(cfg->build_opts);
  free(cfg->preferred_device);
  free(cfg->program_text);
  free(cfg->cache_fname);
  free(cfg->tuning_params);
  free(cfg);
}

void futhark_context_config_set_debugging(struct futhark_context_config *cfg, int flag) {
  cfg->profiling = cfg->logging = cfg->debugging = flag;
}
void futhark_context_config_set_profiling(struct futhark_context_config *cfg, int flag) {
  cfg->profiling = flag;
}
void futhark_context_config_set_logging(struct futhark_context_config *cfg, int flag) {
  cfg->logging = flag;
}
void futhark_context_config_set_cache_file(struct futhark_context_config *cfg, const char *f) {
  free(cfg->cache_fname);
  cfg->cache_fname = strdup(f);
}

int futhark_get_tuning_param_count(void) { return futhark_program.num_tuning_params; }
const char *futhark_get_tuning_param_name(int i) { return futhark_program.tuning_param_names[i]; }
const char *futhark_get_tuning_param_class(int i) {
  return futhark_program.tuning_param_classes[i];
}

int futhark_context_config_set_tuning_param(struct futhark_context_config *cfg,
                                            const char *param_name, size_t new_value) {
  for (int i = 0; i < cfg->num_tuning_params; i++) {
    if (strcmp(param_name, cfg->tuning_params[i].name) == 0) {
      cfg->tuning_params[i].val = (int64_t)new_value;
      cfg->tuning_params[i].set = true;
      return 0;
    }
  }
  static const struct {
    const char *name;
    size_t offset;
  } generic[] = {
      {"default_thread_block_size", offsetof(struct futhark_context_config, default_block_size)},
      {"default_group_size", offsetof(struct futhark_context_config, default_block_size)},
      {"default_grid_size", offsetof(struct futhark_context_config, default_grid_size)},
      {"default_num_groups", offsetof(struct futhark_context_config, default_grid_size)},
      {"default_threshold", offsetof(struct futhark_context_config, default_threshold)},
      {"default_tile_size", offsetof(struct futhark_context_config, default_tile_size)},
      {"default_reg_tile_size", offsetof(struct futhark_context_config, default_reg_tile_size)},
      {"default_cache", offsetof(struct futhark_context_config, default_cache)},
      {"default_registers", offsetof(struct futhark_context_config, default_registers)},
  };
  for (size_t i = 0; i < sizeof(generic) / sizeof(generic[0]); i++) {
    if (strcmp(param_name, generic[i].name) == 0) {
      *(size_t *)((char *)cfg + generic[i].offset) = new_value;
      return 0;
    }
  }
  return 1;
}

void futhark_context_config_set_default_thread_block_size(struct futhark_context_config *cfg,
                                                          int size) {
  cfg->default_block_size = (size_t)size;
}
void futhark_context_config_set_default_group_size(struct futhark_context_config *cfg, int size) {
  futhark_context_config_set_default_thread_block_size(cfg, size);
}
void futhark_context_config_set_default_grid_size(struct futhark_context_config *cfg, int num) {
  cfg->default_grid_size = (size_t)num;
}
void futhark_context_config_set_default_num_groups(struct futhark_context_config *cfg, int num) {
  futhark_context_config_set_default_grid_size(cfg, num);
}
void futhark_context_config_set_default_tile_size(struct futhark_context_config *cfg, int size) {
  cfg->default_tile_size = (size_t)size;
}
void futhark_context_config_set_default_reg_tile_size(struct futhark_context_config *cfg,
                                                      int size) {
  cfg->default_reg_tile_size = (size_t)size;
}
void futhark_context_config_set_default_cache(struct futhark_context_config *cfg, int size) {
  cfg->default_cache = (size_t)size;
}
void futhark_context_config_set_default_registers(struct futhark_context_config *cfg, int size) {
  cfg->default_registers = (size_t)size;
}
void futhark_context_config_set_default_threshold(struct futhark_context_config *cfg, int size) {
  cfg->default_threshold = (size_t)size;
}

void futhark_context_config_add_build_option(struct futhark_context_config *cfg,
                                             const char *opt) {
  cfg->build_opts =
      (char **)realloc(cfg->build_opts, (size_t)(cfg->num_build_opts + 2) * sizeof(char *));
  cfg->build_opts[cfg->num_build_opts++] = strdup(opt);
  cfg->build_opts[cfg->num_build_opts] = NULL;
}

/* "#k" picks the k-th matching device; the rest of the string must occur in
 * the device name (hip.h:130-146). */
void futhark_context_config_set_device(struct futhark_context_config *cfg, const char *s) {
  int k = 0;
  if (*s == '#') {
    s++;
    while (isdigit((unsigned char)*s)) k = k * 10 + (*s++ - '0');
    while (isspace((unsigned char)*s)) s++;
  }
  free(cfg->preferred_device);
  cfg->preferred_device = strdup(s);
  cfg->preferred_device_num = k;
}

const char *futhark_context_config_get_program(struct futhark_context_config *cfg) {
  return cfg->program_text;
}
void futhark_context_config_set_program(struct futhark_context_config *cfg, const char *s) {
  free(cfg->program_text);
  cfg->program_text = strdup(s);
}
void futhark_context_config_set_unified_memory(struct futhark_context_config *cfg, int flag) {
  cfg->unified_memory = flag;
}

/* ---------------------------------------------------------------- device */

static int pick_device(struct futhark_context *ctx) {
  struct futhark_context_config *cfg = ctx->cfg;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) return 1;
  int matches = 0;
  for (int i = 0; i < count; i++) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, i) != hipSuccess) continue;
    if (cfg->logging) fprintf(ctx->log, "Device #%d: name=\"%s\"\n", i, prop.name);
    if (strstr(prop.name, cfg->preferred_device) != NULL &&
        matches++ == cfg->preferred_device_num) {
      ctx->device = i;
      snprintf(ctx->device_name, sizeof(ctx->device_name), "%s", prop.name);
      ctx->num_cus = prop.multiProcessorCount;
      ctx->max_shared_memory = prop.sharedMemPerBlock;
      ctx->max_block_size = (size_t)prop.maxThreadsPerBlock;
      ctx->l2_cache_bytes = (size_t)prop.l2CacheSize;
      if (cfg->logging) fprintf(ctx->log, "Using device #%d\n", i);
      return 0;
    }
  }
  return 1;
}

static int backend_setup(struct futhark_context *ctx) {
  if (hipInit(0) != hipSuccess || pick_device(ctx) != 0) {
    rts_set_error(ctx, strdup("No suitable HIP device found.\n"));
    return 1;
  }
  if (hip_check(ctx, hipSetDevice(ctx->device), "hipSetDevice") != 0) return 1;
  if (ctx->cfg->unified_memory == 2) {
    int managed = 0;
    hipDeviceGetAttribute(&managed, hipDeviceAttributeManagedMemory, ctx->device);
    ctx->cfg->unified_memory = managed;
  }
  ctx->unified = ctx->cfg->unified_memory;
  if (ctx->cfg->default_cache != 0) ctx->l2_cache_bytes = ctx->cfg->default_cache;
  hipStream_t s;
  if (hip_check(ctx, hipStreamCreate(&s), "hipStreamCreate") != 0) return 1;
  ctx->stream = (void *)s;
  if (hip_check(ctx, hipHostMalloc(&ctx->scalar_stage, RTS_SCALAR_STAGE_BYTES, hipHostMallocDefault),
                "hipHostMalloc (scalar slots)") != 0) {
    ctx->scalar_stage = NULL;
    (void)hipStreamDestroy(s);
    ctx->stream = NULL;
    return 1;
  }
  memset(ctx->scalar_stage, 0, RTS_SCALAR_STAGE_BYTES);
  if (ctx->logging) {
    fprintf(ctx->log, "Device: %s, %d CUs, %zu B LDS per block, %zu B L2, %s memory\n",
            ctx->device_name, ctx->num_cus, ctx->max_shared_memory, ctx->l2_cache_bytes,
            ctx->unified ? "managed" : "unmanaged");
  }
  return 0;
}

/* --------------------------------------------------------- device memory */

static int gpu_alloc_actual(struct futhark_context *ctx, size_t size, void **mem_out) {
  hipError_t e = ctx->unified ? hipMallocManaged(mem_out, size, hipMemAttachGlobal)
                              : hipMalloc(mem_out, size);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError(); /* clear the sticky status */
    return FUTHARK_OUT_OF_MEMORY;
  }
  return hip_check(ctx, e, "hipMalloc");
}

static int gpu_free_actual(struct futhark_context *ctx, void *mem) {
  return hip_check(ctx, hipFree(mem), "hipFree");
}

int rts_gpu_alloc(struct futhark_context *ctx, size_t min_size, const char *tag, void **mem_out,
                  size_t *size_out) {
  if (min_size < sizeof(int)) min_size = sizeof(int);
  min_size = (min_size + 3) & ~(size_t)3;

  uintptr_t pooled;
  if (free_list_find(&ctx->gpu_free_list, min_size, tag, size_out, &pooled) == 0) {
    if (ctx->debugging) fprintf(ctx->log, "No need to allocate: found a pooled block.\n");
    *mem_out = (void *)pooled;
    return FUTHARK_SUCCESS;
  }

  *size_out = min_size;
  if (ctx->debugging) fprintf(ctx->log, "Allocating %zu bytes on the device.\n", min_size);
  int err = gpu_alloc_actual(ctx, min_size, mem_out);
  /* Out of memory: give pooled blocks back to the driver one at a time and
   * try again after each (gpu.h:280-305). */
  while (err == FUTHARK_OUT_OF_MEMORY) {
    uintptr_t victim;
    if (free_list_first(&ctx->gpu_free_list, NULL, &victim) != 0) break;
    if (ctx->debugging) fprintf(ctx->log, "Out of device memory: releasing a pooled block.\n");
    int ferr = gpu_free_actual(ctx, (void *)victim);
    if (ferr != 0) return ferr;
    err = gpu_alloc_actual(ctx, min_size, mem_out);
  }
  return err;
}

int rts_gpu_free(struct futhark_context *ctx, void *mem, size_t size, const char *tag) {
  free_list_insert(&ctx->gpu_free_list, size, (uintptr_t)mem, tag);
  return FUTHARK_SUCCESS;
}

int rts_gpu_free_all(struct futhark_context *ctx) {
  free_list_pack(&ctx->gpu_free_list);
  uintptr_t mem;
  while (free_list_first(&ctx->gpu_free_list, NULL, &mem) == 0) {
    int err = gpu_free_actual(ctx, (void *)mem);
    if (err != 0) return err;
  }
  return FUTHARK_SUCCESS;
}

int rts_memblock_unref(struct futhark_context *ctx, struct memblock_device *block,
                       const char *desc) {
  if (block->references != NULL) {
    *block->references -= 1;
    if (ctx->detail_memory) {
      fprintf(ctx->log, "Unreferencing block %s (allocated as %s) in space 'device': %d left.\n",
              desc, block->desc, *block->references);
    }
    if (*block->references == 0) {
      ctx->cur_mem_usage_device -= block->size;
      (void)rts_gpu_free(ctx, block->mem, (size_t)block->size, desc);
      free(block->references);
      if (ctx->detail_memory) {
        fprintf(ctx->log, "%lld bytes freed (now allocated: %lld bytes)\n",
                (long long)block->size, (long long)ctx->cur_mem_usage_device);
      }
    }
    block->references = NULL;
  }
  return 0;
}

int rts_memblock_alloc(struct futhark_context *ctx, struct memblock_device *block, int64_t size,
                       const char *desc) {
  if (size < 0) {
    rts_panic(1, "Negative allocation of %lld bytes attempted for %s in space 'device'.\n",
              (long long)size, desc);
  }
  int ret = rts_memblock_unref(ctx, block, desc);
  if (ret != FUTHARK_SUCCESS) return ret;
  if (ctx->detail_memory) {
    fprintf(ctx->log, "Allocating %lld bytes for %s in space 'device' (currently allocated: %lld).\n",
            (long long)size, desc, (long long)ctx->cur_mem_usage_device);
  }
  size_t got = 0;
  int err = rts_gpu_alloc(ctx, (size_t)size, desc, &block->mem, &got);
  if (err == FUTHARK_SUCCESS) {
    block->references = (int *)malloc(sizeof(int));
    *block->references = 1;
    block->size = (int64_t)got;
    block->desc = desc;
    ctx->cur_mem_usage_device += block->size;
    if (ctx->cur_mem_usage_device > ctx->peak_mem_usage_device)
      ctx->peak_mem_usage_device = ctx->cur_mem_usage_device;
    return FUTHARK_SUCCESS;
  }
  if (err == FUTHARK_OUT_OF_MEMORY) {
    char *old = futhark_context_get_error(ctx);
    rts_set_error(ctx,
                  rts_msgprintf("Failed to allocate memory in space 'device'.\n"
                                "Attempted allocation: %12lld bytes\n"
                                "Currently allocated:  %12lld bytes\n%s",
                                (long long)size, (long long)ctx->cur_mem_usage_device,
                                old ? old : ""));
    free(old);
  }
  return err;
}

int rts_memblock_set(struct futhark_context *ctx, struct memblock_device *lhs,
                     struct memblock_device *rhs, const char *lhs_desc) {
  int ret = rts_memblock_unref(ctx, lhs, lhs_desc);
  if (rhs->references != NULL) (*rhs->references)++;
  *lhs = *rhs;
  return ret;
}

int rts_copy_h2d(struct futhark_context *ctx, void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return 0;
  return hip_check(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
                                       (hipStream_t)ctx->stream), "hipMemcpyAsync (H2D)");
}
int rts_copy_d2h(struct futhark_context *ctx, void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return 0;
  return hip_check(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
                                       (hipStream_t)ctx->stream), "hipMemcpyAsync (D2H)");
}
/* Hands over the scalars of slots [head, upto): the caller has drained the
 * stream after `upto` was read, so their kernels have finished. */
static void deliver_scalars(struct futhark_context *ctx, uint64_t upto) {
  pthread_mutex_lock(&ctx->scalar_lock);
  while (ctx->scalar_head < upto) {
    const size_t i = (size_t)(ctx->scalar_head % RTS_SCALAR_SLOTS);
    memcpy(ctx->scalar_pending[i].dst, (char *)ctx->scalar_stage + 256 + i * RTS_SCALAR_SLOT_BYTES,
           ctx->scalar_pending[i].bytes);
    ctx->scalar_head++;
  }
  pthread_mutex_unlock(&ctx->scalar_lock);
}
static uint64_t scalars_queued(struct futhark_context *ctx) {
  pthread_mutex_lock(&ctx->scalar_lock);
  const uint64_t tail = ctx->scalar_tail;
  pthread_mutex_unlock(&ctx->scalar_lock);
  return tail;
}
void *rts_scalar_slot(struct futhark_context *ctx) {
  /* Entry points run one at a time (the context's lock), so the tail does not
   * move between this call and rts_take_scalar. */
  pthread_mutex_lock(&ctx->scalar_lock);
  const uint64_t tail = ctx->scalar_tail;
  const int full = tail - ctx->scalar_head >= RTS_SCALAR_SLOTS;
  pthread_mutex_unlock(&ctx->scalar_lock);
  if (full) {
    if (hip_check(ctx, hipStreamSynchronize((hipStream_t)ctx->stream), "hipStreamSynchronize") != 0)
      return NULL;
    deliver_scalars(ctx, tail);
  }
  return (char *)ctx->scalar_stage + 256 + (size_t)(tail % RTS_SCALAR_SLOTS) * RTS_SCALAR_SLOT_BYTES;
}
int rts_take_scalar(struct futhark_context *ctx, void *slot, void *dst, size_t bytes) {
  if (bytes > RTS_SCALAR_SLOT_BYTES || dst == NULL) return 1;
  pthread_mutex_lock(&ctx->scalar_lock);
  const size_t i = (size_t)(ctx->scalar_tail % RTS_SCALAR_SLOTS);
  const int ok = slot == (char *)ctx->scalar_stage + 256 + i * RTS_SCALAR_SLOT_BYTES;
  if (ok) {
    ctx->scalar_pending[i].dst = dst;
    ctx->scalar_pending[i].bytes = bytes;
    ctx->scalar_tail++;
  }
  pthread_mutex_unlock(&ctx->scalar_lock);
  return ok ? 0 : 1;
}
int rts_copy_d2d(struct futhark_context *ctx, void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return 0;
  return hip_check(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice,
                                       (hipStream_t)ctx->stream), "hipMemcpyAsync (D2D)");
}
int rts_memset0(struct futhark_context *ctx, void *dst, size_t bytes) {
  if (bytes == 0) return 0;
  return hip_check(ctx, hipMemsetAsync(dst, 0, bytes, (hipStream_t)ctx->stream),
                   "hipMemsetAsync");
}

/* ---------------------------------------------------------------- scratch */

enum { SCAN_EPOCH_LIMIT = (1 << 28) - 1 };

void *rts_scan_scratch(struct futhark_context *ctx, size_t bytes, uint32_t *epoch_out) {
  if (bytes > ctx->scan_scratch_bytes || ctx->scan_epoch >= SCAN_EPOCH_LIMIT) {
    size_t want = bytes > ctx->scan_scratch_bytes ? bytes : ctx->scan_scratch_bytes;
    if (want < (1u << 20)) want = 1u << 20;
    if (want > ctx->scan_scratch_bytes) {
      /* The old buffer may still be in use by queued kernels; the stream is
       * in-order, and hipFree waits for the device. */
      if (ctx->scan_scratch != NULL) (void)gpu_free_actual(ctx, ctx->scan_scratch);
      ctx->scan_scratch = NULL;
      ctx->scan_scratch_bytes = 0;
      void *mem = NULL;
      int err = gpu_alloc_actual(ctx, want, &mem);
      if (err != 0) {
        if (err == FUTHARK_OUT_OF_MEMORY)
          rts_set_error(ctx, rts_msgprintf("Failed to allocate %zu bytes of scan scratch.\n", want));
        return NULL;
      }
      ctx->scan_scratch = mem;
      ctx->scan_scratch_bytes = want;
    }
    if (rts_memset0(ctx, ctx->scan_scratch, ctx->scan_scratch_bytes) != 0) return NULL;
    ctx->scan_epoch = 0;
  }
  *epoch_out = ++ctx->scan_epoch;
  return ctx->scan_scratch;
}

/* -------------------------------------------------------------- profiling */

static void event_list_free(struct futhark_context *ctx) {
  struct event_list *l = &ctx->event_list;
  for (int i = 0; i < l->num_events; i++) {
    free(l->events[i].description);
    if (l->events[i].start) (void)hipEventDestroy((hipEvent_t)l->events[i].start);
    if (l->events[i].end) (void)hipEventDestroy((hipEvent_t)l->events[i].end);
  }
  free(l->events);
  l->events = NULL;
  l->num_events = l->capacity = 0;
}

struct rts_event *rts_kernel_begin(struct futhark_context *ctx, const char *name, char *desc) {
  if (ctx->logging) {
    fprintf(ctx->log, "Launching %s %s\n", name, desc ? desc : "");
  }
  if (!ctx->profiling || ctx->profiling_paused) {
    free(desc);
    return NULL;
  }
  struct event_list *l = &ctx->event_list;
  if (l->num_events == l->capacity) {
    l->capacity = l->capacity ? l->capacity * 2 : 64;
    l->events = (struct rts_event *)realloc(l->events, (size_t)l->capacity * sizeof(*l->events));
  }
  /* The events only measure time (the report is read after a synchronisation
   * of the stream), so they skip the system-scope fence an event carries by
   * default: its cache write-back and invalidation would be timed with the
   * kernel and slow the work that follows. */
  hipEvent_t a = NULL, b = NULL;
  if (hipEventCreateWithFlags(&a, hipEventDisableSystemFence) != hipSuccess ||
      hipEventCreateWithFlags(&b, hipEventDisableSystemFence) != hipSuccess) {
    if (a) (void)hipEventDestroy(a);
    free(desc);
    return NULL;
  }
  struct rts_event *ev = &l->events[l->num_events++];
  ev->name = name;
  ev->description = desc;
  ev->start = (void *)a;
  ev->end = (void *)b;
  (void)hipEventRecord(a, (hipStream_t)ctx->stream);
  return ev;
}

int rts_kernel_end(struct futhark_context *ctx, struct rts_event *ev, const char *name, int code) {
  if (ev != NULL) (void)hipEventRecord((hipEvent_t)ev->end, (hipStream_t)ctx->stream);
  if (code != 0) {
    if (code > 0) {
      rts_set_error(ctx, rts_msgprintf("%s: HIP error %d (%s)\n", name, code,
                                       hipGetErrorString((hipError_t)code)));
    } else {
      rts_set_error(ctx, rts_msgprintf("%s: rejected by the kernel library (code %d)\n", name, code));
    }
    return 1;
  }
  if (ctx->debugging) {
    int64_t t0 = rts_wall_time_us();
    hipError_t e = hipStreamSynchronize((hipStream_t)ctx->stream);
    if (e != hipSuccess) return hip_check(ctx, e, name);
    fprintf(ctx->log, "  %s: synchronised after %lldus\n", name,
            (long long)(rts_wall_time_us() - t0));
  }
  return 0;
}

char *futhark_context_report(struct futhark_context *ctx);
int futhark_context_sync(struct futhark_context *ctx);

char *futhark_context_report(struct futhark_context *ctx) {
  if (futhark_context_sync(ctx) != 0) return NULL;
  struct str_builder b;
  str_builder_init(&b);
  str_builder_printf(&b, "{\"memory\":{\"device\":%lld},\"events\":[",
                     (long long)ctx->peak_mem_usage_device);
  struct event_list *l = &ctx->event_list;
  for (int i = 0; i < l->num_events; i++) {
    struct rts_event *ev = &l->events[i];
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, (hipEvent_t)ev->start, (hipEvent_t)ev->end) != hipSuccess)
      ms = 0.0f;
    if (i != 0) str_builder_printf(&b, ",");
    str_builder_printf(&b, "{\"name\":");
    str_builder_json_str(&b, ev->name);
    str_builder_printf(&b, ",\"provenance\":\"unknown\",\"duration\":%f,\"details\":%s}",
                       (double)ms * 1000.0, ev->description ? ev->description : "{}");
  }
  str_builder_printf(&b, "]}");
  event_list_free(ctx);
  return b.str;
}

void futhark_context_pause_profiling(struct futhark_context *ctx) { ctx->profiling_paused = 1; }
void futhark_context_unpause_profiling(struct futhark_context *ctx) { ctx->profiling_paused = 0; }
void futhark_context_set_logging_file(struct futhark_context *ctx, FILE *f) { ctx->log = f; }

/* ---------------------------------------------------------------- context */

int futhark_context_sync(struct futhark_context *ctx) {
  if (ctx->stream == NULL) return 1;
  /* Scalars queued up to here belong to work this synchronisation waits for. */
  const uint64_t queued = scalars_queued(ctx);
  hipError_t e = hipStreamSynchronize((hipStream_t)ctx->stream);
  if (e != hipSuccess) return hip_check(ctx, e, "hipStreamSynchronize");
  deliver_scalars(ctx, queued);
  /* The device's failure word is read and cleared whatever else is pending, so
   * that a failure of this interval cannot surface at a later, unrelated
   * synchronisation; an error deferred by the host goes first (it was raised
   * first: the first error wins, rts/c/context.h:5-13). */
  volatile int32_t *failure = ctx->scalar_stage != NULL ? RTS_FAILURE_WORD(ctx) : NULL;
  const int32_t code = failure != NULL ? *failure : 0;
  if (code != 0) *failure = 0;
  if (ctx->pending_error != 0) {
    int p = ctx->pending_error;
    ctx->pending_error = 0;
    return p;
  }
  if (code != 0) {
    rts_set_error(ctx, rts_msgprintf(
        code == RTS_FAILURE_SEGMENTS
            ? "Error: segments are not in order, overlap or leave the array (offsets[i] + lens[i] "
              "<= offsets[i+1] <= n required).\n"
            : "Error: a kernel reported failure %d.\n", (int)code));
    return FUTHARK_PROGRAM_ERROR;
  }
  return FUTHARK_SUCCESS;
}

int futhark_context_clear_caches(struct futhark_context *ctx) {
  pthread_mutex_lock(&ctx->lock);
  if (ctx->stream != NULL) {
    /* Pooled blocks may still be read by queued work. */
    (void)hipStreamSynchronize((hipStream_t)ctx->stream);
    ctx->peak_mem_usage_device = ctx->cur_mem_usage_device;
    (void)rts_gpu_free_all(ctx);
  }
  pthread_mutex_unlock(&ctx->lock);
  return ctx->error != NULL;
}

/* Contexts alive in this process (counted from backend set-up to free). */
static int live_contexts = 0;
static pthread_mutex_t live_contexts_lock = PTHREAD_MUTEX_INITIALIZER;
static void count_context(int delta) {
  pthread_mutex_lock(&live_contexts_lock);
  live_contexts += delta;
  pthread_mutex_unlock(&live_contexts_lock);
}
int rts_device_is_ours(struct futhark_context *ctx) {
  (void)ctx;
  pthread_mutex_lock(&live_contexts_lock);
  const int alone = live_contexts <= 1;
  pthread_mutex_unlock(&live_contexts_lock);
  if (!alone) return 0;
  const char *m1 = getenv("HSA_CU_MASK"), *m2 = getenv("ROC_GLOBAL_CU_MASK");
  return (m1 == NULL || m1[0] == '\0') && (m2 == NULL || m2[0] == '\0');
}

struct futhark_context *futhark_context_new(struct futhark_context_config *cfg) {
  struct futhark_context *ctx =
      (struct futhark_context *)calloc(1, sizeof(struct futhark_context));
  if (ctx == NULL) return NULL;
  assert(!cfg->in_use);
  ctx->cfg = cfg;
  cfg->in_use = 1;
  pthread_mutex_init(&ctx->lock, NULL);
  pthread_mutex_init(&ctx->error_lock, NULL);
  pthread_mutex_init(&ctx->scalar_lock, NULL);
  free_list_init(&ctx->gpu_free_list);
  ctx->debugging = cfg->debugging;
  ctx->logging = cfg->logging;
  ctx->detail_memory = cfg->logging;
  ctx->profiling = cfg->profiling;
  ctx->log = stderr;
  if (backend_setup(ctx) == 0) {
    ctx->program_initialised = true;
    count_context(1);
    (void)futhark_context_clear_caches(ctx);
    (void)futhark_context_sync(ctx);
  }
  if (ctx->error == NULL && futhark_program.apply_tuning != NULL) futhark_program.apply_tuning(ctx);
  return ctx;
}

void futhark_context_free(struct futhark_context *ctx) {
  if (ctx->program_initialised) count_context(-1);
  if (ctx->stream != NULL) {
    (void)hipStreamSynchronize((hipStream_t)ctx->stream);
    if (ctx->scan_scratch) (void)hipFree(ctx->scan_scratch);
    if (ctx->scalar_stage) (void)hipHostFree(ctx->scalar_stage);
    (void)rts_gpu_free_all(ctx);
    (void)hipStreamDestroy((hipStream_t)ctx->stream);
  }
  event_list_free(ctx);
  free_list_destroy(&ctx->gpu_free_list);
  free(ctx->error);
  pthread_mutex_destroy(&ctx->lock);
  pthread_mutex_destroy(&ctx->error_lock);
  pthread_mutex_destroy(&ctx->scalar_lock);
  ctx->cfg->in_use = 0;
  free(ctx);
}

int64_t rts_tuning_param(struct futhark_context *ctx, const char *name, int64_t fallback) {
  for (int i = 0; i < ctx->cfg->num_tuning_params; i++) {
    if (strcmp(name, ctx->cfg->tuning_params[i].name) == 0) return ctx->cfg->tuning_params[i].val;
  }
  return fallback;
}
