/*
 * rts.h -- internal interface of the MI355X runtime backend that sits under the
 * generated-library API (futhark_context_*, futhark_new_*, futhark_entry_*).
 *
 * It plays the part of rts/c/{context,gpu,free_list,event_list,util,lock}.h and
 * rts/c/backends/hip.h in the reference, as ordinary separately compiled C
 * instead of text pasted into each generated program.  A "program" (the file
 * that defines array types and entry points) describes itself with a
 * struct rts_program and calls the services declared here.
 */
#ifndef FUTHARK_AMD_RTS_H
#define FUTHARK_AMD_RTS_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <pthread.h>

#define FUTHARK_SUCCESS 0
#define FUTHARK_PROGRAM_ERROR 2
#define FUTHARK_OUT_OF_MEMORY 3

/* ------------------------------------------------------------------ util */
char *rts_msgprintf(const char *fmt, ...);
void rts_panic(int eval, const char *fmt, ...);
int64_t rts_wall_time_us(void);

struct str_builder {
  char *str;
  size_t capacity;
  size_t used;
};
void str_builder_init(struct str_builder *b);
void str_builder_printf(struct str_builder *b, const char *fmt, ...);
void str_builder_json_str(struct str_builder *b, const char *s);

/* ------------------------------------------------------------- free list
 * Pool of released blocks, reused by size and tag
 * (behaviour of rts/c/free_list.h:100-166). */
struct free_list_entry {
  size_t size;
  uintptr_t mem;
  const char *tag;
  bool valid;
};
struct free_list {
  struct free_list_entry *entries;
  int capacity;
  int used;
  pthread_mutex_t lock;
};
void free_list_init(struct free_list *l);
void free_list_destroy(struct free_list *l);
void free_list_insert(struct free_list *l, size_t size, uintptr_t mem, const char *tag);
/* 0 and a block on success, 1 if nothing suitable is pooled. */
int free_list_find(struct free_list *l, size_t size, const char *tag, size_t *size_out,
                   uintptr_t *mem_out);
/* Removes any one block; 1 if the list is empty. */
int free_list_first(struct free_list *l, size_t *size_out, uintptr_t *mem_out);
void free_list_pack(struct free_list *l);

/* ------------------------------------------------------------ event list
 * Profiling records; rendered by futhark_context_report
 * (behaviour of rts/c/event_list.h and hip.h:540-577). */
struct rts_event {
  const char *name;      /* static string */
  char *description;     /* owned: JSON object text with grid/bytes/... or NULL */
  void *start, *end;     /* hipEvent_t pair */
};
struct event_list {
  struct rts_event *events;
  int num_events;
  int capacity;
};

/* ---------------------------------------------------------------- tuning */
struct tuning_param {
  const char *name;
  const char *param_class;
  int64_t default_value;
  bool set;
  int64_t val;
};

/* What a program tells the runtime about itself. */
struct futhark_context;
struct rts_program {
  const char *name;
  int num_tuning_params;
  const char *const *tuning_param_names;
  const char *const *tuning_param_classes;
  const int64_t *tuning_param_defaults;
  /* called once a context is up: hands the tuning values to whoever uses them */
  void (*apply_tuning)(struct futhark_context *ctx);
};
extern const struct rts_program futhark_program; /* defined by the program */

/* ---------------------------------------------------------------- config */
struct futhark_context_config {
  int in_use;
  int debugging;
  int profiling;
  int logging;
  char *cache_fname;
  int num_tuning_params;
  struct tuning_param *tuning_params;
  /* GPU backend part (rts/c/backends/hip.h:75-94). */
  char *preferred_device;   /* substring of the device name, or NULL */
  int preferred_device_num; /* k of "#k" */
  int unified_memory;       /* 0 no, 1 yes, 2 if the device supports it */
  size_t default_block_size;
  size_t default_grid_size;
  size_t default_tile_size;
  size_t default_reg_tile_size;
  size_t default_cache;
  size_t default_registers;
  size_t default_threshold;
  char *program_text; /* get/set_program: informational here, kernels are prebuilt */
  int num_build_opts;
  char **build_opts;
};

/* --------------------------------------------------------------- context */
struct memblock_device {
  int *references; /* NULL for memory owned by the caller */
  void *mem;       /* device pointer */
  int64_t size;
  const char *desc;
};

struct futhark_context {
  struct futhark_context_config *cfg;
  int debugging, profiling, profiling_paused, logging, detail_memory;
  pthread_mutex_t lock;       /* serialises public calls on this context */
  pthread_mutex_t error_lock; /* protects `error` */
  char *error;
  FILE *log;
  bool program_initialised;

  /* device */
  int device;
  char device_name[256];
  void *stream; /* hipStream_t */
  int num_cus;
  size_t max_shared_memory;
  size_t max_block_size;
  size_t l2_cache_bytes;
  int unified;

  /* pooled device memory (rts/c/gpu.h:240-331) */
  struct free_list gpu_free_list;
  int64_t cur_mem_usage_device;
  int64_t peak_mem_usage_device;

  /* profiling */
  struct event_list event_list;

  /* look-back / partials scratch owned by the context, grown on demand; it is
   * zero-filled when (re)allocated and then used with a strictly increasing
   * epoch, one per kernel launch. */
  void *scan_scratch;
  size_t scan_scratch_bytes;
  uint32_t scan_epoch;

  /* pinned host memory (hipHostMalloc) the device can write: 256 bytes of
   * header, then a ring of RTS_SCALAR_SLOTS slots of 16 bytes.  A kernel that
   * produces one scalar stores it into a slot; the entry point records where
   * the caller wants it, and futhark_context_sync hands it over once the
   * stream has drained (docs/c-api.rst:578-581: a scalar result may be used
   * after the synchronisation).  No copy operation and no wait inside the
   * entry point (a copy into pageable memory costs about 20 us per call, a
   * wait per call about 10). */
  void *scalar_stage;
#define RTS_SCALAR_SLOTS 64
#define RTS_SCALAR_SLOT_BYTES 16
#define RTS_SCALAR_STAGE_BYTES (256 + RTS_SCALAR_SLOTS * RTS_SCALAR_SLOT_BYTES)
  struct {
    void *dst;     /* where the caller wants the value */
    size_t bytes;
  } scalar_pending[RTS_SCALAR_SLOTS];
  uint64_t scalar_head, scalar_tail; /* slots [head, tail) await delivery; slot = index mod RTS_SCALAR_SLOTS */
  pthread_mutex_t scalar_lock;
  /* a word of that slot (byte 128) kernels raise when the program must fail, as
   * the reference's global_failure (rts/c/gpu.h): checked and cleared at every
   * synchronisation, which then returns FUTHARK_PROGRAM_ERROR */
#define RTS_FAILURE_WORD(ctx) ((int32_t *)((char *)(ctx)->scalar_stage + 128))
#define RTS_FAILURE_SEGMENTS 1

  /* deferred error from an asynchronous call, reported at the next sync */
  int pending_error;
};

/* error slot: first error wins (rts/c/context.h:5-13); takes ownership. */
void rts_set_error(struct futhark_context *ctx, char *msg);

/* pooled allocation: 0, FUTHARK_OUT_OF_MEMORY, or another nonzero code.
 * Sizes are rounded up to a multiple of 4, at least 4 (gpu.h:243-249). */
int rts_gpu_alloc(struct futhark_context *ctx, size_t min_size, const char *tag, void **mem_out,
                  size_t *size_out);
int rts_gpu_free(struct futhark_context *ctx, void *mem, size_t size, const char *tag);
int rts_gpu_free_all(struct futhark_context *ctx);

/* refcounted blocks (src/Futhark/CodeGen/Backends/GenericC.hs:155-283) */
int rts_memblock_alloc(struct futhark_context *ctx, struct memblock_device *block, int64_t size,
                       const char *desc);
int rts_memblock_unref(struct futhark_context *ctx, struct memblock_device *block,
                       const char *desc);
int rts_memblock_set(struct futhark_context *ctx, struct memblock_device *lhs,
                     struct memblock_device *rhs, const char *lhs_desc);

/* copies on the context's stream; asynchronous (hip.h:790-862) */
int rts_copy_h2d(struct futhark_context *ctx, void *dst, const void *src, size_t bytes);
int rts_copy_d2h(struct futhark_context *ctx, void *dst, const void *src, size_t bytes);
/* A pinned slot for one scalar result of the launch about to be queued (NULL on
 * failure, error set); when every slot awaits delivery the stream is drained
 * and the values are handed over first. */
void *rts_scalar_slot(struct futhark_context *ctx);
/* After the launch: `bytes` (at most RTS_SCALAR_SLOT_BYTES) of `slot` go to
 * `dst` at the next futhark_context_sync.  dst must stay valid until then. */
int rts_take_scalar(struct futhark_context *ctx, void *slot, void *dst, size_t bytes);
int rts_copy_d2d(struct futhark_context *ctx, void *dst, const void *src, size_t bytes);
int rts_memset0(struct futhark_context *ctx, void *dst, size_t bytes);

/* look-back scratch for scans and reductions with a fresh epoch for one launch;
 * NULL on failure (error set). */
void *rts_scan_scratch(struct futhark_context *ctx, size_t bytes, uint32_t *epoch_out);

/* Profiling bracket around one kernel-library call.  `desc` is JSON object
 * text or NULL.  rts_kernel_end turns a nonzero launcher code into an error. */
struct rts_event *rts_kernel_begin(struct futhark_context *ctx, const char *name, char *desc);
int rts_kernel_end(struct futhark_context *ctx, struct rts_event *ev, const char *name, int code);

int64_t rts_tuning_param(struct futhark_context *ctx, const char *name, int64_t fallback);

/* Nonzero while, as far as this process can tell, a kernel of this context has
 * the device to itself: no other context is alive in the process and the
 * environment sets no CU mask (HSA_CU_MASK, ROC_GLOBAL_CU_MASK). */
int rts_device_is_ours(struct futhark_context *ctx);

#endif /* FUTHARK_AMD_RTS_H */
