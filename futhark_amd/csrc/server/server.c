/* segops-server: the line-oriented server executable of the `segops` program
 * (docs/server-protocol.rst), i.e. what `futhark hip --server segops.fut` would
 * give `futhark bench/test/autotune` to talk to.  It sits entirely on the public
 * C API of libsegops.so (include/segops.h) plus the value reader/writer of
 * values.c.  Command set, replies and error texts follow rts/c/server.h
 * (dispatcher :1447-1535, call :344-403, restore/store :405-480); the program
 * has no sum types and its only records are the pair results of the by-key
 * sorts.
 *
 * Variables hold either a scalar (stored inline) or a pointer to a library
 * array; records hold the variables of their fields. */
#define _POSIX_C_SOURCE 200809L
#include <ctype.h>
#include <errno.h>
#include <getopt.h>
#include <inttypes.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "segops.h"
#include "futhark_amd_values.h"

#include "program_table.h"

/* ----------------------------------------------------------------- server */

struct server {
  struct futhark_context_config *cfg;
  struct futhark_context *ctx;
  struct variable *vars;
};

static void reply_ok(void) {
  printf("%%%%%% OK\n");
  fflush(stdout);
}

/* After this marker everything up to the next OK is the error message. */
static void reply_failure(const char *fmt, ...) {
  printf("%%%%%% FAILURE\n");
  if (fmt != NULL) {
    va_list ap;
    va_start(ap, fmt);
    vprintf(fmt, ap);
    va_end(ap);
  }
}

static void report_context_error(struct server *s, int err) {
  if (err == 0) return;
  reply_failure(NULL);
  char *msg = futhark_context_get_error(s->ctx);
  if (msg != NULL) puts(msg);
  free(msg);
}

static struct variable *find_var(struct server *s, const char *name) {
  for (struct variable *v = s->vars; v != NULL; v = v->next)
    if (strcmp(v->name, name) == 0) return v;
  return NULL;
}

static struct variable *alloc_var(const char *name, const struct stype *t) {
  struct variable *v = calloc(1, sizeof *v);
  if (v == NULL) abort();
  v->name = name ? strdup(name) : NULL;
  v->value.type = t;
  if (t->kind == K_RECORD)
    for (int i = 0; i < t->num_fields; i++)
      v->value.u.fields[i] = alloc_var(NULL, find_type(t->field_types[i]));
  return v;
}

/* NULL if the name is taken. */
static struct variable *create_var(struct server *s, const char *name, const struct stype *t) {
  if (find_var(s, name) != NULL) return NULL;
  struct variable *v = alloc_var(name, t);
  v->next = s->vars;
  s->vars = v;
  return v;
}

static void release_value(struct server *s, struct value *val) {
  const struct stype *t = val->type;
  if (t->kind == K_ARRAY) {
    if (val->u.arr != NULL) t->arr_free(s->ctx, val->u.arr);
    val->u.arr = NULL;
  } else if (t->kind == K_RECORD) {
    for (int i = 0; i < t->num_fields; i++) {
      if (val->u.fields[i] == NULL) continue;
      release_value(s, &val->u.fields[i]->value);
      free(val->u.fields[i]);
      val->u.fields[i] = NULL;
    }
  }
}

static void drop_var(struct server *s, struct variable *v, int release) {
  for (struct variable **p = &s->vars; *p != NULL; p = &(*p)->next)
    if (*p == v) {
      *p = v->next;
      break;
    }
  if (release) {
    release_value(s, &v->value);
  } else if (v->value.type->kind == K_RECORD) {
    for (int i = 0; i < v->value.type->num_fields; i++) free(v->value.u.fields[i]);
  }
  free(v->name);
  free(v);
}

static int count_args(char **args) {
  int n = 0;
  while (args[n] != NULL) n++;
  return n;
}

/* A missing argument ends the server, as in the reference (get_arg,
 * rts/c/server.h:296-308). */
static const char *need_arg(char **args, int i) {
  for (int k = 0; k <= i; k++)
    if (args[k] == NULL) {
      fprintf(stderr, "Insufficient command args.\n");
      exit(1);
    }
  return args[i];
}

static int64_t now_usec(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000 + ts.tv_nsec / 1000;
}

static void cmd_call(struct server *s, char **args) {
  const char *name = need_arg(args, 0);
  const char *out_name = need_arg(args, 1);
  const struct entry *e = find_entry(name);
  if (e == NULL) {
    reply_failure("Unknown entry point: %s\n", name);
    return;
  }
  struct value *ins[ENTRY_MAX_INPUTS] = {0};
  for (int i = 0; i < e->num_ins; i++) {
    const char *in_name = need_arg(args, 2 + i);
    struct variable *v = find_var(s, in_name);
    if (v == NULL) {
      reply_failure("Unknown variable: %s\n", in_name);
      return;
    }
    if (strcmp(v->value.type->name, e->in_types[i]) != 0) {
      reply_failure("Wrong input type.  Expected %s, got %s.\n", e->in_types[i],
                    v->value.type->name);
      return;
    }
    ins[i] = &v->value;
  }
  struct variable *out = create_var(s, out_name, find_type(e->out_type));
  if (out == NULL) {
    reply_failure("Variable already exists: %s\n", out_name);
    return;
  }
  const int64_t t0 = now_usec();
  int err = e->f(s->ctx, &out->value, ins);
  err |= futhark_context_sync(s->ctx);
  const int64_t t1 = now_usec();
  printf("runtime: %lld\n", (long long)(t1 - t0));
  report_context_error(s, err);
  if (err != 0) drop_var(s, out, 0); /* the outputs were left untouched */
}

/* Reads one value of type t from f into val (val->type already set). */
static int restore_value(struct server *s, FILE *f, struct value *val) {
  const struct stype *t = val->type;
  if (t->kind == K_RECORD) {
    for (int i = 0; i < t->num_fields; i++)
      if (restore_value(s, f, &val->u.fields[i]->value) != 0) return 1;
    return 0;
  }
  int64_t shape[FV_MAX_RANK];
  void *data = NULL;
  if (fv_read_binary(f, fv_primtype(t->prim), t->rank, shape, &data, NULL, 0) != 0) return 1;
  int rc = 0;
  if (t->kind == K_PRIMITIVE) {
    memcpy(val->u.bytes, data, (size_t)fv_primtype(t->prim)->size);
  } else {
    val->u.arr = t->arr_new(s->ctx, data, shape);
    if (val->u.arr == NULL) rc = 1;
    /* The copy to the device is asynchronous and reads `data`. */
    if (rc == 0 && futhark_context_sync(s->ctx) != 0) rc = 1;
  }
  free(data);
  return rc;
}

static void cmd_restore(struct server *s, char **args) {
  const char *fname = need_arg(args, 0);
  FILE *f = fopen(fname, "rb");
  if (f == NULL) {
    reply_failure("Failed to open %s: %s\n", fname, strerror(errno));
    return;
  }
  int bad = 0, values = 0;
  for (int i = 1; args[i] != NULL; i += 2, values++) {
    const char *vname = args[i];
    const char *tname = need_arg(args, i + 1);
    const struct stype *t = find_type(tname);
    if (t == NULL) {
      bad = 1;
      reply_failure("Unknown type: %s\n", tname);
      break;
    }
    struct variable *v = create_var(s, vname, t);
    if (v == NULL) {
      bad = 1;
      reply_failure("Variable already exists: %s\n", vname);
      break;
    }
    errno = 0;
    if (restore_value(s, f, &v->value) != 0) {
      bad = 1;
      reply_failure("Failed to restore variable %s.\n"
                    "Possibly malformed data in %s (errno: %s)\n",
                    vname, fname, strerror(errno));
      drop_var(s, v, 1);
      break;
    }
  }
  if (!bad && fv_end_of_input(f) != 0)
    reply_failure("Expected EOF after reading %d values from %s\n", values, fname);
  fclose(f);
  if (!bad) report_context_error(s, futhark_context_sync(s->ctx));
}

static int store_value(struct server *s, FILE *f, struct value *val) {
  const struct stype *t = val->type;
  if (t->kind == K_RECORD) {
    for (int i = 0; i < t->num_fields; i++)
      if (store_value(s, f, &val->u.fields[i]->value) != 0) return 1;
    return 0;
  }
  const struct fv_primtype *p = fv_primtype(t->prim);
  if (t->kind == K_PRIMITIVE) return fv_write_binary(f, p, 0, NULL, val->u.bytes);
  const int64_t *shape = t->arr_shape(s->ctx, val->u.arr);
  size_t count = 1;
  for (int i = 0; i < t->rank; i++) count *= (size_t)shape[i];
  void *host = malloc(count * (size_t)p->size + 1);
  if (host == NULL) return 1;
  int rc = t->arr_values(s->ctx, val->u.arr, host);
  rc |= futhark_context_sync(s->ctx);
  if (rc == 0) rc = fv_write_binary(f, p, t->rank, shape, host);
  free(host);
  return rc;
}

static void cmd_store(struct server *s, char **args) {
  const char *fname = need_arg(args, 0);
  FILE *f = fopen(fname, "wb");
  if (f == NULL) {
    reply_failure("Failed to open %s: %s\n", fname, strerror(errno));
    return;
  }
  for (int i = 1; args[i] != NULL; i++) {
    struct variable *v = find_var(s, args[i]);
    if (v == NULL) {
      reply_failure("Unknown variable: %s\n", args[i]);
      break;
    }
    if (store_value(s, f, &v->value) != 0) {
      report_context_error(s, 1);
      break;
    }
  }
  fclose(f);
}

static void cmd_free(struct server *s, char **args) {
  for (int i = 0; args[i] != NULL; i++) {
    struct variable *v = find_var(s, args[i]);
    if (v == NULL) {
      reply_failure("Unknown variable: %s\n", args[i]);
      return;
    }
    drop_var(s, v, 1);
  }
}

static void cmd_rename(struct server *s, char **args) {
  const char *oldname = need_arg(args, 0), *newname = need_arg(args, 1);
  struct variable *v = find_var(s, oldname);
  if (v == NULL) {
    reply_failure("Unknown variable: %s\n", oldname);
    return;
  }
  if (find_var(s, newname) != NULL) {
    reply_failure("Variable already exists: %s\n", newname);
    return;
  }
  free(v->name);
  v->name = strdup(newname);
}

static void cmd_inputs(char **args) {
  const struct entry *e = find_entry(need_arg(args, 0));
  if (e == NULL) {
    reply_failure("Unknown entry point: %s\n", args[0]);
    return;
  }
  for (int i = 0; i < e->num_ins; i++)
    printf("%s%s\n", e->in_consumed[i] ? "*" : "", e->in_types[i]);
}

static void cmd_output(char **args) {
  const struct entry *e = find_entry(need_arg(args, 0));
  if (e == NULL) {
    reply_failure("Unknown entry point: %s\n", args[0]);
    return;
  }
  printf("%s%s\n", e->out_unique ? "*" : "", e->out_type);
}

static void cmd_report(struct server *s) {
  char *report = futhark_context_report(s->ctx);
  if (report != NULL) {
    puts(report);
  } else {
    reply_failure("Failed to produce profiling report.\n");
  }
  free(report);
}

static void cmd_set_tuning_param(struct server *s, char **args) {
  const char *param = need_arg(args, 0), *val_s = need_arg(args, 1);
  const size_t val = (size_t)strtoull(val_s, NULL, 10);
  if (futhark_context_config_set_tuning_param(s->cfg, param, val) != 0)
    reply_failure("Failed to set tuning parameter %s to %ld\n", param, (long)val);
}

static void cmd_tuning_params(char **args) {
  const struct entry *e = find_entry(need_arg(args, 0));
  if (e == NULL) {
    reply_failure("Unknown entry point: %s\n", args[0]);
    return;
  }
  for (int i = 0; i < 3 && e->tuning_params[i] != NULL; i++) {
    const char *cls = "";
    for (int k = 0; k < futhark_get_tuning_param_count(); k++)
      if (strcmp(futhark_get_tuning_param_name(k), e->tuning_params[i]) == 0)
        cls = futhark_get_tuning_param_class(k);
    printf("%s %s\n", e->tuning_params[i], cls);
  }
}

static void cmd_tuning_param_class(char **args) {
  const char *param = need_arg(args, 0);
  for (int k = 0; k < futhark_get_tuning_param_count(); k++)
    if (strcmp(futhark_get_tuning_param_name(k), param) == 0) {
      printf("%s\n", futhark_get_tuning_param_class(k));
      return;
    }
  reply_failure("Unknown tuning parameter: %s\n", param);
}

static void cmd_kind(char **args) {
  const struct stype *t = find_type(need_arg(args, 0));
  if (t == NULL) {
    reply_failure("Unknown type: %s\n", args[0]);
    return;
  }
  puts(t->kind == K_PRIMITIVE ? "primitive" : t->kind == K_ARRAY ? "array" : "record");
}

static const struct stype *array_type_arg(char **args) {
  const struct stype *t = find_type(need_arg(args, 0));
  if (t == NULL || t->kind != K_ARRAY) {
    reply_failure("Not an array type\n");
    return NULL;
  }
  return t;
}

static void cmd_shape(struct server *s, char **args) {
  struct variable *v = find_var(s, need_arg(args, 0));
  if (v == NULL) {
    reply_failure("Unknown variable: %s\n", args[0]);
    return;
  }
  if (v->value.type->kind != K_ARRAY) {
    reply_failure("Not an array type\n");
    return;
  }
  const int64_t *shape = v->value.type->arr_shape(s->ctx, v->value.u.arr);
  for (int i = 0; i < v->value.type->rank; i++) printf("%lld\n", (long long)shape[i]);
}

/* Parses a whole decimal integer. */
static int parse_i64(const char *s, int64_t *out) {
  char *end;
  errno = 0;
  const long long v = strtoll(s, &end, 10);
  if (errno != 0 || end == s || *end != 0) return 1;
  *out = v;
  return 0;
}

static void cmd_new_array(struct server *s, char **args) {
  const char *to = need_arg(args, 0);
  const struct stype *t = find_type(need_arg(args, 1));
  if (find_var(s, to) != NULL) {
    reply_failure("Variable already exists: %s\n", to);
    return;
  }
  if (t == NULL || t->kind != K_ARRAY) {
    reply_failure("Not an array type\n");
    return;
  }
  const int num_args = count_args(args + 2);
  if (num_args < t->rank) {
    reply_failure("Expected %d dimensions, but got %d.\n", t->rank, num_args);
    return;
  }
  int64_t shape[FV_MAX_RANK], count = 1;
  for (int i = 0; i < t->rank; i++) {
    if (parse_i64(args[2 + i], &shape[i]) != 0 || shape[i] < 0) {
      reply_failure("Invalid size `%s` of dimension %d.\n", args[2 + i], i + 1);
      return;
    }
    count *= shape[i];
  }
  if (count != num_args - t->rank) {
    reply_failure("Expected %d values, but got %d.\n", (int)count, num_args - t->rank);
    return;
  }
  const struct fv_primtype *p = fv_primtype(t->prim);
  unsigned char *host = malloc((size_t)count * (size_t)p->size + 1);
  if (host == NULL) {
    reply_failure("Out of memory.\n");
    return;
  }
  for (int64_t i = 0; i < count; i++) {
    const char *vn = args[2 + t->rank + i];
    struct variable *v = find_var(s, vn);
    if (v == NULL) {
      reply_failure("Unknown variable: %s\n", vn);
      free(host);
      return;
    }
    if (v->value.type->kind != K_PRIMITIVE || strcmp(v->value.type->prim, t->prim) != 0) {
      reply_failure("Value %d mismatch: expected type %s, got %s\n", (int)i, t->prim,
                    v->value.type->name);
      free(host);
      return;
    }
    memcpy(host + (size_t)i * (size_t)p->size, v->value.u.bytes, (size_t)p->size);
  }
  struct variable *out = create_var(s, to, t);
  out->value.u.arr = t->arr_new(s->ctx, host, shape);
  int err = out->value.u.arr == NULL;
  err |= futhark_context_sync(s->ctx);
  free(host);
  report_context_error(s, err);
  if (err != 0) drop_var(s, out, 1);
}

static void cmd_index(struct server *s, char **args) {
  const char *to = need_arg(args, 0);
  struct variable *from = find_var(s, need_arg(args, 1));
  if (from == NULL) {
    reply_failure("Unknown variable: %s\n", args[1]);
    return;
  }
  const struct stype *t = from->value.type;
  if (t->kind != K_ARRAY) {
    reply_failure("Not an array type\n");
    return;
  }
  int64_t idx[FV_MAX_RANK];
  for (int i = 0; i < t->rank; i++) {
    if (args[2 + i] == NULL) {
      reply_failure("%d indices expected but %d values provided.\n", t->rank, i);
      return;
    }
    if (parse_i64(args[2 + i], &idx[i]) != 0) {
      reply_failure("Invalid index `%s` on dimension %d.\n", args[2 + i], i + 1);
      return;
    }
  }
  struct variable *out = create_var(s, to, find_type(t->prim));
  if (out == NULL) {
    reply_failure("Variable already exists: %s\n", to);
    return;
  }
  int err = t->arr_index(s->ctx, out->value.u.bytes, from->value.u.arr, idx);
  err |= futhark_context_sync(s->ctx);
  report_context_error(s, err);
  if (err != 0) drop_var(s, out, 0);
}

static void cmd_fields(char **args) {
  const struct stype *t = find_type(need_arg(args, 0));
  if (t == NULL || t->kind != K_RECORD) {
    reply_failure("Not a record type\n");
    return;
  }
  for (int i = 0; i < t->num_fields; i++) printf("%s %s\n", t->field_names[i], t->field_types[i]);
}

/* The library's public API has no way to take a second reference to an
 * array, so a projected field is a copy made through host memory. */
/* dst (an array value of the same type, still empty) becomes a copy of src. */
static int copy_array_value(struct server *s, const struct value *src, struct value *dst) {
  const struct stype *ft = src->type;
  const struct fv_primtype *p = fv_primtype(ft->prim);
  const int64_t *shape = ft->arr_shape(s->ctx, src->u.arr);
  size_t count = 1;
  for (int i = 0; i < ft->rank; i++) count *= (size_t)shape[i];
  void *host = malloc(count * (size_t)p->size + 1);
  if (host == NULL) return 1;
  int err = ft->arr_values(s->ctx, src->u.arr, host);
  err |= futhark_context_sync(s->ctx);
  if (err == 0) {
    dst->u.arr = ft->arr_new(s->ctx, host, shape);
    err = dst->u.arr == NULL;
    err |= futhark_context_sync(s->ctx);
  }
  free(host);
  return err;
}

static void cmd_project(struct server *s, char **args) {
  const char *to = need_arg(args, 0);
  struct variable *from = find_var(s, need_arg(args, 1));
  const char *field = need_arg(args, 2);
  if (from == NULL) {
    reply_failure("Unknown variable: %s\n", args[1]);
    return;
  }
  const struct stype *t = from->value.type;
  if (t->kind != K_RECORD) {
    reply_failure("Not a record type\n");
    return;
  }
  int fi = -1;
  for (int i = 0; i < t->num_fields; i++)
    if (strcmp(t->field_names[i], field) == 0) fi = i;
  if (fi < 0) {
    reply_failure("No such field\n");
    return;
  }
  if (find_var(s, to) != NULL) {
    reply_failure("Variable already exists: %s\n", to);
    return;
  }
  struct value *src = &from->value.u.fields[fi]->value;
  struct variable *out = create_var(s, to, src->type);
  int err = copy_array_value(s, src, &out->value);
  report_context_error(s, err);
  if (err != 0) drop_var(s, out, 1);
}

/* new v0 type v1 v2 ...: a record of the given type with copies of the fields
 * (cmd_new, rts/c/server.h:1220-1271). */
static void cmd_new(struct server *s, char **args) {
  const char *to = need_arg(args, 0);
  const struct stype *t = find_type(need_arg(args, 1));
  if (t == NULL) {
    reply_failure("Unknown type: %s\n", args[1]);
    return;
  }
  if (find_var(s, to) != NULL) {
    reply_failure("Variable already exists: %s\n", to);
    return;
  }
  if (t->kind != K_RECORD) {
    reply_failure("Not a record type\n");
    return;
  }
  const int given = count_args(args) - 2;
  if (given != t->num_fields) {
    reply_failure("%d fields expected but %d values provided.\n", given, t->num_fields);
    return;
  }
  struct variable *from[4] = {0};
  for (int i = 0; i < given; i++) {
    from[i] = find_var(s, args[2 + i]);
    if (from[i] == NULL) {
      reply_failure("Unknown variable: %s\n", args[2 + i]);
      return;
    }
    if (strcmp(from[i]->value.type->name, t->field_types[i]) != 0) {
      reply_failure("Field %s mismatch: expected type %s, got %s\n", t->field_names[i],
                    t->field_types[i], from[i]->value.type->name);
      return;
    }
  }
  struct variable *out = create_var(s, to, t);
  int err = 0;
  for (int i = 0; i < given && err == 0; i++)
    err = copy_array_value(s, &from[i]->value, &out->value.u.fields[i]->value);
  report_context_error(s, err);
  if (err != 0) drop_var(s, out, 1);
}

static char *next_word(char **line) {
  char *p = *line;
  while (isspace((unsigned char)*p)) p++;
  if (*p == 0) return NULL;
  char *word;
  if (*p == '"') {
    word = ++p;
    while (*p != 0 && *p != '"') p++;
    if (*p != '"') return NULL; /* unterminated quote ends the line */
  } else {
    word = p;
    while (*p != 0 && !isspace((unsigned char)*p)) p++;
  }
  if (*p != 0) {
    *p = 0;
    *line = p + 1;
  } else {
    *line = p;
  }
  return word;
}

#define MAX_WORDS 1000

static void process_line(struct server *s, char *line) {
  static char *words[MAX_WORDS + 1];
  int n = 0;
  while ((words[n] = next_word(&line)) != NULL) {
    if (++n == MAX_WORDS) {
      fprintf(stderr, "Line too long.\n");
      exit(1);
    }
  }
  const char *cmd = words[0];
  char **args = words + 1;
  if (cmd == NULL) {
    reply_failure("Empty line\n");
  } else if (strcmp(cmd, "call") == 0) {
    cmd_call(s, args);
  } else if (strcmp(cmd, "restore") == 0) {
    cmd_restore(s, args);
  } else if (strcmp(cmd, "store") == 0) {
    cmd_store(s, args);
  } else if (strcmp(cmd, "free") == 0) {
    cmd_free(s, args);
  } else if (strcmp(cmd, "rename") == 0) {
    cmd_rename(s, args);
  } else if (strcmp(cmd, "inputs") == 0) {
    cmd_inputs(args);
  } else if (strcmp(cmd, "output") == 0) {
    cmd_output(args);
  } else if (strcmp(cmd, "clear") == 0) {
    report_context_error(s, futhark_context_clear_caches(s->ctx));
  } else if (strcmp(cmd, "pause_profiling") == 0) {
    futhark_context_pause_profiling(s->ctx);
  } else if (strcmp(cmd, "unpause_profiling") == 0) {
    futhark_context_unpause_profiling(s->ctx);
  } else if (strcmp(cmd, "report") == 0) {
    cmd_report(s);
  } else if (strcmp(cmd, "set_tuning_param") == 0) {
    cmd_set_tuning_param(s, args);
  } else if (strcmp(cmd, "tuning_params") == 0) {
    cmd_tuning_params(args);
  } else if (strcmp(cmd, "tuning_param_class") == 0) {
    cmd_tuning_param_class(args);
  } else if (strcmp(cmd, "attributes") == 0) {
    if (find_entry(need_arg(args, 0)) == NULL) reply_failure("Unknown entry point: %s\n", args[0]);
  } else if (strcmp(cmd, "kind") == 0) {
    cmd_kind(args);
  } else if (strcmp(cmd, "type") == 0) {
    struct variable *v = find_var(s, need_arg(args, 0));
    if (v == NULL) reply_failure("Unknown variable: %s\n", args[0]);
    else puts(v->value.type->name);
  } else if (strcmp(cmd, "shape") == 0) {
    cmd_shape(s, args);
  } else if (strcmp(cmd, "elemtype") == 0) {
    const struct stype *t = array_type_arg(args);
    if (t != NULL) puts(t->prim);
  } else if (strcmp(cmd, "rank") == 0) {
    const struct stype *t = array_type_arg(args);
    if (t != NULL) printf("%d\n", t->rank);
  } else if (strcmp(cmd, "new_array") == 0) {
    cmd_new_array(s, args);
  } else if (strcmp(cmd, "index") == 0) {
    cmd_index(s, args);
  } else if (strcmp(cmd, "fields") == 0) {
    cmd_fields(args);
  } else if (strcmp(cmd, "project") == 0) {
    cmd_project(s, args);
  } else if (strcmp(cmd, "entry_points") == 0) {
    for (int i = 0; i < NUM_ENTRIES; i++) puts(entries[i].name);
  } else if (strcmp(cmd, "types") == 0) {
    for (int i = 0; i < NUM_TYPES; i++) puts(types[i].name);
  } else if (strcmp(cmd, "new") == 0) {
    cmd_new(s, args);
  } else if (strcmp(cmd, "set") == 0 || strcmp(cmd, "zip") == 0 || strcmp(cmd, "unzip") == 0) {
    /* In-place array update and arrays of records: this program has neither. */
    reply_failure("Command `%s` is not supported by this program.\n", cmd);
  } else if (strcmp(cmd, "variants") == 0 || strcmp(cmd, "variant") == 0 ||
             strcmp(cmd, "construct") == 0 || strcmp(cmd, "destruct") == 0) {
    reply_failure("Not a sum type\n");
  } else {
    fprintf(stderr, "Unknown command: %s\n", cmd);
    exit(1);
  }
}

static void usage(const char *prog) {
  printf("Usage: %s [OPTIONS]...\nOptions:\n\n"
         "  -D/--debugging     Perform possibly expensive internal correctness checks and "
         "verbose logging.\n"
         "  -L/--log           Print various low-overhead logging information while running.\n"
         "  -P/--profile       Enable the collection of profiling information.\n"
         "  -h/--help          Print help information and exit.\n"
         "  --print-params     Print all tuning parameters that can be set with --param or "
         "--tuning.\n"
         "  --param NAME=INT   Set a tuning parameter to the given value.\n"
         "  --tuning FILE      Read tuning parameters (NAME=INT lines) from the indicated file.\n"
         "  -d/--device NAME   Use the first device whose name contains the given string.\n"
         "\nFor more information, consult the Futhark User's Guide or the man pages.\n",
         prog);
}

static void set_param_or_die(struct futhark_context_config *cfg, const char *assignment) {
  const char *eq = strchr(assignment, '=');
  int64_t value;
  if (eq == NULL || parse_i64(eq + 1, &value) != 0) {
    fprintf(stderr, "Invalid argument for --param option: %s\n", assignment);
    exit(1);
  }
  char *name = strndup(assignment, (size_t)(eq - assignment));
  if (futhark_context_config_set_tuning_param(cfg, name, (size_t)value) != 0) {
    fprintf(stderr, "Unknown parameter: %s\n", name);
    exit(1);
  }
  free(name);
}

int main(int argc, char **argv) {
  struct futhark_context_config *cfg = futhark_context_config_new();
  if (cfg == NULL) abort();
  static const struct option long_opts[] = {
      {"debugging", no_argument, NULL, 'D'},   {"log", no_argument, NULL, 'L'},
      {"profile", no_argument, NULL, 'P'},     {"help", no_argument, NULL, 'h'},
      {"print-params", no_argument, NULL, 1},  {"param", required_argument, NULL, 2},
      {"tuning", required_argument, NULL, 3},  {"device", required_argument, NULL, 'd'},
      {0, 0, 0, 0}};
  int c;
  while ((c = getopt_long(argc, argv, ":DLPhd:", long_opts, NULL)) != -1) {
    switch (c) {
      case 'D': futhark_context_config_set_debugging(cfg, 1); break;
      case 'L': futhark_context_config_set_logging(cfg, 1); break;
      case 'P': futhark_context_config_set_profiling(cfg, 1); break;
      case 'h': usage(argv[0]); return 0;
      case 'd': futhark_context_config_set_device(cfg, optarg); break;
      case 1:
        for (int i = 0; i < futhark_get_tuning_param_count(); i++)
          printf("%s (%s)\n", futhark_get_tuning_param_name(i), futhark_get_tuning_param_class(i));
        return 0;
      case 2: set_param_or_die(cfg, optarg); break;
      case 3: {
        FILE *f = fopen(optarg, "r");
        if (f == NULL) {
          fprintf(stderr, "Cannot open %s: %s\n", optarg, strerror(errno));
          return 1;
        }
        char buf[512];
        while (fgets(buf, sizeof buf, f) != NULL) {
          buf[strcspn(buf, "\r\n")] = 0;
          if (buf[0] != 0) set_param_or_die(cfg, buf);
        }
        fclose(f);
        break;
      }
      case ':': fprintf(stderr, "Missing argument for option %s\n", argv[optind - 1]); return 1;
      default: fprintf(stderr, "Unknown option: %s\n", argv[optind - 1]); return 1;
    }
  }
  if (optind < argc) {
    fprintf(stderr, "Excess non-option: %s\n", argv[optind]);
    return 1;
  }

  struct futhark_context *ctx = futhark_context_new(cfg);
  if (ctx == NULL) abort();
  futhark_context_set_logging_file(ctx, stdout);
  char *error = futhark_context_get_error(ctx);
  if (error != NULL) {
    fprintf(stderr, "Error during context initialisation:\n%s\n", error);
    return 1;
  }

  struct server s = {cfg, ctx, NULL};
  char *line = NULL;
  size_t cap = 0;
  reply_ok();
  while (getline(&line, &cap, stdin) > 0) {
    process_line(&s, line);
    reply_ok();
  }
  while (s.vars != NULL) drop_var(&s, s.vars, 1);
  free(line);
  futhark_context_free(ctx);
  futhark_context_config_free(cfg);
  return 0;
}
