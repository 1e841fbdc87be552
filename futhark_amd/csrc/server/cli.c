/* segops: the command-line executable of the `segops` program, i.e. what
 * `futhark hip segops.fut` builds (src/Futhark/CodeGen/Backends/GenericC/CLI.hs):
 * reads the arguments of one entry point from standard input, in the textual
 * or the binary value syntax, runs it (optionally several times, writing the
 * time of each run in microseconds to a file), and prints the result, textual
 * or binary.  Options, messages and exit codes follow CLI.hs:28-171,329-521.
 * It uses the public C API of libsegops.so and the value reader/writer only. */
#define _POSIX_C_SOURCE 200809L
#include <errno.h>
#include <getopt.h>
#include <inttypes.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>
#include <unistd.h>

#include "futhark_amd_values.h"
#include "program_table.h"

static const char *progname = "segops";

static void panic(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fprintf(stderr, "%s: ", progname);
  vfprintf(stderr, fmt, ap);
  va_end(ap);
  exit(code);
}

static int64_t wall_time_us(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000 + ts.tv_nsec / 1000;
}

static void context_panic(struct futhark_context *ctx) {
  char *msg = futhark_context_get_error(ctx);
  panic(1, "%s", msg != NULL ? msg : "(no error message)\n");
}

/* One parsed argument: the host data as read, kept until the runs are over. */
struct parsed {
  const struct stype *type;
  int64_t shape[FV_MAX_RANK];
  void *data;
};

static void read_inputs(const struct entry *e, struct parsed *in) {
  for (int i = 0; i < e->num_ins; i++) {
    const struct stype *t = find_type(e->in_types[i]);
    in[i].type = t;
    if (t->kind == K_RECORD) panic(1, "Cannot read input #%d of type %s\n", i, t->name);
    errno = 0;
    if (fv_read_value(stdin, fv_primtype(t->prim), t->rank, in[i].shape, &in[i].data, NULL, 0) != 0)
      panic(1, t->kind == K_ARRAY ? "Cannot read input #%d of type %s (errno: %s).\n"
                                  : "Error when reading input #%d of type %s (errno: %s).\n",
            i, t->name, strerror(errno));
  }
  if (fv_end_of_input(stdin) != 0)
    panic(1, "Expected EOF on stdin after reading input for \"%s\".\n", e->name);
}

/* Arrays go to the device anew for every run, as in the generated code
 * (pack_input / free_input, CLI.hs:329-365): an entry point may consume them. */
static void pack_inputs(struct futhark_context *ctx, const struct entry *e,
                        const struct parsed *in, struct value *vals) {
  for (int i = 0; i < e->num_ins; i++) {
    vals[i].type = in[i].type;
    if (in[i].type->kind == K_ARRAY) {
      vals[i].u.arr = in[i].type->arr_new(ctx, in[i].data, in[i].shape);
      if (vals[i].u.arr == NULL) context_panic(ctx);
    } else {
      memcpy(vals[i].u.bytes, in[i].data, (size_t)fv_primtype(in[i].type->prim)->size);
    }
  }
}

static void free_inputs(struct futhark_context *ctx, const struct entry *e, struct value *vals) {
  for (int i = 0; i < e->num_ins; i++)
    if (vals[i].type->kind == K_ARRAY && vals[i].type->arr_free(ctx, vals[i].u.arr) != 0)
      context_panic(ctx);
}

static void free_result(struct futhark_context *ctx, struct value *v) {
  if (v->type->kind == K_ARRAY) {
    if (v->u.arr != NULL && v->type->arr_free(ctx, v->u.arr) != 0) context_panic(ctx);
    v->u.arr = NULL;
  } else if (v->type->kind == K_RECORD) {
    for (int i = 0; i < v->type->num_fields; i++) free_result(ctx, &v->u.fields[i]->value);
  }
}

static void print_value(struct futhark_context *ctx, const struct value *v, int binary) {
  const struct stype *t = v->type;
  if (t->kind == K_RECORD) {
    /* a tuple prints its fields one per line (printStm, CLI.hs:263-281) */
    for (int i = 0; i < t->num_fields; i++) {
      if (i > 0) puts("");
      print_value(ctx, &v->u.fields[i]->value, binary);
    }
    return;
  }
  const struct fv_primtype *pt = fv_primtype(t->prim);
  if (t->kind == K_PRIMITIVE) {
    if (binary) fv_write_binary(stdout, pt, 0, NULL, v->u.bytes);
    else fv_write_text(stdout, pt, 0, NULL, v->u.bytes);
    return;
  }
  const int64_t *shape = t->arr_shape(ctx, v->u.arr);
  int64_t n = 1;
  for (int i = 0; i < t->rank; i++) n *= shape[i];
  void *host = calloc((size_t)(n > 0 ? n : 1), (size_t)pt->size);
  if (host == NULL) panic(1, "Out of host memory.\n");
  if (t->arr_values(ctx, v->u.arr, host) != 0 || futhark_context_sync(ctx) != 0) context_panic(ctx);
  if (binary) fv_write_binary(stdout, pt, t->rank, shape, host);
  else fv_write_text(stdout, pt, t->rank, shape, host);
  free(host);
}

static void usage(void) {
  printf("Usage: %s [OPTION]...\nOptions:\n\n"
         "  -t/--write-runtime-to FILE Print the time taken to execute the program to the "
         "indicated file, an integral number of microseconds.\n"
         "  -r/--runs INT              Perform NUM runs of the program.\n"
         "  -D/--debugging             Perform possibly expensive internal correctness checks and "
         "verbose logging.\n"
         "  -L/--log                   Print various low-overhead logging information to stderr "
         "while running.\n"
         "  -P/--profile               Enable the collection of profiling information.\n"
         "  -e/--entry-point NAME      The entry point to run. Defaults to main.\n"
         "  -b/--binary-output         Print the program result in the binary output format.\n"
         "  -n/--no-print-result       Do not print the program result.\n"
         "  -h/--help                  Print help information and exit.\n"
         "  --print-params             Print all tuning parameters that can be set with --param "
         "or --tuning.\n"
         "  --param ASSIGNMENT         Set a tuning parameter to the given value.\n"
         "  --tuning FILE              Read size=value assignments from the given file.\n"
         "  --cache-file FILE          Store program cache here.\n"
         "  -d/--device NAME           Use the first device whose name contains the given "
         "string.\n"
         "\nFor more information, consult the Futhark User's Guide or the man pages.\n",
         progname);
}

static void set_param(struct futhark_context_config *cfg, char *assignment, const char *what) {
  char *eq = strchr(assignment, '=');
  if (eq == NULL) panic(1, "Invalid argument for --parameter option: %s\n", what);
  *eq = 0;
  if (futhark_context_config_set_tuning_param(cfg, assignment, (size_t)atoi(eq + 1)) != 0)
    panic(1, "Unknown tuning parameter: %s\n", assignment);
}

int main(int argc, char **argv) {
  progname = argv[0];
  struct futhark_context_config *cfg = futhark_context_config_new();
  if (cfg == NULL) abort();

  const char *entry_point = "main";
  FILE *runtime_file = NULL;
  int num_runs = 1, perform_warmup = 0, binary_output = 0, print_result = 1, profiling = 0;
  static const struct option long_opts[] = {
      {"write-runtime-to", required_argument, NULL, 't'}, {"runs", required_argument, NULL, 'r'},
      {"debugging", no_argument, NULL, 'D'},              {"log", no_argument, NULL, 'L'},
      {"profile", no_argument, NULL, 'P'},                {"entry-point", required_argument, NULL, 'e'},
      {"binary-output", no_argument, NULL, 'b'},          {"no-print-result", no_argument, NULL, 'n'},
      {"help", no_argument, NULL, 'h'},                   {"print-params", no_argument, NULL, 1},
      {"param", required_argument, NULL, 2},              {"tuning", required_argument, NULL, 3},
      {"cache-file", required_argument, NULL, 4},         {"device", required_argument, NULL, 'd'},
      {0, 0, 0, 0}};
  int c;
  while ((c = getopt_long(argc, argv, ":t:r:DLPe:bnhd:", long_opts, NULL)) != -1) {
    switch (c) {
      case 't':
        runtime_file = fopen(optarg, "w");
        if (runtime_file == NULL) panic(1, "Cannot open %s: %s\n", optarg, strerror(errno));
        break;
      case 'r':
        num_runs = atoi(optarg);
        perform_warmup = 1;
        if (num_runs <= 0) panic(1, "Need a positive number of runs, not %s\n", optarg);
        break;
      case 'D': futhark_context_config_set_debugging(cfg, 1); break;
      case 'L': futhark_context_config_set_logging(cfg, 1); break;
      case 'P': futhark_context_config_set_profiling(cfg, 1); profiling = 1; break;
      case 'e': entry_point = optarg; break;
      case 'b': binary_output = 1; break;
      case 'n': print_result = 0; break;
      case 'h': usage(); return 0;
      case 'd': futhark_context_config_set_device(cfg, optarg); break;
      case 1:
        for (int i = 0; i < futhark_get_tuning_param_count(); i++)
          printf("%s (%s)\n", futhark_get_tuning_param_name(i), futhark_get_tuning_param_class(i));
        return 0;
      case 2: set_param(cfg, optarg, optarg); break;
      case 3: {
        FILE *f = fopen(optarg, "r");
        if (f == NULL)
          panic(1, "When loading tuning file '%s': %s\n", optarg, strerror(errno));
        char line[512];
        while (fgets(line, sizeof line, f) != NULL) {
          line[strcspn(line, "\r\n")] = 0;
          if (line[0] != 0) set_param(cfg, line, line);
        }
        fclose(f);
        break;
      }
      case 4: futhark_context_config_set_cache_file(cfg, optarg); break;
      case ':': panic(1, "Missing argument for option %s\n", argv[optind - 1]); break;
      default: panic(1, "Unknown option: %s\n", argv[optind - 1]); break;
    }
  }
  if (optind < argc) panic(1, "Excess non-option: %s\n", argv[optind]);

  struct futhark_context *ctx = futhark_context_new(cfg);
  if (ctx == NULL) abort();
  char *error = futhark_context_get_error(ctx);
  if (error != NULL) panic(1, "%s", error);

  const struct entry *e = find_entry(entry_point);
  if (e == NULL) {
    fprintf(stderr, "No entry point '%s'.  Select another with --entry-point.  Options are:\n",
            entry_point);
    for (int i = 0; i < NUM_ENTRIES; i++) fprintf(stderr, "%s\n", entries[i].name);
    return 1;
  }
  if (isatty(fileno(stdin))) {
    fprintf(stderr, "Reading input from TTY.\n");
    fprintf(stderr, "Send EOF (CTRL-d) after typing all input values.\n");
  }

  /* Initialisation is not profiled; of the runs, only the last one is. */
  futhark_context_pause_profiling(ctx);
  struct parsed in[ENTRY_MAX_INPUTS] = {{0}};
  read_inputs(e, in);

  struct variable fields[2] = {{0}};
  struct value result = {0};
  result.type = find_type(e->out_type);
  if (result.type->kind == K_RECORD)
    for (int i = 0; i < result.type->num_fields; i++) {
      fields[i].value.type = find_type(result.type->field_types[i]);
      result.u.fields[i] = &fields[i];
    }

  const int total = num_runs + (perform_warmup ? 1 : 0);
  for (int run = 0; run < total; run++) {
    const int timed = !perform_warmup || run > 0;
    const int last = run == total - 1;
    struct value vals[ENTRY_MAX_INPUTS];
    struct value *ins[ENTRY_MAX_INPUTS];
    for (int i = 0; i < ENTRY_MAX_INPUTS; i++) ins[i] = &vals[i];
    pack_inputs(ctx, e, in, vals);
    if (futhark_context_sync(ctx) != 0) context_panic(ctx);
    if (last) futhark_context_unpause_profiling(ctx);
    const int64_t t_start = wall_time_us();
    if (e->f(ctx, &result, ins) != 0) context_panic(ctx);
    if (futhark_context_sync(ctx) != 0) context_panic(ctx);
    if (last) futhark_context_pause_profiling(ctx);
    const int64_t t_end = wall_time_us();
    if (timed && runtime_file != NULL) {
      fprintf(runtime_file, "%lld\n", (long long)(t_end - t_start));
      fflush(runtime_file);
    }
    free_inputs(ctx, e, vals);
    if (!last) free_result(ctx, &result);
  }
  for (int i = 0; i < e->num_ins; i++) free(in[i].data);

  if (print_result) {
    print_value(ctx, &result, binary_output);
    puts("");
  }
  free_result(ctx, &result);
  if (runtime_file != NULL) fclose(runtime_file);
  if (profiling) {
    /* where the generated executable leaves the report to `futhark profile`
     * through the server, this one prints it for whoever asked with -P */
    char *report = futhark_context_report(ctx);
    if (report != NULL) fprintf(stderr, "%s\n", report);
    free(report);
  }
  futhark_context_free(ctx);
  futhark_context_config_free(cfg);
  return 0;
}
