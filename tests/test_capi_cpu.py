"""Boundary checks that need no GPU: the libraries load, export every symbol the
headers declare, and the host-side runtime behaves like the reference's
(docs/c-api.rst; rts/c/free_list.h:100-166; tests_lib/c/test_const_error.c)."""
import ctypes as C
import os
import re
import subprocess
from pathlib import Path

import pytest

from futhark_amd import Segops, Context, FutharkError, lib_path
from futhark_amd.capi import ARRAY_TYPES, NUM_TYPES, OPS, ops_for

ROOT = Path(__file__).resolve().parent.parent


def _exports(path):
    out = subprocess.check_output(["nm", "-D", "--defined-only", str(path)], text=True)
    return {l.split()[-1] for l in out.splitlines() if l.strip()}


def test_kernel_library_exports_every_declared_launcher():
    hdr = (ROOT / "include" / "futhark_amd_kernels.h").read_text()
    declared = set(re.findall(r"\b(fa_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 15
    missing = declared - _exports(lib_path("libfuthark_amd_kernels.so"))
    assert not missing, missing


def test_values_library_exports_every_declared_function():
    hdr = (ROOT / "include" / "futhark_amd_values.h").read_text()
    names = set(re.findall(r"\b(fv_\w+)\s*\(", hdr))
    assert {"fv_read_binary", "fv_write_binary", "fv_write_text", "fv_primtype"} <= names
    missing = names - _exports(lib_path("libfuthark_amd_values.so"))
    assert not missing, missing


def test_program_library_exports_the_generated_api():
    hdr = (ROOT / "include" / "segops.h").read_text()
    body = "\n".join(l for l in hdr.splitlines() if not l.rstrip().endswith("\\") and "#define" not in l)
    declared = set(re.findall(r"\b(futhark_[a-z0-9_]+)\s*\(", body))
    for kind in ARRAY_TYPES:
        for f in ("new", "new_raw", "free", "values", "index", "values_raw", "shape"):
            declared.add(f"futhark_{f}_{kind}")
    for t in NUM_TYPES:
        for op in ops_for(t):
            for e in ("reduce", "scan", "exscan", "segscan", "segred", "segreduce", "vecreduce", "rbi_vec", "rbi_2d", "scanrows", "vecscan", "seghist", "hist", "rbi"):
                declared.add(f"futhark_entry_{e}_{op}_{t}")
    declared = {d for d in declared if not d.endswith("_")}
    missing = declared - _exports(lib_path())
    assert not missing, sorted(missing)
    assert len(declared) > 200


def test_tuning_param_table(segops_lib):
    L = segops_lib.lib
    n = L.futhark_get_tuning_param_count()
    assert n >= 1
    names = [L.futhark_get_tuning_param_name(i).decode() for i in range(n)]
    assert all(nm.startswith("segops.") for nm in names)
    assert all(L.futhark_get_tuning_param_class(i) for i in range(n))
    cfg = L.futhark_context_config_new()
    assert L.futhark_context_config_set_tuning_param(cfg, names[0].encode(), 7) == 0
    assert L.futhark_context_config_set_tuning_param(cfg, b"default_tile_size", 16) == 0
    assert L.futhark_context_config_set_tuning_param(cfg, b"no_such_param", 1) == 1
    L.futhark_context_config_set_device(cfg, b"#1 gfx")
    L.futhark_context_config_free(cfg)


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_context_without_device_reports_error_and_can_be_freed(segops_lib):
    # docs/c-api.rst:153-166: the caller checks futhark_context_get_error right
    # after futhark_context_new, and may still free the context.
    L = segops_lib.lib
    cfg = L.futhark_context_config_new()
    ctx = L.futhark_context_new(cfg)
    assert ctx
    msg = segops_lib.take_string(L.futhark_context_get_error(ctx))
    assert msg and "HIP device" in msg
    assert segops_lib.take_string(L.futhark_context_get_error(ctx)) is None  # slot cleared
    L.futhark_context_free(ctx)
    L.futhark_context_config_free(cfg)
    with pytest.raises(FutharkError):
        Context(segops_lib)


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError):
        Segops(tmp_path / "libsegops.so")


def test_free_list_policy(tmp_path):
    """Size/tag reuse rules of the device memory pool, exercised on the host."""
    src = tmp_path / "fl.c"
    src.write_text(r'''
#include "rts.h"
#include <assert.h>
int main(void) {
  struct free_list l; free_list_init(&l);
  static const char *A = "a", *B = "b";
  size_t sz; uintptr_t m;
  assert(free_list_find(&l, 100, A, &sz, &m) == 1);           /* empty */
  free_list_insert(&l, 10000, 1, A);
  free_list_insert(&l, 6000, 2, B);
  free_list_insert(&l, 100, 3, B);
  assert(free_list_find(&l, 20000, A, &sz, &m) == 1);          /* nothing big enough */
  assert(free_list_find(&l, 50, A, &sz, &m) == 0 && m == 3);   /* < 4096: any tag, smallest */
  assert(free_list_find(&l, 1000, A, &sz, &m) == 0 && m == 1); /* same tag: any slack */
  assert(free_list_find(&l, 1000, A, &sz, &m) == 1);           /* other tag, > 50% waste */
  assert(free_list_find(&l, 3001, A, &sz, &m) == 0 && m == 2 && sz == 6000);
  for (int i = 0; i < 100; i++) free_list_insert(&l, 4096 + i, 100 + i, A);  /* grows */
  assert(l.used == 100);
  free_list_pack(&l);
  int n = 0; while (free_list_first(&l, &sz, &m) == 0) n++;
  assert(n == 100);
  free_list_destroy(&l);
  return 0;
}''')
    exe = tmp_path / "fl"
    rts = ROOT / "futhark_amd" / "csrc" / "rts"
    subprocess.check_call(["gcc", "-std=c99", "-O1", f"-I{rts}", str(src), str(rts / "free_list.c"),
                           "-lpthread", "-o", str(exe)])
    subprocess.check_call([str(exe)])
