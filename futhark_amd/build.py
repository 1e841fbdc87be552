"""Builds the native libraries in-tree.

  futhark_amd/lib/libfuthark_amd_kernels.so   HIP kernels for gfx950 + C ABI (hipcc)
  futhark_amd/lib/libsegops.so                C runtime + `segops` program API (gcc)
  futhark_amd/lib/libfuthark_amd_values.so    Futhark value reader/writer (gcc)
  futhark_amd/bin/segops-server               server executable of the program (gcc)
  futhark_amd/bin/segops                      command-line executable of the program (gcc)
  futhark_amd/bin/capi-harness                tests/c/capi_harness.c against include/segops.h
  include/segops.json                         manifest of the program library
  oracle/liboracle.so                         CPU oracle and CPU baseline (gcc)

Run as `python -m futhark_amd.build` or through `__graft_entry__.build()`.
hipcc cross-compiles for gfx950, so no GPU is needed to build.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
PKG = ROOT / "futhark_amd"
CSRC = PKG / "csrc"
LIB = PKG / "lib"
OBJ = ROOT / "build" / "obj"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    f"-I{ROOT / 'include'}", f"-I{CSRC / 'kernels'}",
    # Keep the compiler from forming packed-FP32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    # The direct-to-LDS loads are inline asm that writes M0 and says so in its
    # clobber list, which is what keeps the compiler's own M0 set-ups apart from
    # it; clang remarks on every reserved register named there.
    "-Wno-inline-asm",
]
CC_FLAGS = [
    "-O2", "-std=c99", "-fPIC", "-Wall", "-Wextra", "-Werror", "-pthread",
    f"-I{ROOT / 'include'}", f"-I{ROCM / 'include'}", "-D__HIP_PLATFORM_AMD__=1",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(map(str, cmd))}\n{err}")
    if err.strip() and os.environ.get("FUTHARK_AMD_BUILD_VERBOSE"):
        print(err, file=sys.stderr)


def kernel_sources() -> list[Path]:
    return sorted((CSRC / "kernels").glob("*.hip"))


def host_sources() -> list[Path]:
    return sorted((CSRC / "rts").glob("*.c")) + sorted((CSRC / "prog").glob("*.c"))


def build_kernels(jobs: int = 8) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    LIB.mkdir(parents=True, exist_ok=True)
    srcs = kernel_sources()
    objs = [OBJ / (s.stem + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        _run(["hipcc", *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)])

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(one, zip(srcs, objs)))
    out = LIB / "libfuthark_amd_kernels.so"
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(out), *map(str, objs)])
    return out


def build_host() -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    objs = []
    for src in host_sources():
        obj = OBJ / ("host_" + src.stem + ".o")
        _run(["gcc", *CC_FLAGS, "-c", str(src), "-o", str(obj)])
        objs.append(obj)
    out = LIB / "libsegops.so"
    _run(["gcc", "-shared", "-o", str(out), *map(str, objs), f"-L{LIB}", "-lfuthark_amd_kernels",
          f"-L{ROCM / 'lib'}", "-lamdhip64", "-lpthread", "-lm",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{ROCM / 'lib'}"])
    return out


def build_server() -> Path:
    """The value reader/writer as a library of its own (tools and tests bind it)
    and the server executable, which needs nothing but the public API."""
    OBJ.mkdir(parents=True, exist_ok=True)
    bindir = PKG / "bin"
    bindir.mkdir(parents=True, exist_ok=True)
    server_flags = ["-O2", "-std=c99", "-fPIC", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}",
                    f"-I{CSRC / 'server'}"]
    values_obj = OBJ / "server_values.o"
    _run(["gcc", *server_flags, "-c", str(CSRC / "server" / "values.c"), "-o", str(values_obj)])
    _run(["gcc", "-shared", "-o", str(LIB / "libfuthark_amd_values.so"), str(values_obj), "-lm"])
    server_obj = OBJ / "server_server.o"
    _run(["gcc", *server_flags, "-c", str(CSRC / "server" / "server.c"), "-o", str(server_obj)])
    out = bindir / "segops-server"
    _run(["gcc", "-o", str(out), str(server_obj), str(values_obj), f"-L{LIB}", "-lsegops",
          "-lfuthark_amd_kernels", f"-L{ROCM / 'lib'}", "-lamdhip64", "-lm",
          "-Wl,-rpath,$ORIGIN/../lib", f"-Wl,-rpath,{ROCM / 'lib'}"])
    # The command-line executable (`futhark hip prog.fut` without --server).
    cli_obj = OBJ / "server_cli.o"
    _run(["gcc", *server_flags, "-c", str(CSRC / "server" / "cli.c"), "-o", str(cli_obj)])
    _run(["gcc", "-o", str(bindir / "segops"), str(cli_obj), str(values_obj), f"-L{LIB}", "-lsegops",
          "-lfuthark_amd_kernels", f"-L{ROCM / 'lib'}", "-lamdhip64", "-lm",
          "-Wl,-rpath,$ORIGIN/../lib", f"-Wl,-rpath,{ROCM / 'lib'}"])
    # A C program written against the public header only, the way a user of a
    # generated library writes one (run by tests/test_capi_harness.py).
    harness = bindir / "capi-harness"
    _run(["gcc", "-O1", "-std=c99", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}",
          str(ROOT / "tests" / "c" / "capi_harness.c"), "-o", str(harness), f"-L{LIB}", "-lsegops",
          "-lfuthark_amd_kernels", f"-L{ROCM / 'lib'}", "-lamdhip64", "-lpthread",
          "-Wl,-rpath,$ORIGIN/../lib", f"-Wl,-rpath,{ROCM / 'lib'}"])
    return out


def build_oracle() -> Path:
    _run(["make", "-B", "-C", str(ROOT / "oracle"), "-s"])  # always compiles, like the rest
    return ROOT / "oracle" / "liboracle.so"


def build_all() -> None:
    build_kernels()
    build_host()
    build_server()
    build_oracle()
    from . import manifest  # include/segops.json, as `futhark hip --library` writes prog.json
    manifest.write()


if __name__ == "__main__":
    build_all()
    print("built:", *(str(p) for p in sorted(LIB.glob("*.so"))), PKG / "bin" / "segops-server",
          ROOT / "oracle" / "liboracle.so")
