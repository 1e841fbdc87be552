"""ctypes view of include/segops.h (the generated-library API, docs/c-api.rst).

This is the host-side mirror a Python caller of a Futhark C library would
write: same function names, argument order and error behaviour.  There is no
fallback: if libsegops.so is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

import os

# FUTHARK_AMD_LIBDIR points at another directory holding the two libraries.
_LIBDIR = Path(os.environ.get("FUTHARK_AMD_LIBDIR") or Path(__file__).resolve().parent / "lib")

NUM_TYPES = {"i32": (C.c_int32, np.int32), "i64": (C.c_int64, np.int64),
             "f32": (C.c_float, np.float32), "f64": (C.c_double, np.float64)}
ARRAY_TYPES = {
    "i32_1d": (np.int32, 1), "i64_1d": (np.int64, 1), "u8_1d": (np.uint8, 1),
    "u32_1d": (np.uint32, 1), "u64_1d": (np.uint64, 1), "f32_1d": (np.float32, 1),
    "f64_1d": (np.float64, 1), "i32_2d": (np.int32, 2), "i64_2d": (np.int64, 2),
    "f32_2d": (np.float32, 2), "f64_2d": (np.float64, 2), "f32_3d": (np.float32, 3),
    "f16_3d": (np.uint16, 3), "u16_3d": (np.uint16, 3),
    "i8_1d": (np.int8, 1), "i16_1d": (np.int16, 1), "u16_1d": (np.uint16, 1),
    "f16_1d": (np.uint16, 1),  # f16 crosses the API as its bits
}
# opaque tuple types: name -> element types of the two component arrays
OPAQUE_PAIRS = {"tup2_arr1d_u32_arr1d_i32": ("u32", "i32"),
                "tup2_arr1d_u64_arr1d_i32": ("u64", "i32")}
OPS = ("add", "max", "min")
BITOPS = ("and", "or", "xor")  # integer types only


# element types that only hist_OP_T and rbi_OP_T exist for
HIST_ONLY_TYPES = ("i8", "u8", "i16", "u16", "u32", "u64", "f16")


def ops_for(t: str):
    return OPS + BITOPS if t[0] in "iu" else OPS


def lib_path(name: str = "libsegops.so") -> Path:
    return _LIBDIR / name


class FutharkError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"futhark error {code}: {message}")
        self.code = code
        self.message = message


class Segops:
    """Loads libsegops.so and declares every prototype of include/segops.h."""

    def __init__(self, path: Path | None = None):
        path = Path(path) if path else lib_path()
        if not path.exists():
            raise FileNotFoundError(
                f"{path} is not built; run `python -m futhark_amd.build` (no CPU fallback exists)")
        self.lib = C.CDLL(str(path))
        L = self.lib
        vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
        L.futhark_context_config_new.restype = vp
        L.futhark_context_config_free.argtypes = [vp]
        L.futhark_context_config_set_tuning_param.argtypes = [vp, C.c_char_p, C.c_size_t]
        for f in ("debugging", "profiling", "logging"):
            getattr(L, f"futhark_context_config_set_{f}").argtypes = [vp, ci]
        L.futhark_context_config_set_device.argtypes = [vp, C.c_char_p]
        L.futhark_context_config_set_cache_file.argtypes = [vp, C.c_char_p]
        L.futhark_get_tuning_param_name.restype = C.c_char_p
        L.futhark_get_tuning_param_name.argtypes = [ci]
        L.futhark_get_tuning_param_class.restype = C.c_char_p
        L.futhark_get_tuning_param_class.argtypes = [ci]
        L.futhark_context_new.restype = vp
        L.futhark_context_new.argtypes = [vp]
        L.futhark_context_free.argtypes = [vp]
        L.futhark_context_sync.argtypes = [vp]
        L.futhark_context_get_error.restype = vp  # malloc'd char*, freed by us
        L.futhark_context_get_error.argtypes = [vp]
        L.futhark_context_report.restype = vp
        L.futhark_context_report.argtypes = [vp]
        L.futhark_context_clear_caches.argtypes = [vp]
        L.futhark_context_pause_profiling.argtypes = [vp]
        L.futhark_context_unpause_profiling.argtypes = [vp]
        L.futhark_context_get_stream.restype = vp
        L.futhark_context_get_stream.argtypes = [vp]
        for name, (dt, rank) in ARRAY_TYPES.items():
            new = getattr(L, f"futhark_new_{name}")
            new.restype = vp
            new.argtypes = [vp, vp] + [i64] * rank
            raw = getattr(L, f"futhark_new_raw_{name}")
            raw.restype = vp
            raw.argtypes = [vp, vp] + [i64] * rank
            getattr(L, f"futhark_free_{name}").argtypes = [vp, vp]
            getattr(L, f"futhark_values_{name}").argtypes = [vp, vp, vp]
            getattr(L, f"futhark_index_{name}").argtypes = [vp, vp, vp] + [i64] * rank
            vr = getattr(L, f"futhark_values_raw_{name}")
            vr.restype = vp
            vr.argtypes = [vp, vp]
            sh = getattr(L, f"futhark_shape_{name}")
            sh.restype = C.POINTER(i64)
            sh.argtypes = [vp, vp]
        pp = C.POINTER(vp)
        for t in NUM_TYPES:
            for op in ops_for(t):
                getattr(L, f"futhark_entry_reduce_{op}_{t}").argtypes = [vp, vp, vp]
                getattr(L, f"futhark_entry_scan_{op}_{t}").argtypes = [vp, pp, vp]
                getattr(L, f"futhark_entry_exscan_{op}_{t}").argtypes = [vp, pp, vp]
                getattr(L, f"futhark_entry_segscan_{op}_{t}").argtypes = [vp, pp, vp, vp]
                getattr(L, f"futhark_entry_segred_{op}_{t}").argtypes = [vp, pp, vp, vp, vp]
                getattr(L, f"futhark_entry_segreduce_{op}_{t}").argtypes = [vp, pp, vp]
                getattr(L, f"futhark_entry_vecreduce_{op}_{t}").argtypes = [vp, pp, vp]
                getattr(L, f"futhark_entry_seghist_{op}_{t}").argtypes = [vp, pp, i64, vp, vp]
                getattr(L, f"futhark_entry_scanrows_{op}_{t}").argtypes = [vp, pp, vp]
                getattr(L, f"futhark_entry_vecscan_{op}_{t}").argtypes = [vp, pp, vp]
                for ix in ("", "_i64"):
                    getattr(L, f"futhark_entry_hist_{op}_{t}{ix}").argtypes = [vp, pp, i64, vp, vp]
                    getattr(L, f"futhark_entry_rbi_{op}_{t}{ix}").argtypes = [vp, pp, vp, vp, vp]
                getattr(L, f"futhark_entry_rbi_vec_{op}_{t}").argtypes = [vp, pp, vp, vp, vp]
                getattr(L, f"futhark_entry_rbi_2d_{op}_{t}").argtypes = [vp, pp, vp, vp, vp, vp]
        for t in HIST_ONLY_TYPES:
            for op in ops_for(t):
                for ix in ("", "_i64"):
                    getattr(L, f"futhark_entry_hist_{op}_{t}{ix}").argtypes = [vp, pp, i64, vp, vp]
                    getattr(L, f"futhark_entry_rbi_{op}_{t}{ix}").argtypes = [vp, pp, vp, vp, vp]
        for e in ("bmm_f32", "bmm_f16", "bmm_bf16", "matmul_f32"):
            getattr(L, f"futhark_entry_{e}").argtypes = [vp, pp, vp, vp]
        L.futhark_entry_scan_compose_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_exscan_compose_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_segscan_compose_i32.argtypes = [vp, pp, vp, vp]
        L.futhark_entry_reduce_argmax_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_scan_argmax_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_hist_argmax_i32.argtypes = [vp, pp, i64, vp, vp]
        L.futhark_entry_reduce_compose_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_sumsq_f32.argtypes = [vp, vp, vp]
        L.futhark_entry_scan_norm_f32.argtypes = [vp, pp, vp]
        L.futhark_entry_reduce_summax_f32.argtypes = [vp, pp, vp]
        L.futhark_entry_rows_fraction_f32.argtypes = [vp, pp, vp]
        L.futhark_entry_segreduce_argmax_i32.argtypes = [vp, pp, vp]
        L.futhark_entry_segreduce_compose_i32.argtypes = [vp, pp, i64, vp]
        L.futhark_entry_scanrows_argmax_i32.argtypes = [vp, pp, i64, vp]
        L.futhark_entry_segred_argmax_i32.argtypes = [vp, pp, vp, vp, vp]
        L.futhark_entry_radix_sort_u32.argtypes = [vp, pp, vp]
        L.futhark_entry_radix_sort_u64.argtypes = [vp, pp, vp]
        for name, (k, v) in OPAQUE_PAIRS.items():
            getattr(L, f"futhark_entry_radix_sort_pairs_{k}_{v}").argtypes = [vp, pp, vp, vp]
            getattr(L, f"futhark_free_opaque_{name}").argtypes = [vp, vp]
            getattr(L, f"futhark_store_opaque_{name}").argtypes = [vp, vp, pp, C.POINTER(C.c_size_t)]
            rs = getattr(L, f"futhark_restore_opaque_{name}")
            rs.restype = vp
            rs.argtypes = [vp, vp]
            getattr(L, f"futhark_new_opaque_{name}").argtypes = [vp, pp, vp, vp]
            for f in (0, 1):
                getattr(L, f"futhark_project_opaque_{name}_{f}").argtypes = [vp, pp, vp]
        L.futhark_entry_transpose_f32.argtypes = [vp, pp, vp]
        L.futhark_entry_iota_i64.argtypes = [vp, pp, i64]
        L.futhark_entry_replicate_i32.argtypes = [vp, pp, i64, C.c_int32]
        self._libc = C.CDLL(None)
        self._libc.free.argtypes = [vp]

    def take_string(self, ptr) -> str | None:
        if not ptr:
            return None
        s = C.string_at(ptr).decode(errors="replace")
        self._libc.free(ptr)
        return s


class Array:
    """A futhark_T_Rd value owned by Python; freed on close()/GC."""

    def __init__(self, ctx: "Context", kind: str, ptr: int):
        self.ctx, self.kind, self.ptr = ctx, kind, ptr

    @property
    def shape(self) -> tuple[int, ...]:
        rank = ARRAY_TYPES[self.kind][1]
        p = getattr(self.ctx.L, f"futhark_shape_{self.kind}")(self.ctx.ptr, self.ptr)
        return tuple(int(p[i]) for i in range(rank))

    @property
    def device_ptr(self) -> int:
        return getattr(self.ctx.L, f"futhark_values_raw_{self.kind}")(self.ctx.ptr, self.ptr) or 0

    def values(self, sync: bool = True) -> np.ndarray:
        dt = ARRAY_TYPES[self.kind][0]
        out = np.empty(self.shape, dtype=dt)
        rc = getattr(self.ctx.L, f"futhark_values_{self.kind}")(
            self.ctx.ptr, self.ptr, out.ctypes.data_as(C.c_void_p))
        self.ctx.check(rc)
        if sync:
            self.ctx.sync()
        return out

    def index(self, *idx: int):
        dt = ARRAY_TYPES[self.kind][0]
        out = np.zeros(1, dtype=dt)
        rc = getattr(self.ctx.L, f"futhark_index_{self.kind}")(
            self.ctx.ptr, out.ctypes.data_as(C.c_void_p), self.ptr, *idx)
        self.ctx.check(rc)
        self.ctx.sync()
        return out[0]

    def free(self) -> None:
        if self.ptr and self.ctx.ptr:
            getattr(self.ctx.L, f"futhark_free_{self.kind}")(self.ctx.ptr, self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Opaque:
    """A futhark_opaque_NAME tuple of two arrays."""

    def __init__(self, ctx: "Context", name: str, ptr: int):
        self.ctx, self.name, self.ptr = ctx, name, ptr

    def project(self, field: int) -> Array:
        slot = C.c_void_p()
        fn = getattr(self.ctx.L, f"futhark_project_opaque_{self.name}_{field}")
        self.ctx.check(fn(self.ctx.ptr, C.byref(slot), self.ptr))
        return Array(self.ctx, f"{OPAQUE_PAIRS[self.name][field]}_1d", slot.value)

    def store(self) -> bytes:
        n = C.c_size_t(0)
        fn = getattr(self.ctx.L, f"futhark_store_opaque_{self.name}")
        self.ctx.check(fn(self.ctx.ptr, self.ptr, None, C.byref(n)))
        buf = (C.c_ubyte * n.value)()
        p = C.c_void_p(C.addressof(buf))
        self.ctx.check(fn(self.ctx.ptr, self.ptr, C.byref(p), C.byref(n)))
        self.ctx.sync()
        return bytes(buf)

    def free(self) -> None:
        if self.ptr and self.ctx.ptr:
            getattr(self.ctx.L, f"futhark_free_opaque_{self.name}")(self.ctx.ptr, self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    """futhark_context_config + futhark_context with numpy conveniences."""

    def __init__(self, so: Segops | None = None, *, profiling=False, logging=False,
                 debugging=False, device: str | None = None, tuning: dict | None = None):
        self.so = so or Segops()
        self.L = self.so.lib
        self.cfg = self.L.futhark_context_config_new()
        if debugging:
            self.L.futhark_context_config_set_debugging(self.cfg, 1)
        if profiling:
            self.L.futhark_context_config_set_profiling(self.cfg, 1)
        if logging:
            self.L.futhark_context_config_set_logging(self.cfg, 1)
        if device is not None:
            self.L.futhark_context_config_set_device(self.cfg, device.encode())
        for k, v in (tuning or {}).items():
            if self.L.futhark_context_config_set_tuning_param(self.cfg, k.encode(), v) != 0:
                raise KeyError(f"unknown tuning parameter {k}")
        self.ptr = self.L.futhark_context_new(self.cfg)
        err = self.get_error()
        if err is not None:
            self.close()
            raise FutharkError(1, err)

    # -- errors ------------------------------------------------------------
    def get_error(self) -> str | None:
        return self.so.take_string(self.L.futhark_context_get_error(self.ptr))

    def check(self, rc: int) -> None:
        if rc != 0:
            raise FutharkError(rc, self.get_error() or "(no message)")

    def sync(self) -> None:
        self.check(self.L.futhark_context_sync(self.ptr))

    def report(self) -> str:
        return self.so.take_string(self.L.futhark_context_report(self.ptr)) or ""

    def clear_caches(self) -> None:
        self.check(self.L.futhark_context_clear_caches(self.ptr))

    @property
    def stream(self) -> int:
        return self.L.futhark_context_get_stream(self.ptr) or 0

    # -- arrays ------------------------------------------------------------
    def new(self, kind: str, data: np.ndarray) -> Array:
        dt, rank = ARRAY_TYPES[kind]
        a = np.ascontiguousarray(data, dtype=dt)
        if a.ndim != rank:
            raise ValueError(f"{kind} needs rank {rank}, got {a.ndim}")
        p = getattr(self.L, f"futhark_new_{kind}")(
            self.ptr, a.ctypes.data_as(C.c_void_p), *[int(d) for d in a.shape])
        if not p:
            raise FutharkError(1, self.get_error() or "futhark_new failed")
        self.sync()  # the copy is asynchronous; `a` may die after we return
        return Array(self, kind, p)

    def new_opaque(self, name: str, f0: Array, f1: Array) -> Opaque:
        slot = C.c_void_p()
        self.check(getattr(self.L, f"futhark_new_opaque_{name}")(self.ptr, C.byref(slot), f0.ptr, f1.ptr))
        return Opaque(self, name, slot.value)

    def restore_opaque(self, name: str, data: bytes) -> Opaque:
        p = getattr(self.L, f"futhark_restore_opaque_{name}")(self.ptr, data)
        if not p:
            raise FutharkError(1, self.get_error() or "futhark_restore_opaque failed")
        self.sync()
        return Opaque(self, name, p)

    def new_raw(self, kind: str, device_ptr: int, *dims: int) -> Array:
        p = getattr(self.L, f"futhark_new_raw_{kind}")(self.ptr, device_ptr, *dims)
        return Array(self, kind, p)

    # -- entry points --------------------------------------------------------
    def call(self, entry: str, out_kinds, *args):
        """futhark_entry_<entry>(ctx, &out..., in...).

        out_kinds: list of array kinds ("f32_1d"), opaque type names or scalar numpy dtypes.
        Array inputs are passed as Array, scalars as Python numbers.
        Returns one value or a tuple; scalar results are read after a sync.
        """
        fn = getattr(self.L, f"futhark_entry_{entry}")
        outs, cargs = [], []
        for k in out_kinds:
            if isinstance(k, str):
                slot = C.c_void_p()
                outs.append((k, slot))
                cargs.append(C.byref(slot))
            else:
                buf = np.zeros(1, dtype=k)
                outs.append((None, buf))
                cargs.append(buf.ctypes.data_as(C.c_void_p))
        for a in args:
            cargs.append(a.ptr if isinstance(a, Array) else a)
        self.check(fn(self.ptr, *cargs))
        res = []
        need_sync = False
        for k, slot in outs:
            if k is None:
                need_sync = True
                res.append(slot)
            elif k in OPAQUE_PAIRS:
                res.append(Opaque(self, k, slot.value))
            else:
                res.append(Array(self, k, slot.value))
        if need_sync:
            self.sync()
            res = [r[0] if isinstance(r, np.ndarray) else r for r in res]
        return res[0] if len(res) == 1 else tuple(res)

    def close(self) -> None:
        if getattr(self, "ptr", None):
            self.L.futhark_context_free(self.ptr)
            self.ptr = None
        if getattr(self, "cfg", None):
            self.L.futhark_context_config_free(self.cfg)
            self.cfg = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
