"""ctypes view of libfuthark_amd_values.so (csrc/server/values.c): Futhark's binary
data format (docs/binary-data-format.rst) and textual output, to and from numpy.

    write_binary(path_or_file, [array, ...])      one value after another
    read_binary(path, [("f32", 1), ("i64", 0)])   element type name and rank per value
    read_text / read_values                       the textual syntax / whichever form each value has
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

from .capi import lib_path

_DTYPES = {
    "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
    "u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64,
    "f16": np.float16, "f32": np.float32, "f64": np.float64, "bool": np.bool_,
}
_NAMES = {np.dtype(v): k for k, v in _DTYPES.items()}
MAX_RANK = 8


class _Lib:
    def __init__(self):
        path = lib_path("libfuthark_amd_values.so")
        if not Path(path).exists():
            raise FileNotFoundError(f"{path} is not built; run `python -m futhark_amd.build`")
        self.v = C.CDLL(str(path))
        self.c = C.CDLL(None)
        self.c.fopen.restype = C.c_void_p
        self.c.fopen.argtypes = [C.c_char_p, C.c_char_p]
        self.c.fclose.argtypes = [C.c_void_p]
        self.v.fv_primtype.restype = C.c_void_p
        self.v.fv_primtype.argtypes = [C.c_char_p]
        self.v.fv_read_binary.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_int64),
                                          C.POINTER(C.c_void_p), C.c_char_p, C.c_size_t]
        self.v.fv_read_text.argtypes = self.v.fv_read_binary.argtypes
        self.v.fv_read_value.argtypes = self.v.fv_read_binary.argtypes
        self.v.fv_write_binary.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_int64),
                                           C.c_void_p]
        self.v.fv_write_text.argtypes = self.v.fv_write_binary.argtypes
        self.v.fv_end_of_input.argtypes = [C.c_void_p]
        self.c.free.argtypes = [C.c_void_p]


_lib = None


def _get() -> _Lib:
    global _lib
    if _lib is None:
        _lib = _Lib()
    return _lib


class ValueError_(ValueError):
    pass


def _open(path, mode: bytes):
    L = _get()
    f = L.c.fopen(str(path).encode(), mode)
    if not f:
        raise OSError(f"cannot open {path}")
    return f


def _write(path, arrays, fn_name: str) -> None:
    L = _get()
    f = _open(path, b"wb")
    try:
        for a in arrays:
            a = np.asarray(a, order="C")  # (ascontiguousarray would make a 0-d value 1-d)
            name = _NAMES[a.dtype]
            shape = (C.c_int64 * MAX_RANK)(*a.shape)
            rc = getattr(L.v, fn_name)(f, L.v.fv_primtype(name.encode()), a.ndim, shape,
                                       a.ctypes.data_as(C.c_void_p))
            if rc != 0:
                raise OSError(f"writing to {path} failed")
    finally:
        L.c.fclose(f)


def write_binary(path, arrays) -> None:
    _write(path, arrays, "fv_write_binary")


def write_text(path, arrays) -> None:
    _write(path, arrays, "fv_write_text")


def read_binary(path, specs, expect_eof: bool = True):
    """specs: [(element type name, rank), ...]; returns numpy arrays (0-d for scalars)."""
    return _read(path, specs, expect_eof, "fv_read_binary")


def read_text(path, specs, expect_eof: bool = True):
    """The same for values in the textual syntax."""
    return _read(path, specs, expect_eof, "fv_read_text")


def read_values(path, specs, expect_eof: bool = True):
    """Each value in whichever of the two forms it is in."""
    return _read(path, specs, expect_eof, "fv_read_value")


def _read(path, specs, expect_eof, fn_name):
    L = _get()
    f = _open(path, b"rb")
    out = []
    try:
        for name, rank in specs:
            shape = (C.c_int64 * MAX_RANK)()
            data = C.c_void_p()
            err = C.create_string_buffer(256)
            rc = getattr(L.v, fn_name)(f, L.v.fv_primtype(name.encode()), rank, shape,
                                       C.byref(data), err, len(err))
            if rc != 0:
                raise ValueError_(err.value.decode())
            dims = tuple(shape[i] for i in range(rank))
            count = int(np.prod(dims, dtype=np.int64)) if rank else 1
            dt = np.dtype(_DTYPES[name])
            buf = C.string_at(data, count * dt.itemsize) if count else b""
            L.c.free(data)
            out.append(np.frombuffer(buf, dtype=dt).reshape(dims).copy())
        if expect_eof and L.v.fv_end_of_input(f) != 0:
            raise ValueError_(f"expected end of input after {len(specs)} values")
    finally:
        L.c.fclose(f)
    return out
