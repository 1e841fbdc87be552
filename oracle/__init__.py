"""ctypes loader for the CPU oracle (liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB = None

_CT = {"i32": (C.c_int32, np.int32), "i64": (C.c_int64, np.int64),
       "f32": (C.c_float, np.float32), "f64": (C.c_double, np.float64),
       # element types of histograms only
       "i8": (C.c_int8, np.int8), "u8": (C.c_uint8, np.uint8),
       "i16": (C.c_int16, np.int16), "u16": (C.c_uint16, np.uint16),
       "u32": (C.c_uint32, np.uint32), "u64": (C.c_uint64, np.uint64),
       "f16": (C.c_uint16, np.float16)}


def lib() -> C.CDLL:
    global _LIB
    if _LIB is None:
        so = _DIR / "liboracle.so"
        if not so.exists():
            subprocess.check_call(["make", "-C", str(_DIR), "-s"])
        _LIB = C.CDLL(str(so))
    return _LIB


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _arr(x, dt):
    return np.ascontiguousarray(x, dtype=dt)


def reduce(op: str, t: str, xs, variant: str = "lit"):
    ct, dt = _CT[t]
    xs = _arr(xs, dt)
    fn = getattr(lib(), f"orc_reduce_{op}_{t}_{variant}")
    fn.restype = ct
    fn.argtypes = [C.c_void_p, C.c_int64]
    return dt(fn(_p(xs), xs.size))


def scan(op: str, t: str, xs, variant: str = "lit", exclusive: bool = False):
    _, dt = _CT[t]
    xs = _arr(xs, dt)
    out = np.empty_like(xs)
    fn = getattr(lib(), f"orc_{'ex' if exclusive else ''}scan_{op}_{t}_{variant}")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
    fn(_p(xs), xs.size, _p(out))
    return out


def segscan(op: str, t: str, flags, xs, variant: str = "lit"):
    _, dt = _CT[t]
    xs, flags = _arr(xs, dt), _arr(flags, np.uint8)
    assert xs.size == flags.size
    out = np.empty_like(xs)
    fn = getattr(lib(), f"orc_segscan_{op}_{t}_{variant}")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    fn(_p(flags), _p(xs), xs.size, _p(out))
    return out


def segred(op: str, t: str, offsets, lens, xs, variant: str = "lit"):
    _, dt = _CT[t]
    xs, offsets, lens = _arr(xs, dt), _arr(offsets, np.int64), _arr(lens, np.int64)
    out = np.empty(offsets.size, dtype=dt)
    fn = getattr(lib(), f"orc_segred_{op}_{t}_{variant}")
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p]
    fn(_p(offsets), _p(lens), offsets.size, _p(xs), xs.size, _p(out))
    return out


def segreduce(op: str, t: str, xss):
    _, dt = _CT[t]
    xss = _arr(xss, dt)
    m, k = xss.shape
    out = np.empty(m, dtype=dt)
    fn = getattr(lib(), f"orc_segreduce_{op}_{t}_lit")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
    fn(_p(xss), m, k, _p(out))
    return out


def vecreduce(op: str, t: str, xss, variant: str = "lit"):
    """reduce (map2 op) (replicate k ne) xss for xss : [n][k] -> [k]."""
    _, dt = _CT[t]
    xss = _arr(xss, dt)
    n, k = xss.shape
    out = np.empty(k, dtype=dt)
    if variant != "lit":  # one reduction per column
        cols = np.ascontiguousarray(xss.T)
        for j in range(k):
            out[j] = reduce(op, t, cols[j], variant)
        return out
    fn = getattr(lib(), f"orc_vecreduce_{op}_{t}_lit")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
    fn(_p(xss), n, k, _p(out))
    return out


def rbi(op: str, t: str, dest, is_, vs, variant: str = "lit"):
    """reduce_by_index on a copy of dest."""
    _, dt = _CT[t]
    dest = _arr(dest, dt).copy()
    is_, vs = _arr(is_, np.int32), _arr(vs, dt)
    assert is_.size == vs.size
    fn = getattr(lib(), f"orc_rbi_{op}_{t}_{variant}")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(dest), dest.size, _p(is_), _p(vs), is_.size)
    return dest


NEUTRAL = {
    ("add", "i32"): 0, ("max", "i32"): np.iinfo(np.int32).min, ("min", "i32"): np.iinfo(np.int32).max,
    ("add", "i64"): 0, ("max", "i64"): np.iinfo(np.int64).min, ("min", "i64"): np.iinfo(np.int64).max,
    ("add", "f32"): 0.0, ("max", "f32"): -np.inf, ("min", "f32"): np.inf,
    ("add", "f64"): 0.0, ("max", "f64"): -np.inf, ("min", "f64"): np.inf,
    ("and", "i32"): -1, ("or", "i32"): 0, ("xor", "i32"): 0,
    ("and", "i64"): -1, ("or", "i64"): 0, ("xor", "i64"): 0,
    ("add", "f16"): 0.0, ("max", "f16"): -np.inf, ("min", "f16"): np.inf,
}
for _t in ("i8", "u8", "i16", "u16", "u32", "u64"):
    _ii = np.iinfo(_CT[_t][1])
    NEUTRAL.update({("add", _t): 0, ("max", _t): _ii.min, ("min", _t): _ii.max,
                    ("and", _t): _ii.max if _ii.min == 0 else -1, ("or", _t): 0, ("xor", _t): 0})


def scan_compose_i32(abs_, flags=None, exclusive: bool = False):
    """scan / exscan / segmented scan of affine maps (a, b) : [n][2]i32 under composition."""
    abs_ = _arr(abs_, np.int32).reshape(-1, 2)
    out = np.empty_like(abs_)
    f = None if flags is None else _arr(flags, np.uint8)
    fn = lib().orc_scan_compose_i32_lit
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p]
    fn(None if f is None else _p(f), _p(abs_), abs_.shape[0], int(exclusive), _p(out))
    return out


def scan_argmax_i32(vis, flags=None, exclusive: bool = False):
    """scan of (value, index) pairs [n][2]i32 under argmax (larger value, then smaller index)."""
    vis = _arr(vis, np.int32).reshape(-1, 2)
    out = np.empty_like(vis)
    f = None if flags is None else _arr(flags, np.uint8)
    fn = lib().orc_scan_argmax_i32_lit
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p]
    fn(None if f is None else _p(f), _p(vis), vis.shape[0], int(exclusive), _p(out))
    return out


def reduce_argmax_i32(xs):
    """reduce argmax (i32.lowest, i32.highest) (zip xs (iota n)) as [v, i]: the last scan element."""
    xs = _arr(xs, np.int32)
    if xs.size == 0:
        return np.array([np.iinfo(np.int32).min, np.iinfo(np.int32).max], np.int32)
    vis = np.stack([xs, np.arange(xs.size, dtype=np.int32)], axis=1)
    return scan_argmax_i32(vis)[-1].copy()


def hist_argmax_i32(k: int, is_, xs):
    """hist argmax ne k is (zip xs (indices xs)) as [k][2]i32."""
    is_, xs = _arr(is_, np.int32), _arr(xs, np.int32)
    ii = np.iinfo(np.int32)
    dest = np.empty((k, 2), np.int32)
    dest[:, 0], dest[:, 1] = ii.min, ii.max
    fn = lib().orc_hist_argmax_i32_lit
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(dest), k, _p(is_), _p(xs), xs.size)
    return dest


def segreduce_argmax_i32(xss):
    """map (\\row -> argmax over zip row (iota k)) xss -> [m][2]: the largest value of a row
    and the first column that holds it; (i32.lowest, i32.highest) for rows of no elements."""
    xss = _arr(xss, np.int32)
    m, k = xss.shape
    out = np.empty((m, 2), np.int32)
    if k == 0:
        out[:] = (np.iinfo(np.int32).min, np.iinfo(np.int32).max)
        return out
    first = np.argmax(xss, axis=1)          # numpy returns the first of equal maxima
    out[:, 0] = xss[np.arange(m), first]
    out[:, 1] = first
    return out


def segreduce_compose_i32(k: int, abs_):
    """Rows of k affine maps composed in element order -> [m][2] (the sequential scan of
    orc_scan_compose_i32_lit restarted at every row, read at the rows' last elements)."""
    abs_ = _arr(abs_, np.int32).reshape(-1, 2)
    if k == 0:
        return np.zeros((0, 2), np.int32)
    flags = np.zeros(abs_.shape[0], np.uint8)
    flags[::k] = 1
    return scan_compose_i32(abs_, flags)[k - 1::k].copy()


def scanrows_argmax_i32(k: int, vis):
    vis = _arr(vis, np.int32).reshape(-1, 2)
    if k == 0:
        return vis.copy()
    flags = np.zeros(vis.shape[0], np.uint8)
    flags[::k] = 1
    return scan_argmax_i32(vis, flags)


def segred_argmax_i32(offsets, lens, vis):
    """Builtins.hs:570-602 with the argmax operator: flags from the offsets, segmented scan,
    the scanned pair at the last element of every segment, the neutral pair for empty ones."""
    vis = _arr(vis, np.int32).reshape(-1, 2)
    offsets, lens = _arr(offsets, np.int64), _arr(lens, np.int64)
    out = np.empty((offsets.size, 2), np.int32)
    out[:] = (np.iinfo(np.int32).min, np.iinfo(np.int32).max)
    if vis.shape[0] == 0:
        return out
    flags = np.zeros(vis.shape[0], np.uint8)
    flags[offsets[lens > 0]] = 1
    sc = scan_argmax_i32(vis, flags)
    live = lens > 0
    out[live] = sc[offsets[live] + lens[live] - 1]
    return out


def reduce_compose_i32(abs_):
    """reduce compose (1, 0) abs: the last element of the scan, (1, 0) for no elements."""
    abs_ = _arr(abs_, np.int32).reshape(-1, 2)
    if abs_.shape[0] == 0:
        return np.array([1, 0], np.int32)
    return scan_compose_i32(abs_)[-1].copy()


def sumsq_f32(xs, variant: str = "lit"):
    """reduce (+) 0 (map (\\x -> x*x) xs): squares in f32, sum sequential in f32 ("lit") or in f64."""
    xs = _arr(xs, np.float32)
    sq = xs * xs
    return reduce("add", "f32", sq, variant)


def reduce_summax_f32(xs, variant: str = "lit"):
    """[reduce (+) 0 xs, reduce f32.max (-inf) xs]: the fold of the pair operator
    (a,b) (c,d) -> (a + c, max b d) from (0, -inf) over zip xs xs."""
    xs = _arr(xs, np.float32)
    return np.array([reduce("add", "f32", xs, variant), reduce("max", "f32", xs)], dtype=np.float64 if variant == "f64acc" else np.float32)


def scan_norm_f32(xs, variant: str = "lit"):
    """map f32.sqrt (scan (+) 0 (map (\\x -> x*x) xs))."""
    xs = _arr(xs, np.float32)
    sq = xs * xs
    return np.sqrt(scan("add", "f32", sq, variant)).astype(np.float32)


def rows_fraction_f32(xss, variant: str = "lit"):
    """map (\\r -> let t = reduce (+) 0 r in map (/ t) (scan (+) 0 r)) xss: per row, the running
    sums divided by the row's sum, in f32 (division as IEEE: a row that sums to zero gives
    NaN or infinities)."""
    xss = _arr(xss, np.float32)
    out = np.empty_like(xss)
    for r in range(xss.shape[0]):
        row = np.ascontiguousarray(xss[r])
        t = np.float32(reduce("add", "f32", row, variant))
        with np.errstate(divide="ignore", invalid="ignore"):
            out[r] = (scan("add", "f32", row, variant).astype(np.float32) / t).astype(np.float32)
    return out


def rbi_vec(op: str, t: str, dest, is_, vss):
    """reduce_by_index dest (map2 op) (replicate m ne) is vss on a copy of dest ([H][m])."""
    _, dt = _CT[t]
    out = np.array(dest, dtype=dt, copy=True, order="C")
    is_ = _arr(is_, np.int64)
    vss = _arr(vss, dt).reshape(is_.size, out.shape[1])
    fn = getattr(lib(), f"orc_rbi_vec_{op}_{t}_lit")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(out), out.shape[0], out.shape[1], _p(is_), _p(vss), is_.size)
    return out


def rbi_2d(op: str, t: str, dest, is_, js, vs):
    """reduce_by_index_2d dest op ne (zip is js) vs on a copy of dest ([H0][H1])."""
    _, dt = _CT[t]
    out = np.array(dest, dtype=dt, copy=True, order="C")
    is_, js, vs = _arr(is_, np.int64), _arr(js, np.int64), _arr(vs, dt)
    fn = getattr(lib(), f"orc_rbi_2d_{op}_{t}_lit")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(out), out.shape[0], out.shape[1], _p(is_), _p(js), _p(vs), is_.size)
    return out


def hist(op: str, t: str, k: int, is_, vs, variant: str = "lit"):
    _, dt = _CT[t]
    return rbi(op, t, np.full(k, NEUTRAL[(op, t)], dtype=dt), is_, vs, variant)


def scanrows(op: str, t: str, xss, variant: str = "lit"):
    """map (scan op ne) xss: every row scanned on its own."""
    _, dt = _CT[t]
    xss = _arr(xss, dt)
    out = np.empty_like(xss)
    for r in range(xss.shape[0]):
        out[r] = scan(op, t, xss[r], variant)
    return out


def vecscan(op: str, t: str, xss, variant: str = "lit"):
    """scan (map2 op) (replicate k ne) xss for xss : [n][k]t, evaluated as the
    sequential loop of FirstOrderTransform.hs:613-656 with the vector operator:
    acc = replicate k ne; for i < n: acc = map2 op acc xss[i]; out[i] = acc.
    Column j of the result therefore is the scan of column j."""
    _, dt = _CT[t]
    xss = _arr(xss, dt)
    out = np.empty_like(xss)
    for j in range(xss.shape[1] if xss.ndim == 2 else 0):
        out[:, j] = scan(op, t, np.ascontiguousarray(xss[:, j]), variant)
    return out


def seghist(op: str, t: str, k: int, iss, vss, variant: str = "lit"):
    """map2 (hist op ne k) iss vss (tests/hist/segmented.fut): one histogram per row."""
    _, dt = _CT[t]
    iss, vss = np.asarray(iss), np.asarray(vss)
    out = np.empty((iss.shape[0], k), dtype=dt)
    for r in range(iss.shape[0]):
        out[r] = hist(op, t, k, iss[r], vss[r], variant)
    return out


def bmm_f32(A, B, variant: str = "f64acc"):
    A, B = _arr(A, np.float32), _arr(B, np.float32)
    if A.ndim == 2:
        A, B = A[None], B[None]
        squeeze = True
    else:
        squeeze = False
    b, M, K = A.shape
    _, K2, N = B.shape
    assert K == K2 and B.shape[0] == b
    out = np.empty((b, M, N), dtype=np.float32)
    fn = getattr(lib(), f"orc_bmm_f32_{variant}")
    fn.restype = None
    fn.argtypes = [C.c_void_p] * 3 + [C.c_int64] * 4
    fn(_p(A), _p(B), _p(out), b, M, N, K)
    return out[0] if squeeze else out


def widen(bits, kind: str):
    bits = _arr(bits, np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    fn = getattr(lib(), f"orc_widen_{kind}")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(bits), _p(out), bits.size)
    return out


def narrow_f16(xs):
    """f32 -> f16, round to nearest even."""
    xs = _arr(xs, np.float32)
    out = np.empty(xs.shape, dtype=np.float16)
    fn = lib().orc_narrow_f16
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
    fn(_p(xs), _p(out), xs.size)
    return out


def radix_sort(keys, vals=None):
    keys = np.ascontiguousarray(keys)
    ko = np.empty_like(keys)
    fn = lib().orc_radix_sort
    fn.restype = None
    fn.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int, C.c_int]
    if vals is None:
        fn(_p(keys), _p(ko), None, None, keys.size, keys.itemsize, 0)
        return ko
    vals = np.ascontiguousarray(vals)
    vo = np.empty_like(vals)
    fn(_p(keys), _p(ko), _p(vals), _p(vo), keys.size, keys.itemsize, vals.itemsize)
    return ko, vo


def transpose_f32(x):
    x = _arr(x, np.float32)
    out = np.empty((x.shape[1], x.shape[0]), dtype=np.float32)
    fn = lib().orc_transpose_f32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]
    fn(_p(x), _p(out), x.shape[0], x.shape[1])
    return out


def lmad_copy(dst, dst_offset, dst_strides, src, src_offset, src_strides, shape):
    """In place on the flat numpy buffer `dst` (same dtype as `src`); strides in elements."""
    assert dst.dtype == src.dtype and dst.flags.c_contiguous and src.flags.c_contiguous
    r = len(shape)
    I64 = C.c_int64 * max(r, 1)
    fn = lib().orc_lmad_copy
    fn.restype = None
    fn.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p,
                   C.c_void_p, C.c_int]
    fn(dst.itemsize, _p(dst), dst_offset, I64(*dst_strides), _p(src), src_offset,
       I64(*src_strides), I64(*shape), r)
    return dst


# ---- futhark-multicore-style CPU baseline (oracle/multicore.c) -------------
def mc_threads() -> int:
    return int(lib().mc_num_threads())


def mc_reduce_add(t: str, xs, threads: int | None = None):
    ct, dt = _CT[t]
    xs = _arr(xs, dt)
    fn = getattr(lib(), f"mc_reduce_add_{t}")
    fn.restype = ct
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int]
    return dt(fn(_p(xs), xs.size, threads or mc_threads()))


def mc_segscan(t: str, flags, xs, op: str = "add", threads: int | None = None, out=None):
    _, dt = _CT[t]
    xs = _arr(xs, dt)
    fl = None if flags is None else _arr(flags, np.uint8)
    if out is None:
        out = np.empty_like(xs)
    fn = getattr(lib(), f"mc_segscan_{t}")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int, C.c_int]
    fn(None if fl is None else _p(fl), _p(xs), xs.size, _p(out), {"add": 0, "max": 1}[op],
       threads or mc_threads())
    return out


def mc_rbi_add_i32(dest, is_, vs, threads: int | None = None):
    dest = _arr(dest, np.int32).copy()
    is_, vs = _arr(is_, np.int32), _arr(vs, np.int32)
    fn = lib().mc_rbi_add_i32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
    fn(_p(dest), dest.size, _p(is_), _p(vs), is_.size, threads or mc_threads())
    return dest


def mc_rbi_f32(op: str, dest, is_, vs, threads: int | None = None):
    dest = _arr(dest, np.float32).copy()
    is_, vs = _arr(is_, np.int32), _arr(vs, np.float32)
    fn = getattr(lib(), f"mc_rbi_{op}_f32")
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
    fn(_p(dest), dest.size, _p(is_), _p(vs), is_.size, threads or mc_threads())
    return dest


def mc_segred_add_f32(offsets, lens, xs, threads: int | None = None, tmp=None):
    """tmp: (u8[n], f32[n]) scratch a caller that times this may keep between calls."""
    xs, offsets, lens = _arr(xs, np.float32), _arr(offsets, np.int64), _arr(lens, np.int64)
    out = np.empty(offsets.size, np.float32)
    ft, st = tmp if tmp is not None else (np.empty(xs.size, np.uint8), np.empty(xs.size, np.float32))
    fn = lib().mc_segred_add_f32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p,
                   C.c_void_p, C.c_int]
    fn(_p(offsets), _p(lens), offsets.size, _p(xs), xs.size, _p(out), _p(ft), _p(st),
       threads or mc_threads())
    return out


def mc_transpose_f32(B, threads: int | None = None):
    B = _arr(B, np.float32)
    b, K, N = B.shape
    Bt = np.empty((b, N, K), np.float32)
    fn = lib().mc_transpose_f32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int]
    fn(_p(B), _p(Bt), b, K, N, threads or mc_threads())
    return Bt


def mc_bmm_rows_f32(A, Bt, C_out, row_lo: int, row_hi: int, threads: int | None = None):
    """Rows [row_lo, row_hi) of the flattened [b*M] rows of C = A x B, with Bt = mc_transpose_f32(B)."""
    A, Bt = _arr(A, np.float32), _arr(Bt, np.float32)
    b, M, K = A.shape
    N = Bt.shape[1]
    assert C_out.shape == (b, M, N) and C_out.dtype == np.float32 and C_out.flags.c_contiguous
    fn = lib().mc_bmm_rows_f32
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                   C.c_int64, C.c_int]
    fn(_p(A), _p(Bt), _p(C_out), M, N, K, row_lo, row_hi, threads or mc_threads())
    return C_out


def mc_transpose_16(B, threads: int | None = None):
    """[b][K][N] 16-bit payloads -> [b][N][K], in parallel over the rows of the result."""
    B = _arr(B, np.uint16)
    b, K, N = B.shape
    Bt = np.empty((b, N, K), np.uint16)
    fn = lib().mc_transpose_16
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int]
    fn(_p(B), _p(Bt), b, K, N, threads or mc_threads())
    return Bt


def mc_bmm_rows_16(A, Bt, C_out, row_lo: int, row_hi: int, bf16: bool, threads: int | None = None):
    """mc_bmm_rows_f32 for f16 (or bf16) bit patterns: widened where they are used, summed in f32."""
    A, Bt = _arr(A, np.uint16), _arr(Bt, np.uint16)
    b, M, K = A.shape
    N = Bt.shape[1]
    assert C_out.shape == (b, M, N) and C_out.dtype == np.float32 and C_out.flags.c_contiguous
    fn = lib().mc_bmm_rows_16
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                   C.c_int64, C.c_int, C.c_int]
    fn(_p(A), _p(Bt), _p(C_out), M, N, K, row_lo, row_hi, 1 if bf16 else 0, threads or mc_threads())
    return C_out


def mc_radix_sort(keys, vals=None, threads: int | None = None):
    keys = np.array(keys, copy=True)
    assert keys.dtype in (np.uint32, np.uint64)
    vals = None if vals is None else np.array(vals, dtype=np.int32, copy=True)
    kt = np.empty_like(keys)
    vt = None if vals is None else np.empty_like(vals)
    fn = lib().mc_radix_sort
    fn.restype = None
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_void_p, C.c_int]
    fn(_p(keys), None if vals is None else _p(vals), keys.size, keys.itemsize, _p(kt),
       None if vt is None else _p(vt), threads or mc_threads())
    return keys if vals is None else (keys, vals)
