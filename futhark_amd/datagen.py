"""Seeded synthetic inputs for the benchmark configurations.

Counter-based: element i of array `array_id` is splitmix64 of (seed, array_id, i),
so any box regenerates identical bytes without carrying a random-number stream.
Arrays are produced in chunks to bound temporary memory at 2^27 elements.
"""
from __future__ import annotations

import numpy as np

SEED = 0x5EEDF07A
_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


def _mix(z: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _key(array_id: int, seed: int = SEED) -> np.uint64:
    with np.errstate(over="ignore"):
        k = np.array([np.uint64(seed) + np.uint64(array_id + 1) * _GOLDEN], dtype=np.uint64)
    return _mix(k)[0]


def raw_u64(array_id: int, n: int, start: int = 0, seed: int = SEED) -> np.ndarray:
    """n 64-bit words: word i = mix(key(array_id) + (start+i+1) * golden)."""
    key = _key(array_id, seed)
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        return _mix(key + idx * _GOLDEN)


def _chunks(n: int):
    for s in range(0, n, _CHUNK):
        yield s, min(_CHUNK, n - s)


def uniform_int(array_id: int, n: int, lo: int, hi: int, dtype=np.int32) -> np.ndarray:
    """Integers uniform in [lo, hi]."""
    out = np.empty(n, dtype=dtype)
    span = np.uint64(hi - lo + 1)
    for s, c in _chunks(n):
        r = raw_u64(array_id, c, s) % span
        out[s:s + c] = (r.astype(np.int64) + lo).astype(dtype)
    return out


def uniform_f32(array_id: int, n: int) -> np.ndarray:
    """f32 uniform in [0,1): a 24-bit draw scaled by 2^-24."""
    out = np.empty(n, dtype=np.float32)
    for s, c in _chunks(n):
        r = raw_u64(array_id, c, s) >> np.uint64(40)
        out[s:s + c] = r.astype(np.float32) * np.float32(2.0 ** -24)
    return out


def uniform_u32(array_id: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    for s, c in _chunks(n):
        out[s:s + c] = (raw_u64(array_id, c, s) >> np.uint64(32)).astype(np.uint32)
    return out


def uniform_u64(array_id: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint64)
    for s, c in _chunks(n):
        out[s:s + c] = raw_u64(array_id, c, s)
    return out


def segments(array_id: int, n: int, mean_len: int = 1024):
    """Irregular segments tiling [0,n): lengths geometric with the given mean (>= 1).

    Returns (offsets i64[m], lens i64[m], flags u8[n]); flags[offsets] == 1.
    """
    if n == 0:
        return (np.zeros(0, np.int64), np.zeros(0, np.int64), np.zeros(0, np.uint8))
    p = 1.0 / mean_len
    lens_parts, total, start = [], 0, 0
    while total < n:
        c = max(1024, int((n - total) / mean_len * 1.2) + 16)
        u = (raw_u64(array_id, c, start) >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
        l = 1 + np.floor(np.log1p(-u) / np.log1p(-p)).astype(np.int64)
        lens_parts.append(l)
        total += int(l.sum())
        start += c
    lens = np.concatenate(lens_parts)
    ends = np.cumsum(lens)
    m = int(np.searchsorted(ends, n, side="left")) + 1
    lens = lens[:m].copy()
    lens[-1] -= int(ends[m - 1]) - n
    offsets = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int64)
    flags = np.zeros(n, dtype=np.uint8)
    flags[offsets] = 1
    return offsets, lens.astype(np.int64), flags


def hist_indices(array_id: int, n: int, H: int, dist: str = "uniform",
                 oob_percent: int = 1) -> np.ndarray:
    """i32 bin indices over [0,H), uniform or Zipf(s=1.1) by inverse CDF; about
    oob_percent % of positions hold out-of-range values (half negative, half >= H)."""
    out = np.empty(n, dtype=np.int32)
    cdf = None
    if dist == "zipf":
        w = 1.0 / np.arange(1, H + 1, dtype=np.float64) ** 1.1
        cdf = np.cumsum(w)
        cdf /= cdf[-1]
    elif dist != "uniform":
        raise ValueError(dist)
    for s, c in _chunks(n):
        r = raw_u64(array_id, c, s)
        if cdf is None:
            idx = (r % np.uint64(H)).astype(np.int64)
        else:
            u = (r >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
            idx = np.minimum(np.searchsorted(cdf, u, side="right"), H - 1).astype(np.int64)
        if oob_percent > 0:
            h = raw_u64(array_id + 0x1000, c, s)
            oob = (h % np.uint64(100)) < np.uint64(oob_percent)
            k = ((h >> np.uint64(8)) % np.uint64(1000)).astype(np.int64)
            neg = ((h >> np.uint64(7)) & np.uint64(1)) == 0
            bad = np.where(neg, -1 - k, np.minimum(H + k, 2 ** 31 - 1))
            idx = np.where(oob, bad, idx)
        out[s:s + c] = idx.astype(np.int32)
    return out


def normal_f32(array_id: int, n: int, scale: float = 1.0) -> np.ndarray:
    """N(0,1)*scale by Box-Muller on the counter stream."""
    out = np.empty(n, dtype=np.float32)
    for s, c in _chunks(n):
        r = raw_u64(array_id, c, s)
        u1 = ((r >> np.uint64(40)).astype(np.float64) + 1.0) * 2.0 ** -24  # (0,1]
        u2 = ((r >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.float64) * 2.0 ** -24
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out[s:s + c] = (z * scale).astype(np.float32)
    return out


def to_f16_bits(x: np.ndarray) -> np.ndarray:
    return x.astype(np.float16).view(np.uint16)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even truncation of f32 to its upper 16 bits."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))
    return (r >> np.uint32(16)).astype(np.uint16)
