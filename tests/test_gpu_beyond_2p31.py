"""Inputs with more than 2^31 elements: every index computation on the path has
to be 64-bit (the reference sizes everything as i64, ImpGen/GPU/Base.hs).  The
data follow closed forms, so the expected results need no second pass over
17 GB on the host: xs[i] = (i mod 7) - 3 sums to 0 over every period, and its
inclusive scan is P[i mod 7] with P = [-3, -5, -6, -6, -5, -3, 0]."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

N = (1 << 31) + 12345
P = np.array([-3, -5, -6, -6, -5, -3, 0], np.int32)


def _pattern(n):
    xs = np.empty(n, np.int32)
    step = 7 * (1 << 22)
    block = (np.arange(step, dtype=np.int32) % 7 - 3).astype(np.int32)
    for lo in range(0, n, step):
        hi = min(lo + step, n)
        xs[lo:hi] = block[: hi - lo]
    return xs


def test_reduce_and_scans_over_more_than_2p31_elements(ctx):
    xs = _pattern(N)
    a = ctx.new("i32_1d", xs)
    del xs
    want_sum = int(P[(N - 1) % 7])
    assert ctx.call("reduce_add_i32", [np.int32], a) == want_sum
    assert ctx.call("reduce_max_i32", [np.int32], a) == 3
    out = ctx.call("scan_add_i32", ["i32_1d"], a)
    got = out.values()
    out.free()
    # the far end in full, the rest at two million sampled positions (and the
    # tile boundaries around 2^31)
    tail = np.arange(N - (1 << 20), N, dtype=np.int64)
    assert np.array_equal(got[tail], P[tail % 7])
    rng = np.random.default_rng(1)
    idx = np.concatenate([rng.integers(0, N, 2_000_000), np.arange((1 << 31) - 70000, (1 << 31) + 12345)])
    assert np.array_equal(got[idx], P[idx % 7])
    del got
    # segmented: a segment start every 1000 elements; inside a segment the scan
    # restarts, so the value depends on the position in the segment and the phase
    flags = np.zeros(N, np.uint8)
    flags[::1000] = 1
    f = ctx.new("u8_1d", flags)
    del flags
    out = ctx.call("segscan_add_i32", ["i32_1d"], f, a)
    got = out.values()
    out.free(); f.free(); a.free()
    idx = np.concatenate([rng.integers(0, N, 1_000_000), np.arange(N - 5000, N)])
    start = idx - idx % 1000
    # sum of xs[start..idx] = S(idx) - S(start - 1), S = the unsegmented scan
    before = np.where(start > 0, P[(start - 1) % 7], 0)
    assert np.array_equal(got[idx], P[idx % 7] - before)


def test_transpose_with_more_blocks_than_one_launch_holds(ctx):
    """[2][2^32 + 4099] bytes -> [2^32 + 4099][2]: the strips of 256 columns are more blocks than a
    launch of 256-thread blocks may have along x (2^32 threads), so the library sends them in
    pieces.  x[r][c] = (3 c + 7 r) mod 251, checked block by block on the host."""
    import ctypes as C
    from futhark_amd import lib_path
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_map_transpose.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                   C.c_int64]
    cols = (1 << 32) + 4099
    period = 251 * (1 << 14)
    base = ((np.arange(period, dtype=np.int64) * 3) % 251).astype(np.uint8)

    def row(r, lo, hi):  # x[r][lo:hi] for lo a multiple of the period
        return ((base[: hi - lo].astype(np.int16) + 7 * r) % 251).astype(np.uint8)

    x = np.empty(2 * cols, np.uint8)
    for r in range(2):
        for lo in range(0, cols, period):
            hi = min(lo + period, cols)
            x[r * cols + lo: r * cols + hi] = row(r, lo, hi)
    s = ctx.new("u8_1d", x)
    del x
    d = ctx.new("u8_1d", np.zeros(2 * cols, np.uint8))
    print("fa_map_transpose u8 batch=1 rows=2 cols=2^32+4099", flush=True)
    assert k.fa_map_transpose(ctx.stream, 1, d.device_ptr, s.device_ptr, 1, 2, cols) == 0
    got = d.values().reshape(cols, 2)
    s.free(); d.free()
    for lo in range(0, cols, period):
        hi = min(lo + period, cols)
        for r in range(2):
            assert np.array_equal(got[lo:hi, r], row(r, lo, hi)), (r, lo)


ODD = 2654435761


def _scrambled(lo, hi):
    """(i * ODD) mod 2^32 for i in [lo, hi): a permutation of the 32-bit numbers over any 2^32
    consecutive i."""
    return ((np.arange(lo, hi, dtype=np.uint64) * np.uint64(ODD)) & np.uint64(0xFFFFFFFF)).astype(np.uint32)


def test_sort_of_more_than_2p32_keys(ctx):
    """From 2^32 - 1 keys on, positions in the output no longer fit 32 bits and the sort counts
    and scatters with 64-bit ones.  keys[i] = (i * odd) mod 2^32 for i < 2^32 + 4099: every
    32-bit number once, the first 4099 of the sequence twice, so the sorted output is known
    position by position: 0, 1, 2, ... with those 4099 values doubled."""
    extra = 4099
    n = (1 << 32) + extra
    step = 1 << 27
    keys = np.empty(n, np.uint32)
    for lo in range(0, n, step):
        hi = min(lo + step, n)
        keys[lo:hi] = _scrambled(lo, hi)
    a = ctx.new("u32_1d", keys)
    del keys
    print("radix_sort_u32 n=2^32+4099", flush=True)
    out = ctx.call("radix_sort_u32", ["u32_1d"], a)
    a.free()
    got = out.values()
    out.free()
    ctx.clear_caches()
    assert got.shape == (n,)
    doubled = np.sort(_scrambled(0, extra)).astype(np.int64)
    second = doubled + np.arange(1, extra + 1)  # where the second copy of each doubled value sits
    for lo in range(0, n, step):
        hi = min(lo + step, n)
        pos = np.arange(lo, hi, dtype=np.int64)
        want = pos - np.searchsorted(second, pos, side="right")
        assert np.array_equal(got[lo:hi], want.astype(np.uint32)), lo


def test_histogram_with_many_bins_over_more_than_2p31_updates(ctx):
    """reduce_by_index into 2^22 bins partitions its updates by bin range, in slices whose
    histograms add up; 2^31 + 12345 updates are nine slices, the last a ragged one.
    is[i] = top 22 bits of (i * odd) mod 2^32, vs[i] = (i mod 7) - 3, dest starts non-zero."""
    H = 1 << 22
    dest = (np.arange(H) % 5).astype(np.int32)
    vs = _pattern(N)
    is_ = np.empty(N, np.int32)
    want = dest.astype(np.int64)
    step = 1 << 27
    for lo in range(0, N, step):
        hi = min(lo + step, N)
        is_[lo:hi] = (_scrambled(lo, hi) >> np.uint32(10)).astype(np.int32)
        want += np.bincount(is_[lo:hi], weights=vs[lo:hi], minlength=H).astype(np.int64)
    d, i, v = ctx.new("i32_1d", dest), ctx.new("i32_1d", is_), ctx.new("i32_1d", vs)
    del is_, vs
    print("rbi_add_i32 H=2^22 n=2^31+12345", flush=True)
    out = ctx.call("rbi_add_i32", ["i32_1d"], d, i, v)
    got = out.values()
    for h in (d, i, v, out):
        h.free()
    ctx.clear_caches()
    assert np.array_equal(got.astype(np.int64), want)
