"""Seeded random shapes against the oracle, for the entry points whose kernels choose among
several paths by shape (rows per span, strips, pieces, tiles with and without row starts, LDS
ranges, flattened indices).  Integers only, so every comparison is exact."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

OPS = ("add", "max", "min", "xor")


def _shape(rng, total_max):
    """(rows, columns) with a log-uniform number of columns and at most total_max elements."""
    k = int(2 ** rng.uniform(0, 17))
    n = int(rng.integers(0, max(1, total_max // k) + 1))
    return n, k


def test_row_shaped_reductions_and_scans(ctx):
    rng = np.random.default_rng(2024)
    for case in range(60):
        n, k = _shape(rng, 300_000)
        t = ("i32", "i64")[case % 2]
        op = OPS[case % 4]
        dt = np.int32 if t == "i32" else np.int64
        xss = rng.integers(-10**6, 10**6, (n, k)).astype(dt)
        a = ctx.new(f"{t}_2d", xss)
        out = ctx.call(f"vecreduce_{op}_{t}", [f"{t}_1d"], a)
        assert np.array_equal(out.values(), oracle.vecreduce(op, t, xss)), ("vecreduce", n, k, op, t)
        out.free()
        out = ctx.call(f"segreduce_{op}_{t}", [f"{t}_1d"], a)
        assert np.array_equal(out.values(), oracle.segreduce(op, t, xss)), ("segreduce", n, k, op, t)
        out.free()
        out = ctx.call(f"scanrows_{op}_{t}", [f"{t}_2d"], a)
        assert np.array_equal(out.values(), oracle.scanrows(op, t, xss)), ("scanrows", n, k, op, t)
        out.free()
        out = ctx.call(f"vecscan_{op}_{t}", [f"{t}_2d"], a)
        assert np.array_equal(out.values(), oracle.vecscan(op, t, xss)), ("vecscan", n, k, op, t)
        out.free()
        a.free()


def test_scans_with_a_vector_operator_over_rows_of_every_width(ctx):
    """vecscan chooses by the bytes of a row: groups of lanes for 16, 32, ... 512 bytes, strips of
    1 KiB of columns from 256 bytes on (a ragged last strip), transposes for the rest; the rows
    are cut into chunks whose first pass runs backwards.  Row counts on both sides of a chunk
    and of a wave-wide load, 4- and 8-byte elements."""
    rng = np.random.default_rng(2027)
    for case in range(48):
        t = ("i32", "i64")[case % 2]
        es = 4 if t == "i32" else 8
        op = OPS[case % 4]
        dt = np.int32 if t == "i32" else np.int64
        row_bytes = [16, 32, 64, 128, 256, 512, 1024, 1040, 2048, 4000, 4096 + 16, 48][case % 12]
        k = row_bytes // es
        n = int(rng.integers(1, max(2, 2_000_000 // k)))
        if case % 5 == 0:
            n = (n // 64) * 64 + int(rng.integers(-1, 2))   # around whole wave-wide loads
        n = max(n, 1)
        xss = rng.integers(-10**6, 10**6, (n, k)).astype(dt)
        a = ctx.new(f"{t}_2d", xss)
        out = ctx.call(f"vecscan_{op}_{t}", [f"{t}_2d"], a)
        assert np.array_equal(out.values(), oracle.vecscan(op, t, xss)), (n, k, op, t)
        out.free(); a.free()


def test_irregular_segments_of_random_lengths(ctx):
    """segred over segments with gaps, empty segments, one-element segments and segments of many
    tiles, laid out at random; integers, exact."""
    rng = np.random.default_rng(2028)
    for case in range(24):
        t = ("i32", "i64")[case % 2]
        op = ("add", "max", "min")[case % 3]
        dt = np.int32 if t == "i32" else np.int64
        m = int(2 ** rng.uniform(0, 14))
        mean = float(2 ** rng.uniform(0, 12))
        lens = rng.geometric(1.0 / mean, m).astype(np.int64) - 1      # zeros included
        if case % 4 == 0:
            lens[int(rng.integers(0, m))] = int(rng.integers(50_000, 400_000))  # one long segment
        gaps = (rng.random(m) < 0.1) * rng.integers(0, 5, m)
        offsets = (np.cumsum(lens + gaps) - lens).astype(np.int64)
        n = int(offsets[-1] + lens[-1] + int(rng.integers(0, 3)))
        vs = rng.integers(-10**6, 10**6, n).astype(dt)
        o, l, v = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens), ctx.new(f"{t}_1d", vs)
        out = ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, v)
        assert np.array_equal(out.values(), oracle.segred(op, t, offsets, lens, vs)), (case, m, n, op, t)
        for h in (out, o, l, v):
            h.free()


def test_shaped_histograms(ctx):
    rng = np.random.default_rng(2025)
    for case in range(40):
        t = ("i32", "i64")[case % 2]
        op = OPS[case % 4]
        dt = np.int32 if t == "i32" else np.int64
        # vector operator: bins from a handful to beyond what LDS ranges hold
        H = int(2 ** rng.uniform(0, 16))
        m = int(2 ** rng.uniform(0, 8))
        n = int(rng.integers(0, 200_000 // m + 1))
        dest = rng.integers(-5, 5, (H, m)).astype(dt)
        is_ = rng.integers(-2, H + 2, n).astype(np.int64)
        vss = rng.integers(-1000, 1000, (n, m)).astype(dt)
        d, i, v = ctx.new(f"{t}_2d", dest), ctx.new("i64_1d", is_), ctx.new(f"{t}_2d", vss)
        out = ctx.call(f"rbi_vec_{op}_{t}", [f"{t}_2d"], d, i, v)
        assert np.array_equal(out.values(), oracle.rbi_vec(op, t, dest, is_, vss)), ("vec", H, m, n, op, t)
        for h in (out, d, i, v):
            h.free()
        # index pairs
        H0, H1 = int(2 ** rng.uniform(0, 11)), int(2 ** rng.uniform(0, 11))
        n = int(rng.integers(0, 200_000))
        dest = rng.integers(-5, 5, (H0, H1)).astype(dt)
        is_ = rng.integers(-2, H0 + 2, n).astype(np.int64)
        js = rng.integers(-2, H1 + 2, n).astype(np.int64)
        vs = rng.integers(-1000, 1000, n).astype(dt)
        d, i, j, v = (ctx.new(f"{t}_2d", dest), ctx.new("i64_1d", is_), ctx.new("i64_1d", js),
                      ctx.new(f"{t}_1d", vs))
        out = ctx.call(f"rbi_2d_{op}_{t}", [f"{t}_2d"], d, i, j, v)
        assert np.array_equal(out.values(), oracle.rbi_2d(op, t, dest, is_, js, vs)), ("2d", H0, H1, n, op, t)
        for h in (out, d, i, j, v):
            h.free()
        # one histogram per row
        rows, length, k = int(rng.integers(1, 40)), int(rng.integers(0, 5000)), int(2 ** rng.uniform(0, 13))
        iss = rng.integers(-2, k + 2, (rows, length)).astype(np.int32)
        vss = rng.integers(-1000, 1000, (rows, length)).astype(dt)
        i, v = ctx.new("i32_2d", iss), ctx.new(f"{t}_2d", vss)
        out = ctx.call(f"seghist_{op}_{t}", [f"{t}_2d"], k, i, v)
        assert np.array_equal(out.values(), oracle.seghist(op, t, k, iss, vss)), ("rows", rows, length, k, op, t)
        for h in (out, i, v):
            h.free()


def test_flag_segmented_scans_and_reductions(ctx):
    rng = np.random.default_rng(2026)
    for case in range(40):
        t = ("i32", "i64")[case % 2]
        op = OPS[case % 4]
        dt = np.int32 if t == "i32" else np.int64
        n = int(2 ** rng.uniform(0, 21))
        xs = rng.integers(-10**6, 10**6, n).astype(dt)
        flags = (rng.random(n) < 2 ** rng.uniform(-16, -1)).astype(np.uint8)
        f, v = ctx.new("u8_1d", flags), ctx.new(f"{t}_1d", xs)
        out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, v)
        assert np.array_equal(out.values(), oracle.segscan(op, t, flags, xs)), ("segscan", n, op, t)
        out.free()
        starts = np.flatnonzero(flags) if flags.any() and flags[0] else np.concatenate(([0], np.flatnonzero(flags[1:]) + 1))
        offsets = starts.astype(np.int64)
        lens = np.diff(np.concatenate((offsets, [n]))).astype(np.int64)
        o, l = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens)
        out = ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, v)
        assert np.array_equal(out.values(), oracle.segred(op, t, offsets, lens, xs)), ("segred", n, op, t)
        for h in (out, o, l, f, v):
            h.free()
