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
        a.free()


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
