"""GPU parity for SegOps with a program's own operators and fused maps (the
kernels of csrc/kernels/custom_ops.hip, instantiated from the public template
header): tuple operator argmax in reduce, scan and reduce_by_index (bins locked),
a reduction that does not commute, maps fused before a reduction and on both
sides of a scan.  Integers bit-exact; f32 within 1e-5 of the f64-accumulated oracle."""
import numpy as np
import pytest

import oracle
from futhark_amd import FutharkError, datagen as dg

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 1023, 4096, 4097, 100003, (1 << 20) + 7, (1 << 24) + 1]


def test_reduce_argmax(ctx):
    for n in SIZES:
        xs = dg.uniform_int(21, n, -1000, 1000)          # ties are common
        a = ctx.new("i32_1d", xs)
        out = ctx.call("reduce_argmax_i32", ["i32_1d"], a)
        assert out.values().tolist() == oracle.reduce_argmax_i32(xs).tolist(), n
        a.free(); out.free()
    # the maximum at the very end, at the very start, and everywhere
    n = (1 << 22) + 3
    for where in (n - 1, 0):
        xs = np.zeros(n, np.int32); xs[where] = 7
        assert ctx.call("reduce_argmax_i32", ["i32_1d"], ctx.new("i32_1d", xs)).values().tolist() == [7, where]
    assert ctx.call("reduce_argmax_i32", ["i32_1d"], ctx.new("i32_1d", np.full(n, 5, np.int32))).values().tolist() == [5, 0]


def test_scan_argmax(ctx):
    for n in SIZES[:-1]:
        xs = dg.uniform_int(22, n, -100000, 100000)
        vis = np.stack([xs, np.arange(n, dtype=np.int32)], axis=1)
        a = ctx.new("i32_2d", vis.reshape(n, 2))
        out = ctx.call("scan_argmax_i32", ["i32_2d"], a)
        assert np.array_equal(out.values(), oracle.scan_argmax_i32(vis)), n
        a.free(); out.free()
    with pytest.raises(FutharkError):
        ctx.call("scan_argmax_i32", ["i32_2d"], ctx.new("i32_2d", np.zeros((5, 3), np.int32)))


def test_reduce_with_an_operator_that_does_not_commute(ctx):
    rng = np.random.default_rng(3)
    for n in SIZES:
        abs_ = rng.integers(-2 ** 31, 2 ** 31, (n, 2)).astype(np.int32)
        a = ctx.new("i32_2d", abs_.reshape(n, 2))
        out = ctx.call("reduce_compose_i32", ["i32_1d"], a)
        assert out.values().tolist() == oracle.reduce_compose_i32(abs_).tolist(), n
        a.free(); out.free()
    # swapping two neighbours changes the result, so operand order is really checked
    abs_ = np.array([[2, 3], [5, 7]], np.int32)
    assert oracle.reduce_compose_i32(abs_).tolist() != oracle.reduce_compose_i32(abs_[::-1]).tolist()


def test_maps_fused_into_reduce_and_scan(ctx):
    for n in SIZES:
        xs = (dg.uniform_f32(23, n) * 4 - 2).astype(np.float32)
        a = ctx.new("f32_1d", xs)
        got = ctx.call("sumsq_f32", [np.float32], a)
        want = oracle.sumsq_f32(xs, "f64acc")
        assert abs(float(got) - float(want)) <= 1e-5 * abs(float(want)) + 1e-30, n
        out = ctx.call("scan_norm_f32", ["f32_1d"], a)
        wn = oracle.scan_norm_f32(xs, "f64acc")
        assert np.all(np.abs(out.values().astype(np.float64) - wn) <= 1e-5 * np.abs(wn) + 1e-30), n
        a.free(); out.free()


def test_hist_with_a_tuple_operator_locks_its_bins(ctx):
    rng = np.random.default_rng(4)
    # up to 8192 bins a block keeps its own in LDS; beyond, every update locks its bin in the
    # destination (the reference's pass over global memory with locks, SegHist.hs:377-467)
    for n, H in [(0, 5), (1, 1), (1000, 7), (100003, 256), ((1 << 22) + 5, 256), ((1 << 22) + 5, 8192),
                 (300000, 1), (5, 0), (200003, 8193), ((1 << 21) + 3, 100000), (500000, 3_000_000)]:
        xs = rng.integers(-50, 50, n).astype(np.int32)           # ties in every bin
        is_ = dg.hist_indices(24, n, max(H, 1), "zipf") if n else np.zeros(0, np.int32)
        out = ctx.call("hist_argmax_i32", ["i32_2d"], H, ctx.new("i32_1d", is_), ctx.new("i32_1d", xs))
        assert out.shape == (H, 2)
        assert np.array_equal(out.values(), oracle.hist_argmax_i32(H, is_, xs)), (n, H)
        out.free()
    with pytest.raises(FutharkError):
        ctx.call("hist_argmax_i32", ["i32_2d"], -1, ctx.new("i32_1d", np.zeros(4, np.int32)),
                 ctx.new("i32_1d", np.zeros(4, np.int32)))


def test_segops_inside_a_block(ctx):
    """rows_fraction_f32: a reduction, a scan and a map over each row by one block.  Rows
    shorter than a wave, off the four elements a thread takes, longer than a chunk of the
    scan, more rows than blocks, empty in either dimension; a row that sums to zero divides
    as IEEE says.  Tolerance 1e-5 relative (positive data, f32 sums in another order)."""
    for m, k in [(1, 1), (5, 3), (7, 64), (9, 255), (6, 256), (5, 257), (3, 1023), (4, 1024), (3, 1025), (2, 40001), (5000, 17),
                 (0, 4), (4, 0),
                 # rows of 4, 8, ... 256 elements share a wave-wide load: whole and ragged last loads
                 (1, 4), (4097, 4), (1000, 8), (33, 16), (65, 32), (5000, 64), (100, 128), (13, 256), (20000, 256)]:
        xss = (dg.uniform_f32(25, m * k) + np.float32(0.01)).reshape(m, k)
        out = ctx.call("rows_fraction_f32", ["f32_2d"], ctx.new("f32_2d", xss))
        got = out.values()
        assert got.shape == (m, k)
        want = oracle.rows_fraction_f32(xss, "f64acc")
        assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-5 * np.abs(want) + 1e-30), (m, k)
        if m and k:
            assert np.all(np.abs(got[:, -1] - 1.0) <= 1e-5)
    z = np.zeros((2, 5), np.float32)
    z[1] = [1, -1, 2, -2, 0]
    got = ctx.call("rows_fraction_f32", ["f32_2d"], ctx.new("f32_2d", z)).values()
    want = oracle.rows_fraction_f32(z)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
    assert np.array_equal(np.sign(got[np.isinf(got)]), np.sign(want[np.isinf(want)]))


def test_two_operators_in_one_reduction(ctx):
    """reduce_summax_f32: sum and maximum side by side, every element read once.  The maximum is
    exact; the sum within 1e-5 of the f64-accumulated oracle (mixed signs: relative to sum |x|)."""
    for n in SIZES:
        xs = (dg.uniform_f32(27, n) * 4 - 2).astype(np.float32)
        got = ctx.call("reduce_summax_f32", ["f32_1d"], ctx.new("f32_1d", xs)).values()
        want = oracle.reduce_summax_f32(xs, "f64acc")
        assert got.shape == (2,)
        assert abs(float(got[0]) - float(want[0])) <= 1e-5 * float(np.abs(xs).sum(dtype=np.float64)) + 1e-30, n
        assert float(got[1]) == float(want[1]) or (n == 0 and np.isneginf(got[1])), n


def test_custom_operators_in_the_segmented_forms(ctx):
    """The program's own operators in `map (reduce op ne)`, `map (scan op ne)` and over irregular
    segments: argmax (a tuple, made from the row by a fused map) and composition of affine maps
    (not commutative, so every row must be folded in element order).  Row lengths on both sides
    of every change of lane-group size and of the change to one block per row; bit-exact."""
    rng = np.random.default_rng(8)
    for m, k in [(0, 5), (3, 0), (1, 1), (1000, 2), (999, 3), (513, 8), (300, 9), (77, 64), (50, 65),
                 (9, 1000), (5, 16384), (3, 16385), (2, 100003), (70000, 5)]:
        xss = rng.integers(-50, 50, (m, k)).astype(np.int32)     # ties in every row
        a = ctx.new("i32_2d", xss)
        out = ctx.call("segreduce_argmax_i32", ["i32_2d"], a)
        assert out.shape == (m, 2)
        assert np.array_equal(out.values(), oracle.segreduce_argmax_i32(xss)), (m, k)
        out.free(); a.free()
        abs_ = rng.integers(-2**31, 2**31, (m * k, 2), dtype=np.int64).astype(np.int32)
        a = ctx.new("i32_2d", abs_)
        if k > 0:
            out = ctx.call("segreduce_compose_i32", ["i32_2d"], k, a)
            assert out.shape == (m, 2)
            assert np.array_equal(out.values(), oracle.segreduce_compose_i32(k, abs_)), (m, k)
            out.free()
            vis = np.stack([rng.integers(-50, 50, m * k), np.arange(m * k) % k], axis=1).astype(np.int32)
            v = ctx.new("i32_2d", vis)
            out = ctx.call("scanrows_argmax_i32", ["i32_2d"], k, v)
            assert np.array_equal(out.values(), oracle.scanrows_argmax_i32(k, vis)), (m, k)
            out.free(); v.free()
        a.free()
    bad = ctx.new("i32_2d", np.zeros((10, 2), np.int32))
    for entry in ("segreduce_compose_i32", "scanrows_argmax_i32"):
        with pytest.raises(FutharkError, match="invalid sizes"):
            ctx.call(entry, ["i32_2d"], 3, bad)          # 10 pairs are no rows of 3
    bad.free()
    # irregular segments: geometric lengths with empty segments in between, and pairs behind
    # the last segment that belong to nobody
    for n, mean in [(0, 4), (1, 1), (5000, 3), (300007, 50), ((1 << 21) + 11, 1000)]:
        lens = rng.geometric(1.0 / mean, max(1, n // mean) + 5).astype(np.int64) - 1 if n else np.zeros(3, np.int64)
        lens = lens[np.cumsum(lens) <= n]
        offsets = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int64) if lens.size else np.zeros(0, np.int64)
        vis = np.stack([rng.integers(-50, 50, n), np.arange(n)], axis=1).astype(np.int32)
        o, l, v = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens), ctx.new("i32_2d", vis)
        out = ctx.call("segred_argmax_i32", ["i32_2d"], o, l, v)
        assert out.shape == (lens.size, 2)
        assert np.array_equal(out.values(), oracle.segred_argmax_i32(offsets, lens, vis)), (n, mean)
        for h in (o, l, v, out):
            h.free()
