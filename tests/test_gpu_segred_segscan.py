"""GPU parity: SegRed and SegScan through the generated-library API against the
CPU oracle.  Integers bit-exact; f32 sums within 1e-5 relative of the
f64-accumulated oracle; max/min bit-exact (order-independent)."""
import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 3, 63, 64, 65, 255, 1023, 4095, 4096, 4097, 8191, 100003, (1 << 20) + 7]
NP = {"i32": np.int32, "i64": np.int64, "f32": np.float32, "f64": np.float64}
F32_RTOL = 1e-5


def _data(t, n, aid):
    if t in ("i32", "i64"):
        return dg.uniform_int(aid, n, -1000 if t == "i32" else -(1 << 20),
                              1000 if t == "i32" else (1 << 20), NP[t])
    x = dg.uniform_f32(aid, n)
    return x.astype(NP[t])


def _close(got, want, rtol=F32_RTOL):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + 1e-30
    bad = err > bound
    assert not bad.any(), (int(bad.sum()), float((err / (np.abs(want) + 1e-30)).max()))


@pytest.mark.parametrize("t", ["i32", "i64", "f32", "f64"])
@pytest.mark.parametrize("op", ["add", "max", "min"])
def test_reduce_sizes(ctx, t, op):
    for n in SIZES:
        xs = _data(t, n, 1)
        a = ctx.new(f"{t}_1d", xs)
        got = ctx.call(f"reduce_{op}_{t}", [NP[t]], a)
        a.free()
        if op == "add" and t == "f32":
            _close(got, oracle.reduce(op, t, xs, "f64acc"))
        elif op == "add" and t == "f64":
            _close(got, np.sum(xs.astype(np.longdouble)), 1e-12)
        else:
            assert got == oracle.reduce(op, t, xs), (n, got)


@pytest.mark.parametrize("t", ["i32", "i64", "f32", "f64"])
@pytest.mark.parametrize("op", ["add", "max"])
@pytest.mark.parametrize("excl", [False, True])
def test_scan_sizes(ctx, t, op, excl):
    for n in SIZES:
        xs = _data(t, n, 2)
        a = ctx.new(f"{t}_1d", xs)
        out = ctx.call(f"{'ex' if excl else ''}scan_{op}_{t}", [f"{t}_1d"], a)
        got = out.values()
        assert got.shape == (n,)
        a.free(); out.free()
        if op == "add" and t == "f32":
            _close(got, oracle.scan(op, t, xs, "f64acc", exclusive=excl))
        elif op == "add" and t == "f64":
            want = np.cumsum(xs.astype(np.longdouble))
            if excl:
                want = np.concatenate(([0], want[:-1]))
            _close(got, want, 1e-12)
        else:
            assert np.array_equal(got, oracle.scan(op, t, xs, exclusive=excl)), n


@pytest.mark.parametrize("t", ["i32", "i64", "f32"])
@pytest.mark.parametrize("op", ["add", "max", "min"])
def test_segscan_sizes(ctx, t, op):
    for n in SIZES:
        xs = _data(t, n, 3)
        for mean in (3, 700, 10 ** 9):  # many short, tile-sized, one segment without flags[0]
            flags = (dg.raw_u64(77 + mean % 13, n) % np.uint64(mean) == 0).astype(np.uint8)
            a, f = ctx.new(f"{t}_1d", xs), ctx.new("u8_1d", flags)
            out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, a)
            got = out.values()
            a.free(); f.free(); out.free()
            if op == "add" and t == "f32":
                _close(got, oracle.segscan(op, t, flags, xs, "f64acc"))
            else:
                assert np.array_equal(got, oracle.segscan(op, t, flags, xs)), (n, mean)


def test_segscan_flag_bytes_other_than_one(ctx):
    xs = np.arange(1, 1001, dtype=np.int32)
    flags = np.zeros(1000, np.uint8)
    flags[[0, 10, 500, 999]] = [255, 2, 128, 7]  # nonzero means start (map (!=0))
    a, f = ctx.new("i32_1d", xs), ctx.new("u8_1d", flags)
    out = ctx.call("segscan_add_i32", ["i32_1d"], f, a)
    assert np.array_equal(out.values(), oracle.segscan("add", "i32", flags, xs))


@pytest.mark.parametrize("t", ["i32", "i64", "f32"])
@pytest.mark.parametrize("op", ["add", "max"])
def test_segred_irregular(ctx, t, op):
    for n in [1, 5, 4096, 4097, 100003, (1 << 20) + 7]:
        for mean in (2, 50, 1024, 1 << 22):
            offsets, lens, flags = dg.segments(5, n, mean)
            # sprinkle empty segments (tests/flattening/reduce/nonuniform-2d.fut has one)
            if len(offsets) > 3:
                pos = [0, len(offsets) // 2, len(offsets)]
                offsets = np.insert(offsets, pos, [0, offsets[len(offsets) // 2], n])
                lens = np.insert(lens, pos, [0, 0, 0])
            xs = _data(t, n, 4)
            o, l, v = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens), ctx.new(f"{t}_1d", xs)
            out = ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, v)
            got = out.values()
            for h in (o, l, v, out):
                h.free()
            if op == "add" and t == "f32":
                _close(got, oracle.segred(op, t, offsets, lens, xs, "f64acc"))
            else:
                assert np.array_equal(got, oracle.segred(op, t, offsets, lens, xs)), (n, mean)


def test_segred_gaps_and_unit_segments(ctx):
    """Elements between segments are ignored; segments of one element; a segment
    that spans hundreds of tiles next to short ones."""
    rng = np.random.default_rng(7)
    n = 3_000_017
    xs = rng.integers(-1000, 1000, n).astype(np.int64)
    # unit segments with gaps of varying width, then one very long segment, then a tail gap
    starts = np.cumsum(rng.integers(1, 9, 20000)).astype(np.int64)
    lens = np.ones_like(starts)
    long_start = int(starts[-1]) + 5
    offsets = np.concatenate([starts, [long_start, n - 40]]).astype(np.int64)
    lens = np.concatenate([lens, [n - 100 - long_start, 30]]).astype(np.int64)
    o, l, v = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens), ctx.new("i64_1d", xs)
    for op in ("add", "max"):
        out = ctx.call(f"segred_{op}_i64", ["i64_1d"], o, l, v)
        assert np.array_equal(out.values(), oracle.segred(op, "i64", offsets, lens, xs)), op
        out.free()
    for h in (o, l, v):
        h.free()


def test_segred_all_empty_and_no_segments(ctx):
    o = ctx.new("i64_1d", np.zeros(4, np.int64)); l = ctx.new("i64_1d", np.zeros(4, np.int64))
    v = ctx.new("f32_1d", np.zeros(0, np.float32))
    out = ctx.call("segred_max_f32", ["f32_1d"], o, l, v)
    assert np.array_equal(out.values(), np.full(4, -np.inf, np.float32))
    e = ctx.new("i64_1d", np.zeros(0, np.int64))
    v2 = ctx.new("f32_1d", np.ones(10, np.float32))
    out2 = ctx.call("segred_add_f32", ["f32_1d"], e, e, v2)
    assert out2.values().shape == (0,)


def test_reference_goldens_on_gpu(ctx, goldens):
    for c in goldens["reduce0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        assert int(ctx.call("reduce_add_i32", [np.int32], ctx.new("i32_1d", xs))) == c["out"]
    for c in goldens["scan0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        out = ctx.call("scan_add_i32", ["i32_1d"], ctx.new("i32_1d", xs))
        assert int(out.index(c["n"] - 1)) == c["out"]
    for c in goldens["exscan0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        out = ctx.call("exscan_add_i32", ["i32_1d"], ctx.new("i32_1d", xs))
        assert int(out.index(c["n"] - 1)) == c["out"]
    c = goldens["scan4"]["cases"][0]
    xs = np.array(c["in"], np.int32)
    for _ in range(2):
        bits = ctx.new("i32_1d", xs + 1)
        ps = ctx.call("scan_add_i32", ["i32_1d"], bits).values()
        s = ctx.call("reduce_add_i32", [np.int32], bits)
        xs = ps + s + xs
    assert xs.tolist() == c["out"]
    c = goldens["nonuniform_2d"]["cases"][0]
    sizes = np.array(c["sizes"], np.int64)
    lens = 3 * sizes
    offsets = np.concatenate(([0], np.cumsum(lens)[:-1]))
    vals = np.concatenate([(np.arange(3)[:, None] + np.arange(s)[None, :]).ravel() for s in sizes])
    out = ctx.call("segred_add_i64", ["i64_1d"], ctx.new("i64_1d", offsets),
                   ctx.new("i64_1d", lens), ctx.new("i64_1d", vals.astype(np.int64)))
    assert out.values().tolist() == c["out"]


@pytest.mark.parametrize("t", ["i32", "f32"])
def test_segreduce_regular(ctx, goldens, t):
    c = goldens["segsum"]["cases"][0]
    out = ctx.call("segreduce_add_f32", ["f32_1d"], ctx.new("f32_2d", np.array(c["xss"], np.float32)))
    assert out.values().tolist() == c["out"]
    # rows of whole 16-byte vectors and not, every group width, rows folded by whole blocks,
    # a few very long rows (cut into pieces, two stages; 33000 leaves an empty last piece)
    for m, k in [(1, 1), (1000, 1), (1000, 2), (777, 7), (300, 33), (100, 64), (50, 1000),
                 (7, 9001), (3, 70000), (0, 5), (5, 0), (4099, 4), (513, 8), (257, 12), (129, 36),
                 (65, 256), (33, 260), (17, 1028), (9, 8192), (5, 8196), (2, 33000), (3, 1 << 20),
                 (1, 3000001)]:
        xss = _data(t, m * k, 9).reshape(m, k)
        out = ctx.call(f"segreduce_add_{t}", [f"{t}_1d"], ctx.new(f"{t}_2d", xss))
        got = out.values()
        if t == "f32":
            _close(got, xss.astype(np.float64).sum(axis=1))
        else:
            assert np.array_equal(got, oracle.segreduce("add", t, xss))
        outm = ctx.call(f"segreduce_max_{t}", [f"{t}_1d"], ctx.new(f"{t}_2d", xss))
        assert np.array_equal(outm.values(), oracle.segreduce("max", t, xss))


@pytest.mark.parametrize("t", ["i32", "i64", "f32", "f64"])
def test_reduce_with_vectorised_operator(ctx, t):
    """reduce (map2 op) (replicate k ne) xss (tests/soacs/reduce7.fut has the shape): vectors
    shorter than a wave's span (several rows per span, whole 16-byte vectors and not), as long,
    longer (several strips, a ragged last one), one row, no rows, many rows (two stages)."""
    for n, k in [(1, 1), (7, 1), (1000, 2), (1000, 3), (999, 4), (513, 12), (100, 64), (300, 100),
                 (100, 100), (77, 128), (50, 252), (33, 256), (200, 260), (64, 1000), (9, 4099),
                 (100003, 8), (70001, 5), (20000, 96), (3000, 1024), (1, 5000), (0, 6), (6, 0),
                 (2, 1 << 20), (1 << 20, 2), (50000, 257)]:
        xss = _data(t, n * k, 21).reshape(n, k)
        a = ctx.new(f"{t}_2d", xss)
        for op in ("add", "max", "min"):
            out = ctx.call(f"vecreduce_{op}_{t}", [f"{t}_1d"], a)
            got = out.values()
            assert got.shape == (k,)
            if t == "f32" and op == "add":
                _close(got, xss.astype(np.float64).sum(axis=0))
            elif t == "f64" and op == "add":
                _close(got, oracle.vecreduce(op, t, xss), 1e-12)
            else:
                assert np.array_equal(got, oracle.vecreduce(op, t, xss)), (n, k, op)
            out.free()
        a.free()


def test_config1_full_size(ctx):
    n = 1 << 24
    xi = dg.uniform_int(16, n, -1000, 1000)
    a = ctx.new("i32_1d", xi)
    assert ctx.call("reduce_add_i32", [np.int32], a) == oracle.reduce("add", "i32", xi)
    out = ctx.call("scan_add_i32", ["i32_1d"], a)
    assert np.array_equal(out.values(), oracle.scan("add", "i32", xi))
    a.free(); out.free()
    xf = dg.uniform_f32(17, n)
    a = ctx.new("f32_1d", xf)
    ref = float(oracle.reduce("add", "f32", xf, "f64acc"))
    got = float(ctx.call("reduce_add_f32", [np.float32], a))
    _close(got, ref)
    out = ctx.call("scan_add_f32", ["f32_1d"], a)
    _close(out.values(), oracle.scan("add", "f32", xf, "f64acc"))
    # The literal `futhark c` left fold in f32 is itself far from the exact sum at this size
    # (about 1.3e-4 relative), which is why the f64-accumulated value is the yardstick.
    lit = float(oracle.reduce("add", "f32", xf))
    dev_gpu, dev_lit = abs(got - ref) / ref, abs(lit - ref) / ref
    print(f"\nreduce (+) f32 2^24: GPU deviates {dev_gpu:.2e} from the f64-accumulated sum, "
          f"the sequential f32 fold {dev_lit:.2e}")
    assert dev_lit > 2e-5 and dev_gpu < dev_lit
    a.free(); out.free()


@pytest.mark.parametrize("t,op", [("f32", "add"), ("f32", "max"), ("i64", "add"), ("i64", "max")])
def test_config2_full_size(ctx, t, op):
    n = 1 << 26
    offsets, lens, flags = dg.segments(32, n, 1024)
    xs = _data(t, n, 33)
    f, v = ctx.new("u8_1d", flags), ctx.new(f"{t}_1d", xs)
    out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, v)
    got = out.values()
    out.free()
    if (t, op) == ("f32", "add"):
        _close(got, oracle.segscan(op, t, flags, xs, "f64acc"))
    else:
        assert np.array_equal(got, oracle.segscan(op, t, flags, xs))
    # size-independent property: last scanned element of a segment == its reduction
    o, l = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens)
    red = ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, v).values()
    ends = offsets + lens - 1
    if (t, op) == ("f32", "add"):
        ref = oracle.segred(op, t, offsets, lens, xs, "f64acc")
        _close(red, ref)
        _close(red, got[ends], 2e-6)
        # informational: per segment (mean 1024 elements) the literal f32 fold stays close too
        lit = oracle.segred(op, t, offsets, lens, xs)
        nz = ref != 0
        print(f"\nsegmented (+) f32: max relative deviation from the f64-accumulated sums: GPU "
              f"{np.abs(red[nz] - ref[nz]).max() and (np.abs(red[nz] - ref[nz]) / np.abs(ref[nz])).max():.2e}, "
              f"sequential f32 fold {(np.abs(lit[nz] - ref[nz]) / np.abs(ref[nz])).max():.2e}")
    else:
        assert np.array_equal(red, got[ends])
        assert np.array_equal(red, oracle.segred(op, t, offsets, lens, xs))


@pytest.mark.parametrize("t,op", [("i32", "add"), ("f32", "max"), ("i64", "add"), ("f32", "add"),
                                  ("i32", "xor")])
def test_scan_of_rows(ctx, t, op):
    """map (scan op ne) xss: rows shorter than a 16-byte vector, rows that straddle lanes, waves
    and tiles, rows longer than a tile, a ragged last tile; the flag-driven scan of the same data
    must agree."""
    for m, k in [(5, 1), (1000, 2), (999, 3), (300, 7), (70, 256), (33, 257), (1000, 1024),
                 (9, 32768), (5, 40001), (3, 300000), (1, 12345), (0, 4), (4, 0), (100003, 10)]:
        xss = _data(t, m * k, 13).reshape(m, k)
        a = ctx.new(f"{t}_2d", xss)
        out = ctx.call(f"scanrows_{op}_{t}", [f"{t}_2d"], a)
        got = out.values()
        assert got.shape == (m, k)
        if t == "f32" and op == "add":
            want = np.cumsum(xss.astype(np.float64), axis=1)
            _close(got.reshape(-1), want.reshape(-1))
        else:
            assert np.array_equal(got, oracle.scanrows(op, t, xss)), (m, k)
        if m * k > 0:
            flags = np.zeros(m * k, np.uint8)
            flags[::k] = 1
            f, v = ctx.new("u8_1d", flags), ctx.new(f"{t}_1d", xss.reshape(-1))
            same = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, v)
            if t == "f32" and op == "add":
                # rows longer than a tile take their prefix from whichever mix of tile aggregates
                # and prefixes the look-back finds published: the sum order is not fixed
                _close(same.values(), got.reshape(-1))
            else:
                assert np.array_equal(same.values(), got.reshape(-1)), (m, k)
            for h in (same, f, v):
                h.free()
        out.free(); a.free()


FA_DTYPE = {"i32": 0, "i64": 1, "f32": 2, "f64": 3}


def _tile_elems(t):
    """Elements per look-back tile, as the kernel library states it."""
    import ctypes as C
    from futhark_amd import lib_path
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_segscan_tile_elems.restype = C.c_int64
    k.fa_segscan_tile_elems.argtypes = [C.c_int]
    tile = int(k.fa_segscan_tile_elems(FA_DTYPE[t]))
    assert tile > 0 and tile * NP[t]().itemsize == int(k.fa_segscan_tile_elems(FA_DTYPE["i32"])) * 4
    return tile


@pytest.mark.parametrize("t", ["i32", "i64"])
def test_segscan_long_look_back_chains(ctx, t):
    """Flag patterns chosen for the look-back: segment starts hundreds of tiles apart (chains that
    cross several 64-tile windows before they meet a start), starts exactly on tile boundaries and
    on their neighbours, and runs of tiles with and without starts in turn.  The tile size is the
    kernel's own; 600 tiles and a ragged end."""
    tile = _tile_elems(t)
    n = 600 * tile + 4099
    xs = _data(t, n, 21)
    a = ctx.new(f"{t}_1d", xs)
    patterns = {
        "four starts": [0, n // 3 + 5, n // 2, n - 7],
        "on tile boundaries": [k * tile for k in range(0, n // tile, 37)],
        "around tile boundaries": [k * tile + d for k in range(1, n // tile, 29) for d in (-1, 1)],
        "dense then none": list(range(0, 5 * tile, 97)) + [200 * tile + 3],
        "alternating tiles": [k * tile + tile // 2 for k in range(0, n // tile, 2)],
        "last element only": [n - 1],
    }
    for name, starts in patterns.items():
        flags = np.zeros(n, np.uint8)
        flags[np.array(starts)] = 1
        f = ctx.new("u8_1d", flags)
        for op in ("add", "max"):
            out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, a)
            assert np.array_equal(out.values(), oracle.segscan(op, t, flags, xs)), (name, op)
            out.free()
        f.free()
    a.free()


def test_scan_with_a_non_commutative_operator(ctx):
    """Composition of affine maps modulo 2^32 (associative, not commutative): every place where
    the kernel combines two partial results - inside a thread, across lanes, rows, waves and the
    look-back over tiles - must keep the operands in order, or some element differs.  Sizes from
    one element to many tiles, ragged ends, segment starts dense and hundreds of tiles apart."""
    rng = np.random.default_rng(17)
    tile = _tile_elems("i64")  # an affine map is a pair of i32: eight bytes
    for n in [0, 1, 2, 63, 64, 65, 4097, tile - 1, tile, tile + 1, 5 * tile + 3, 700 * tile + 11]:
        abs_ = rng.integers(-2**31, 2**31, (n, 2), dtype=np.int64).astype(np.int32)
        a = ctx.new("i32_2d", abs_)
        for excl in (False, True):
            out = ctx.call(("exscan" if excl else "scan") + "_compose_i32", ["i32_2d"], a)
            assert out.shape == (n, 2)
            assert np.array_equal(out.values(), oracle.scan_compose_i32(abs_, None, excl)), (n, excl)
            out.free()
        for every in (3, 1000, 300 * tile):
            flags = np.zeros(n, np.uint8)
            flags[::every] = 1
            if n > 10:
                flags[rng.integers(0, n, 3)] = 1
            f = ctx.new("u8_1d", flags)
            out = ctx.call("segscan_compose_i32", ["i32_2d"], f, a)
            assert np.array_equal(out.values(), oracle.scan_compose_i32(abs_, flags)), (n, every)
            out.free(); f.free()
        a.free()
    bad = ctx.new("i32_2d", np.zeros((4, 3), np.int32))
    with pytest.raises(Exception, match="invalid sizes"):
        ctx.call("scan_compose_i32", ["i32_2d"], bad)
    bad.free()


@pytest.mark.parametrize("t", ["i32", "i64", "f32"])
def test_scans_of_whole_tiles_and_their_neighbours(ctx, t):
    """n = k tiles exactly and one element either side, for the plain scan, the scan with flags
    and the scan of rows: the last tile is whole, one element long, or one element short, and
    with k = 257 and 513 the persistent blocks take more than one and more than two tiles each."""
    tile = _tile_elems(t)
    for k in (1, 2, 3, 257, 513):
        for d in (-1, 0, 1):
            n = k * tile + d
            xs = _data(t, n, 40 + k)
            a = ctx.new(f"{t}_1d", xs)
            for excl in (False, True):
                out = ctx.call(f"{'ex' if excl else ''}scan_add_{t}", [f"{t}_1d"], a)
                if t == "f32":
                    _close(out.values(), oracle.scan("add", t, xs, "f64acc", exclusive=excl))
                else:
                    assert np.array_equal(out.values(), oracle.scan("add", t, xs, exclusive=excl)), (n, excl)
                out.free()
            flags = np.zeros(n, np.uint8)
            starts = [s for s in (0, tile - 1, tile, tile + 1, (k // 2) * tile, n - tile, n - 1) if 0 <= s < n]
            flags[np.array(starts)] = 1
            f = ctx.new("u8_1d", flags)
            for op in ("add", "max"):
                out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, a)
                if t == "f32" and op == "add":
                    _close(out.values(), oracle.segscan(op, t, flags, xs, "f64acc"))
                else:
                    assert np.array_equal(out.values(), oracle.segscan(op, t, flags, xs)), (n, op)
                out.free()
            f.free(); a.free()
    # rows whose length divides the tile, equals it, and exceeds it by one
    for m, k in ((8, tile), (9, tile // 2), (5, tile + 1), (3, 2 * tile - 1), (tile, 3)):
        xss = _data(t, m * k, 47).reshape(m, k)
        a = ctx.new(f"{t}_2d", xss)
        out = ctx.call(f"scanrows_add_{t}", [f"{t}_2d"], a)
        if t == "f32":
            _close(out.values().reshape(-1), np.cumsum(xss.astype(np.float64), axis=1).reshape(-1))
        else:
            assert np.array_equal(out.values(), oracle.scanrows("add", t, xss)), (m, k)
        out.free(); a.free()


def test_more_than_2p31_elements(ctx):
    """Positions beyond 2^31: every index in the kernels and the runtime is 64 bits wide.
    reduce and scan (+) over 2^31 + 4099 i32 (8 GiB in, 8 GiB out), wrap-around sums."""
    n = (1 << 31) + 4099
    block = dg.uniform_int(61, 1 << 20, -1000, 1000, np.int32)
    xs = np.resize(block, n)
    xs[-4099:] = 7
    a = ctx.new("i32_1d", xs)
    want = np.cumsum(xs, dtype=np.int32)
    assert int(ctx.call("reduce_add_i32", [np.int32], a)) == int(want[-1])
    out = ctx.call("scan_add_i32", ["i32_1d"], a)
    got = out.values()
    assert got.shape == (n,)
    assert np.array_equal(got, want)
    out.free(); a.free()


@pytest.mark.parametrize("t", ["i32", "i64"])
def test_reduce_after_scans_on_one_scratch(segops_lib, t):
    """Scans and reductions of a context share the look-back scratch and its
    epoch counter.  A scan of many tiles at epoch 1 leaves final descriptor words
    ending in 8*1+2; eight one-block calls advance the epoch to 10 = 8*1+2
    without touching those slots.  The many-block reduction that follows must
    not take the stale scan words for partials of its own."""
    from futhark_amd import Context
    n = 1 << 22
    xs = _data(t, n, 41)
    small = _data(t, 100, 42)
    for pad in range(0, 10):  # the colliding epoch, and its neighbours
        with Context(segops_lib) as c:
            a, s = c.new(f"{t}_1d", xs), c.new(f"{t}_1d", small)
            out = c.call(f"scan_add_{t}", [f"{t}_1d"], a)
            assert np.array_equal(out.values()[-5:], oracle.scan("add", t, xs)[-5:])
            out.free()
            for _ in range(pad):
                assert c.call(f"reduce_add_{t}", [NP[t]], s) == oracle.reduce("add", t, small)
            for _ in range(3):
                assert c.call(f"reduce_add_{t}", [NP[t]], a) == oracle.reduce("add", t, xs), pad


def test_segred_reports_segments_that_are_not_segments(segops_lib):
    """Offsets and lengths that overlap, run backwards or leave the array are an error a
    compiled program reports at the next synchronisation; good ones right after work."""
    from futhark_amd import Context, FutharkError
    n = 1000
    xs = _data("i32", n, 9)
    bad_cases = [([0, 10], [20, 5]),          # the first runs into the second
                 ([50, 10], [5, 5]),          # out of order
                 ([0, 990], [10, 20]),        # past the end
                 ([-1, 10], [5, 5]),          # before the start
                 ([0, 10], [5, -2])]          # a negative length
    with Context(segops_lib) as c:
        v = c.new("i32_1d", xs)
        for offs, lens in bad_cases:
            o, l = c.new("i64_1d", np.array(offs, np.int64)), c.new("i64_1d", np.array(lens, np.int64))
            with pytest.raises(FutharkError) as e:
                out = c.call("segred_add_i32", ["i32_1d"], o, l, v)
                c.sync()
            assert e.value.code == 2 and "segments" in e.value.message
        o, l = c.new("i64_1d", np.array([0, 10, 500], np.int64)), c.new("i64_1d", np.array([10, 0, 500], np.int64))
        out = c.call("segred_add_i32", ["i32_1d"], o, l, v)
        c.sync()
        assert np.array_equal(out.values(), oracle.segred("add", "i32", np.array([0, 10, 500]), np.array([10, 0, 500]), xs))


@pytest.mark.parametrize("t,op", [("i32", "add"), ("f32", "max"), ("i64", "add"), ("f32", "add"),
                                  ("i32", "xor")])
def test_scan_with_a_vector_operator(ctx, t, op):
    """scan (map2 op) (replicate k ne) xss: column j of the result is the scan of column j.
    Shapes: one column (an ordinary scan), few and many columns, more rows than a tile of the row
    scan holds, sizes off every tile of the transposes, empty in either dimension; rows of whole
    strips with fewer rows than chunks, rows that do not divide into chunks, one row."""
    for n, k in [(1, 1), (1000, 1), (7, 3), (1, 300), (1000, 4), (333, 33), (40001, 5), (70, 1000),
                 (20000, 64), (0, 4), (4, 0),
                 # rows of whole 1 KiB strips take the kernels without a transposed copy
                 (5, 256), (1000, 256), (40001, 512), (17, 1024), (1, 768), (3000, 128), (16385, 256),
                 # ... and so do rows of whole 16-byte units: a last strip that is not full,
                 (1000, 100), (40001, 68), (333, 260), (50, 1028), (9, 300000),
                 # rows of 16 to 128 bytes, several to a wave-wide load (ragged last loads,
                 # fewer rows than a load holds, many chunks),
                 (1, 4), (63, 4), (64, 4), (65, 4), (100003, 4), (5000, 8), (70001, 16), (33, 32),
                 (1 << 20, 4), (300000, 2),
                 # and enough strips to fill the chip with one chunk: the input is read once
                 (100, 1 << 18), (17, (1 << 18) + 4)]:
        xss = _data(t, n * k, 17).reshape(n, k)
        out = ctx.call(f"vecscan_{op}_{t}", [f"{t}_2d"], ctx.new(f"{t}_2d", xss))
        got = out.values()
        assert got.shape == (n, k)
        if t == "f32" and op == "add":
            _close(got.reshape(-1), np.cumsum(xss.astype(np.float64), axis=0).reshape(-1))
        else:
            assert np.array_equal(got, oracle.vecscan(op, t, xss)), (n, k)
        # the last row is what the reduction with the same operator gives
        if n > 0 and k > 0 and not (t == "f32" and op == "add"):
            red = ctx.call(f"vecreduce_{op}_{t}", [f"{t}_1d"], ctx.new(f"{t}_2d", xss)).values()
            assert np.array_equal(got[-1], red), (n, k)
