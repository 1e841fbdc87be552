"""GPU parity: SegHist (hist / reduce_by_index) through the generated-library
API against the CPU oracle.  Integer operators and float max/min bit-exact;
f32 add within 1e-5 relative of the f64-accumulated oracle (atomic order is
not fixed)."""
import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu
NP = {"i32": np.int32, "i64": np.int64, "f32": np.float32, "f64": np.float64}


def _vals(t, n, aid):
    if t in ("i32", "i64"):
        return dg.uniform_int(aid, n, -1000, 1000, NP[t])
    return (dg.uniform_f32(aid, n) - np.float32(0.25)).astype(NP[t])  # mixed signs


def _check(t, op, got, want_lit, want_acc=None):
    if op == "add" and t in ("f32", "f64"):
        ref = want_acc if want_acc is not None else want_lit
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
        assert np.all(err <= 1e-5 * np.abs(ref) + 1e-6), float(err.max())
    else:
        assert np.array_equal(got, want_lit)


@pytest.mark.parametrize("t", ["i32", "i64", "f32", "f64"])
@pytest.mark.parametrize("op", ["add", "max", "min"])
def test_hist_small_and_ragged(ctx, t, op):
    for n, H in [(0, 5), (5, 0), (1, 1), (100, 7), (4097, 256), (100003, 1000), (300001, 32768),
                 (300001, 32769), (200000, 65536), (150000, 100001), (100000, 200000)]:
        is_ = dg.hist_indices(40, n, max(H, 1), "uniform", 3)
        vs = _vals(t, n, 41)
        i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
        out = ctx.call(f"hist_{op}_{t}", [f"{t}_1d"], H, i, v)
        got = out.values()
        assert got.shape == (H,)
        acc = oracle.hist(op, t, H, is_, vs, "f64acc") if (op, t) == ("add", "f32") else None
        _check(t, op, got, oracle.hist(op, t, H, is_, vs), acc)
        for h in (i, v, out):
            h.free()


@pytest.mark.parametrize("t", ["f32", "f64"])
def test_float_sums_every_size_class_exactly(ctx, t):
    """Sums of floats: f32 reads the cell and puts the sum back with compare-and-swap (one to
    four attempts, by the number of copies a bin has, then the float atomic), f64 uses the atomic;
    both keep more copies of a small range than the integer operators.  Bin counts on both sides
    of every change in the number of copies and ranges, uniform and skewed indices, one bin for
    everything; the values are small whole numbers, so the sums are exact in any order and must
    match bit for bit."""
    dt = {"f32": np.float32, "f64": np.float64}[t]
    rng = np.random.default_rng(77)
    n = 600011
    for H in (1, 2, 255, 256, 257, 512, 1024, 1025, 2048, 2049, 4096, 8192, 16385, 40000):
        for how in ("uniform", "skewed", "one"):
            if how == "uniform":
                is_ = rng.integers(-2, H + 2, n).astype(np.int32)
            elif how == "skewed":     # runs of skew between runs without: waves change over and back
                is_ = rng.integers(0, H, n).astype(np.int32)
                hot = (np.arange(n) // 50000) % 2 == 1
                is_[hot] = np.minimum(rng.geometric(0.4, int(hot.sum())) - 1, H - 1).astype(np.int32)
            else:
                is_ = np.full(n, H - 1, np.int32)
            vs = rng.integers(-8, 9, n).astype(dt)
            i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
            out = ctx.call(f"hist_add_{t}", [f"{t}_1d"], H, i, v)
            assert np.array_equal(out.values(), oracle.hist("add", t, H, is_, vs)), (t, H, how)
            for h in (i, v, out):
                h.free()


def test_reference_goldens(ctx, goldens):
    for c in goldens["hist_simple"]["cases"]:
        img = np.array(c["image"], np.int32)
        d, i = ctx.new("i32_1d", np.array(c["dest"], np.int32)), ctx.new("i32_1d", img)
        out = ctx.call("rbi_add_i32", ["i32_1d"], d, i, i)
        assert out.values().tolist() == c["out"]
        assert d.values().tolist() == c["dest"]  # the input is not consumed
    for c in goldens["hist_large"]["cases"]:
        n, m = c["n"], c["m"]
        k = np.arange(m, dtype=np.int64)
        out = ctx.call("hist_add_i32", ["i32_1d"], n, ctx.new("i32_1d", (k % n).astype(np.int32)),
                       ctx.new("i32_1d", k.astype(np.int32)))
        assert int(ctx.call("reduce_add_i32", [np.int32], out)) == c["out"]
        out.free()
    f = lambda xs: np.array([np.nan if x == "nan" else x for x in xs], np.float32)
    for c in goldens["hist_f32"]["cases"]:
        out = ctx.call("rbi_add_f32", ["f32_1d"], ctx.new("f32_1d", f(c["dest"])),
                       ctx.new("i32_1d", np.array(c["is"], np.int32)), ctx.new("f32_1d", f(c["vs"])))
        np.testing.assert_allclose(out.values(), f(c["out"]), rtol=2e-3, equal_nan=True)
    for name, op in (("hist_max", "max"), ("hist_min", "min")):
        for c in goldens[name]["cases"]:
            out = ctx.call(f"rbi_{op}_i32", ["i32_1d"], ctx.new("i32_1d", np.zeros(c["n"], np.int32)),
                           ctx.new("i32_1d", np.array(c["is"], np.int32)),
                           ctx.new("i32_1d", np.array(c["vs"], np.int32)))
            assert out.values().tolist() == c["out"]


def test_float_max_with_nan_and_negative_values(ctx):
    dest = np.array([np.nan, -np.inf, 2.0, -3.0, 0.0, -0.5], np.float32)
    is_ = np.array([0, 0, 1, 1, 2, 3, 3, 4, 5, 5, 9, -1], np.int32)
    vs = np.array([-7.0, -9.0, np.nan, -4.0, 1.0, -2.0, -2.5, -1.0, np.nan, -0.25, 5.0, 5.0], np.float32)
    for op in ("max", "min"):
        out = ctx.call(f"rbi_{op}_f32", ["f32_1d"], ctx.new("f32_1d", dest), ctx.new("i32_1d", is_),
                       ctx.new("f32_1d", vs))
        want = oracle.rbi(op, "f32", dest, is_, vs)
        assert np.array_equal(out.values(), want, equal_nan=True), (op, out.values(), want)


@pytest.mark.parametrize("H", [256, 65536, 1 << 22])
@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_config3_full_size_i32(ctx, H, dist):
    n = 1 << 27
    is_ = dg.hist_indices(48, n, H, dist)
    vs = dg.uniform_int(49, n, -1000, 1000)
    i, v = ctx.new("i32_1d", is_), ctx.new("i32_1d", vs)
    out = ctx.call("hist_add_i32", ["i32_1d"], H, i, v)
    got = out.values()
    assert np.array_equal(got, oracle.hist("add", "i32", H, is_, vs))
    # size-independent property: the total equals the sum of the in-range values
    ok = (is_ >= 0) & (is_ < H)
    assert int(got.astype(np.int64).sum()) == int(vs[ok].astype(np.int64).sum())
    for h in (i, v, out):
        h.free()


@pytest.mark.parametrize("H", [256, 65536, 1 << 22])
@pytest.mark.parametrize("dist", ["uniform", "zipf"])
def test_config3_full_size_f32(ctx, H, dist):
    """f32 (+) and f32 max at 2^27 for every bin count and index distribution of the
    configuration: max bit-exact, sums within 1e-5 of the f64-accumulated oracle."""
    n = 1 << 27
    is_ = dg.hist_indices(48, n, H, dist)
    ws = dg.uniform_f32(50, n)
    i, w = ctx.new("i32_1d", is_), ctx.new("f32_1d", ws)
    out = ctx.call("hist_max_f32", ["f32_1d"], H, i, w)
    assert np.array_equal(out.values(), oracle.hist("max", "f32", H, is_, ws))
    out.free()
    out = ctx.call("hist_add_f32", ["f32_1d"], H, i, w)
    got, ref = out.values(), oracle.hist("add", "f32", H, is_, ws, "f64acc")
    assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(ref))
    # size-independent property: the bins add up to the sum of the in-range weights
    ok = (is_ >= 0) & (is_ < H)
    total = float(ws[ok].astype(np.float64).sum())
    assert abs(float(got.astype(np.float64).sum()) - total) <= 1e-5 * total
    for h in (i, w, out):
        h.free()


# ------------------------------------------------------------ segmented histograms
SEG_SHAPES = [  # (rows, row length, bins per row)
    (3, 3, 10),          # tests/hist/segmented.fut
    (1, 100003, 50),     # a single row is the unsegmented histogram
    (1000, 1, 7),        # rows shorter than a vector
    (777, 3, 5), (50, 1001, 64), (4096, 256, 16),
    (7, 70001, 5000),    # several LDS ranges
    (40, 5003, 30011),   # more bins than one launch of LDS ranges holds: flattened indices
    (0, 5, 3), (4, 0, 3), (4, 6, 0),
]


@pytest.mark.parametrize("t,op", [("i32", "add"), ("i64", "max"), ("f32", "min"), ("i32", "xor"),
                                  ("f64", "add")])
def test_segmented_hist(ctx, t, op):
    rng = np.random.default_rng(17)
    for m, k, H in SEG_SHAPES:
        iss = rng.integers(-2, max(H, 1) + 2, (m, k)).astype(np.int32)
        if t[0] == "f":
            vss = rng.integers(-50, 50, (m, k)).astype(NP[t])  # sums exact in any order
        else:
            vss = rng.integers(-1000, 1000, (m, k)).astype(NP[t])
        i, v = ctx.new("i32_2d", iss), ctx.new(f"{t}_2d", vss)
        out = ctx.call(f"seghist_{op}_{t}", [f"{t}_2d"], H, i, v)
        assert out.shape == (m, H)
        want = oracle.seghist(op, t, H, iss, vss)
        assert np.array_equal(out.values(), want), (m, k, H)
        for h in (out, i, v):
            h.free()


def test_segmented_hist_reference_golden_and_size_check(ctx, goldens):
    c = goldens["hist_segmented"]["cases"][0]
    xss = np.array(c["xss"], np.int32)
    i, v = ctx.new("i32_2d", xss), ctx.new("i32_2d", np.ones_like(xss))
    out = ctx.call("seghist_add_i32", ["i32_2d"], c["m"], i, v)
    assert out.values().tolist() == c["out"]
    out.free()
    w = ctx.new("i32_2d", np.ones((3, 4), np.int32))
    with pytest.raises(Exception, match="invalid sizes"):
        ctx.call("seghist_add_i32", ["i32_2d"], 5, i, w)
    for h in (i, v, w):
        h.free()


def test_segmented_hist_full_size_matches_row_sums(ctx):
    # 2^27 elements in 2^14 rows; every row's histogram total equals the row's in-range sum
    m, k, H = 1 << 14, 1 << 13, 64
    iss = dg.hist_indices(90, m * k, H, "uniform", 1).reshape(m, k)
    vss = dg.uniform_int(91, m * k, -1000, 1000).reshape(m, k)
    i, v = ctx.new("i32_2d", iss), ctx.new("i32_2d", vss)
    out = ctx.call("seghist_add_i32", ["i32_2d"], H, i, v)
    got = out.values()
    ok = (iss >= 0) & (iss < H)
    assert np.array_equal(got.sum(axis=1, dtype=np.int64), np.where(ok, vss, 0).sum(axis=1, dtype=np.int64))
    rows = [0, 1, m // 2, m - 1]
    assert np.array_equal(got[rows], oracle.seghist("add", "i32", H, iss[rows], vss[rows]))
    for h in (out, i, v):
        h.free()


def test_i64_indices_through_the_kernel_library(ctx):
    """fa_seghist takes i64 indices as well (Futhark's hist does; the entry points of this program
    widen i32 ones): every path with is64 = 1 against the oracle, including indices that only fit
    64 bits."""
    import ctypes as C
    from futhark_amd import lib_path
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_seghist.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p,
                             C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_size_t]
    k.fa_seghist_scratch_bytes.restype = C.c_size_t
    k.fa_seghist_scratch_bytes.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int64]
    FA_I32, FA_F32, FA_ADD, FA_MAX = 0, 2, 0, 1
    rng = np.random.default_rng(23)
    n = 300001
    for H in (200, 5000, 200000, 9000000):   # wave-private / LDS, LDS ranges, partitioned, global
        is64 = rng.integers(-3, H + 3, n).astype(np.int64)
        is64[::1000] = (1 << 40) + 5          # far out of range, and not an i32
        is64[1::1000] = -(1 << 35)
        is32 = np.where((is64 >= 0) & (is64 < H), is64, -1).astype(np.int32)
        for t, code, op, opname, vals in (
                ("i32", FA_I32, FA_ADD, "add", rng.integers(-1000, 1000, n).astype(np.int32)),
                ("f32", FA_F32, FA_ADD, "add", rng.integers(-8, 8, n).astype(np.float32)),
                ("f32", FA_F32, FA_MAX, "max", rng.standard_normal(n).astype(np.float32))):
            d_is, d_vs = ctx.new("i64_1d", is64), ctx.new(f"{t}_1d", vals)
            dest0 = oracle.hist(opname, t, H, np.zeros(0, np.int32), vals[:0])   # neutral elements
            dest = ctx.new(f"{t}_1d", dest0)
            sb = k.fa_seghist_scratch_bytes(code, 1, n, H)
            scratch = ctx.new("u8_1d", np.zeros(max(sb, 256), np.uint8))
            print(f"fa_seghist is64 {t} {opname} H={H}", flush=True)
            rc = k.fa_seghist(ctx.stream, code, op, d_is.device_ptr, 1, d_vs.device_ptr, n,
                              dest.device_ptr, H, scratch.device_ptr, sb)
            assert rc == 0
            assert np.array_equal(dest.values(), oracle.hist(opname, t, H, is32, vals)), (t, opname, H)
            for h in (d_is, d_vs, dest, scratch):
                h.free()


def test_hist_with_vector_operator_goldens_and_shapes(ctx, goldens):
    """reduce_by_index dest (map2 op) (replicate m ne) is vss: tests/hist/{array,equiv}.fut, then
    vectors shorter and longer than what a thread loads at once, indices out of range, bins that
    fit one LDS range, several, and none (flattened indices and the partition path)."""
    for name in ("hist_array", "hist_equiv"):
        for c in goldens[name]["cases"]:
            d = ctx.new("i32_2d", np.array(c["dest"], np.int32))
            i = ctx.new("i64_1d", np.array(c["is"], np.int64))
            v = ctx.new("i32_2d", np.array(c["vss"], np.int32))
            out = ctx.call("rbi_vec_add_i32", ["i32_2d"], d, i, v)
            assert out.values().tolist() == c["out"]
            for h in (out, d, i, v):
                h.free()
    rng = np.random.default_rng(3)
    for t, op, H, m, n in [("i32", "add", 5, 1, 1000), ("i32", "add", 100, 3, 5000),
                           ("i64", "max", 33, 4, 4099), ("i32", "xor", 1000, 7, 30001),
                           ("f64", "min", 50, 16, 777), ("i32", "add", 3000, 100, 20000),
                           ("i32", "add", 1 << 15, 64, 50000), ("i64", "add", 2, 1000, 300),
                           ("i32", "min", 0, 4, 10), ("i32", "add", 4, 6, 0)]:
        dt = {"i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        is_ = rng.integers(-3, H + 3, n).astype(np.int64)
        vss = (rng.standard_normal((n, m)) if t == "f64" else rng.integers(-1000, 1000, (n, m))).astype(dt)
        dest = (rng.standard_normal((H, m)) if t == "f64" else rng.integers(-5, 5, (H, m))).astype(dt)
        d, i, v = ctx.new(f"{t}_2d", dest), ctx.new("i64_1d", is_), ctx.new(f"{t}_2d", vss)
        out = ctx.call(f"rbi_vec_{op}_{t}", [f"{t}_2d"], d, i, v)
        assert out.shape == (H, m)
        assert np.array_equal(out.values(), oracle.rbi_vec(op, t, dest, is_, vss)), (t, op, H, m, n)
        for h in (out, d, i, v):
            h.free()
    # f32 sums: tolerance against the f64 accumulation
    H, m, n = 64, 8, 100000
    is_ = rng.integers(0, H, n).astype(np.int64)
    vss = rng.random((n, m), dtype=np.float32)
    d, i, v = ctx.new("f32_2d", np.zeros((H, m), np.float32)), ctx.new("i64_1d", is_), ctx.new("f32_2d", vss)
    out = ctx.call("rbi_vec_add_f32", ["f32_2d"], d, i, v)
    want = np.zeros((H, m))
    np.add.at(want, is_, vss.astype(np.float64))
    assert np.allclose(out.values(), want, rtol=1e-5, atol=0)
    w = ctx.new("f32_2d", np.zeros((n, m + 1), np.float32))
    with pytest.raises(Exception, match="invalid sizes"):
        ctx.call("rbi_vec_add_f32", ["f32_2d"], d, i, w)
    for h in (out, d, i, v, w):
        h.free()


def test_float_sums_into_vector_bins(ctx):
    """reduce_by_index dest (map2 (+)) (replicate m 0) is vss with float elements: bins that a
    wave can keep for itself (16-byte pieces of a row per lane, so m a multiple of 4 f32 or 2 f64)
    and the shapes next to them that take the other kernels; indices out of range, every row on
    one bin, rows longer than a wave's step, enough rows for the unrolled loop and its ragged end,
    i32 indices through the kernel library.  Values are small whole numbers: sums are exact in any
    order, so the comparison with the oracle is bit for bit."""
    import ctypes as C
    from futhark_amd import lib_path
    rng = np.random.default_rng(41)
    cases = [("f32", 256, 16, 700001, "uniform"), ("f32", 256, 16, 5000, "one"),
             ("f32", 7, 4, 1, "uniform"), ("f32", 1, 4, 100000, "uniform"),
             ("f32", 3, 1024, 2001, "uniform"), ("f32", 630, 16, 30011, "skewed"),
             ("f32", 631, 16, 30011, "uniform"),          # one bin too many for a wave: LDS kernel
             ("f32", 100, 6, 30011, "uniform"),           # rows are not whole 16-byte pieces
             ("f64", 256, 8, 300007, "uniform"), ("f64", 50, 2, 99999, "skewed"),
             ("f64", 9, 3, 5000, "uniform")]
    for t, H, m, n, how in cases:
        dt = {"f32": np.float32, "f64": np.float64}[t]
        if how == "one":
            is_ = np.full(n, H // 2, np.int64)
        elif how == "skewed":
            is_ = np.minimum(rng.geometric(0.3, n) - 1, H + 2).astype(np.int64)
        else:
            is_ = rng.integers(-3, H + 3, n).astype(np.int64)
        vss = rng.integers(-8, 9, (n, m)).astype(dt)
        dest = rng.integers(-5, 5, (H, m)).astype(dt)
        d, i, v = ctx.new(f"{t}_2d", dest), ctx.new("i64_1d", is_), ctx.new(f"{t}_2d", vss)
        print(f"rbi_vec_add_{t} H={H} m={m} n={n} {how}", flush=True)
        out = ctx.call(f"rbi_vec_add_{t}", [f"{t}_2d"], d, i, v)
        want = oracle.rbi_vec("add", t, dest, is_, vss)
        assert np.array_equal(out.values(), want), (t, H, m, n, how)
        for h in (out, d, i, v):
            h.free()
    # i32 indices: the kernel library directly
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_seghist_shaped.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                                    C.c_void_p, C.c_int64, C.c_void_p, C.c_int64, C.c_int64,
                                    C.c_int64, C.c_void_p, C.c_size_t]
    k.fa_seghist_shaped_scratch_bytes.restype = C.c_size_t
    k.fa_seghist_shaped_scratch_bytes.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64,
                                                  C.c_int64]
    FA_F32, FA_ADD = 2, 0
    H, m, n = 100, 8, 123457
    is32 = rng.integers(-3, H + 3, n).astype(np.int32)
    vss = rng.integers(-8, 9, (n, m)).astype(np.float32)
    dest0 = rng.integers(-5, 5, (H, m)).astype(np.float32)
    d_is, d_vs, dest = ctx.new("i32_1d", is32), ctx.new("f32_2d", vss), ctx.new("f32_2d", dest0)
    sb = k.fa_seghist_shaped_scratch_bytes(FA_F32, 0, n, H, 1, m)
    scratch = ctx.new("u8_1d", np.zeros(max(sb, 256), np.uint8))
    print("fa_seghist_shaped f32 with i32 indices", flush=True)
    rc = k.fa_seghist_shaped(ctx.stream, FA_F32, FA_ADD, d_is.device_ptr, None, 0, d_vs.device_ptr,
                             n, dest.device_ptr, H, 1, m, scratch.device_ptr, sb)
    assert rc == 0
    assert np.array_equal(dest.values(), oracle.rbi_vec("add", "f32", dest0, is32.astype(np.int64), vss))
    for h in (d_is, d_vs, dest, scratch):
        h.free()


def test_hist_with_2d_indices_goldens_and_shapes(ctx, goldens):
    """reduce_by_index_2d: tests/hist/hist2d.fut (an update is dropped when either coordinate is
    outside), then random cases of both sizes of bin space."""
    for c in goldens["hist2d"]["cases"]:
        d = ctx.new("i32_2d", np.array(c["dest"], np.int32))
        i, j = ctx.new("i64_1d", np.array(c["is"], np.int64)), ctx.new("i64_1d", np.array(c["js"], np.int64))
        v = ctx.new("i32_1d", np.array(c["vs"], np.int32))
        out = ctx.call("rbi_2d_add_i32", ["i32_2d"], d, i, j, v)
        assert out.values().tolist() == c["out"]
        for h in (out, d, i, j, v):
            h.free()
    rng = np.random.default_rng(4)
    for t, op, H0, H1, n in [("i32", "add", 10, 10, 5000), ("i64", "max", 300, 7, 100003),
                             ("i32", "or", 1000, 1000, 200000), ("f64", "max", 3, 50000, 99999),
                             ("i32", "add", 3000, 3000, 1 << 20), ("i32", "add", 0, 5, 100)]:
        dt = {"i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        is_ = rng.integers(-2, H0 + 2, n).astype(np.int64)
        js = rng.integers(-2, H1 + 2, n).astype(np.int64)
        vs = (rng.standard_normal(n) if t == "f64" else rng.integers(-1000, 1000, n)).astype(dt)
        dest = (rng.standard_normal((H0, H1)) if t == "f64" else rng.integers(-5, 5, (H0, H1))).astype(dt)
        d, i, j, v = (ctx.new(f"{t}_2d", dest), ctx.new("i64_1d", is_), ctx.new("i64_1d", js),
                      ctx.new(f"{t}_1d", vs))
        out = ctx.call(f"rbi_2d_{op}_{t}", [f"{t}_2d"], d, i, j, v)
        assert np.array_equal(out.values(), oracle.rbi_2d(op, t, dest, is_, js, vs)), (t, op, H0, H1, n)
        for h in (out, d, i, j, v):
            h.free()
    # the sparse 2-D histogram of tests/hist/large2d.fut, 100 x 100 bins, k = 10^6: closed form modulo 2^32
    n_, m_, k = 100, 100, 1000000
    it = np.arange(k, dtype=np.int64)
    d = ctx.new("i32_2d", np.zeros((m_, n_), np.int32))
    i, j, v = ctx.new("i64_1d", it % n_), ctx.new("i64_1d", it % m_), ctx.new("i32_1d", it.astype(np.int32))
    out = ctx.call("rbi_2d_add_i32", ["i32_2d"], d, i, j, v)
    assert int(out.values().sum(dtype=np.int64)) % 2**32 == (k * (k - 1) // 2) % 2**32  # bins wrap
    for h in (out, d, i, j, v):
        h.free()


@pytest.mark.parametrize("t,op", [("i32", "add"), ("i64", "max"), ("f32", "add"), ("f32", "max"), ("f64", "min")])
def test_i64_indices_small_and_ragged(ctx, t, op):
    """hist_OP_T_i64 / rbi_OP_T_i64: the []i64 indices `hist` and `reduce_by_index` are defined
    over (prelude/soacs.fut:132-146), with indices far outside the bins that a 32-bit view would
    fold back into range (2^32 + 3 must be ignored, not counted in bin 3)."""
    for n, H in [(0, 5), (5, 0), (100, 7), (4097, 256), (300001, 32769), (150000, 100001),
                 (100000, 200000), (400000, 2_000_000)]:
        is_ = dg.hist_indices(40, n, max(H, 1), "uniform", 3).astype(np.int64)
        if n > 50:
            is_[::17] += np.int64(1) << 32          # out of range only as 64-bit numbers
            is_[5::29] = -(np.int64(1) << 40) + 2
        vs = _vals(t, n, 41)
        i, v = ctx.new("i64_1d", is_), ctx.new(f"{t}_1d", vs)
        ok = (is_ >= 0) & (is_ < H)
        narrow = np.where(ok, is_, -1).astype(np.int32)   # the oracle takes 32-bit indices
        out = ctx.call(f"hist_{op}_{t}_i64", [f"{t}_1d"], H, i, v)
        got = out.values()
        assert got.shape == (H,)
        acc = oracle.hist(op, t, H, narrow, vs, "f64acc") if (op, t) == ("add", "f32") else None
        _check(t, op, got, oracle.hist(op, t, H, narrow, vs), acc)
        out.free()
        dest = _vals(t, H, 43)
        d = ctx.new(f"{t}_1d", dest)
        out = ctx.call(f"rbi_{op}_{t}_i64", [f"{t}_1d"], d, i, v)
        acc = oracle.rbi(op, t, dest, narrow, vs, "f64acc") if (op, t) == ("add", "f32") else None
        _check(t, op, out.values(), oracle.rbi(op, t, dest, narrow, vs), acc)
        for h in (i, v, d, out):
            h.free()


@pytest.mark.parametrize("H", [65536, 1 << 22])
def test_config3_full_size_i64_indices(ctx, H):
    """The i32 (+) histogram of the configuration at 2^27 with its indices widened to i64."""
    n = 1 << 27
    is32 = dg.hist_indices(48, n, H, "uniform")
    vs = dg.uniform_int(49, n, -1000, 1000)
    i, v = ctx.new("i64_1d", is32.astype(np.int64)), ctx.new("i32_1d", vs)
    out = ctx.call("hist_add_i32_i64", ["i32_1d"], H, i, v)
    got = out.values()
    assert np.array_equal(got, oracle.hist("add", "i32", H, is32, vs))
    for h in (i, v, out):
        h.free()
