"""Pins the CPU oracle: reference-held golden vectors, closed forms and library
routines.  Each check is chosen so that a plausible slip in the oracle (wrong
neutral element, dropped wrap-around, off-by-one exclusive scan, unstable sort,
transposed operand) fails it."""
import math
import numpy as np
import pytest

import oracle


def _f(xs):
    return np.array([np.nan if x == "nan" else x for x in xs], dtype=np.float32)


def test_reduce0_iota_wraps(goldens):
    for c in goldens["reduce0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        assert int(oracle.reduce("add", "i32", xs)) == c["out"]


def test_scan0_and_exscan0(goldens):
    for c in goldens["scan0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        assert int(oracle.scan("add", "i32", xs)[-1]) == c["out"]
    for c in goldens["exscan0"]["cases"]:
        xs = np.arange(c["n"], dtype=np.int64).astype(np.int32)
        assert int(oracle.scan("add", "i32", xs, exclusive=True)[-1]) == c["out"]


def test_scan4_radix_distilled(goldens):
    for c in goldens["scan4"]["cases"]:
        xs = np.array(c["in"], dtype=np.int32)
        for _ in range(2):
            bits = xs + 1
            ps = oracle.scan("add", "i32", bits)
            s = oracle.reduce("add", "i32", bits)
            xs = ps + s + xs
        assert xs.tolist() == c["out"]


def test_hist_simple_large_max_min(goldens):
    for c in goldens["hist_simple"]["cases"]:
        img = np.array(c["image"], dtype=np.int32)
        out = oracle.rbi("add", "i32", np.array(c["dest"], dtype=np.int32), img, img)
        assert out.tolist() == c["out"]
    for c in goldens["hist_large"]["cases"][:2] + goldens["hist_large"]["cases"][2:]:
        n, m = c["n"], c["m"]
        i = np.arange(m, dtype=np.int64)
        h = oracle.hist("add", "i32", n, (i % n).astype(np.int32), i.astype(np.int32))
        assert int(oracle.reduce("add", "i32", h)) == c["out"]
    for name, op in (("hist_max", "max"), ("hist_min", "min")):
        for c in goldens[name]["cases"]:
            out = oracle.rbi(op, "i32", np.zeros(c["n"], np.int32), c["is"], c["vs"])
            assert out.tolist() == c["out"]


def test_hist_bitwise_operators(goldens):
    # tests/hist/{and,or,xor,and64,xor64}.fut: neutral elements -1, 0, 0
    for name in ("hist_and", "hist_or", "hist_xor", "hist_and64", "hist_xor64"):
        op = name[5:].rstrip("64")
        t = goldens[name]["type"]
        for c in goldens[name]["cases"]:
            out = oracle.hist(op, t, c["n"], c["is"], c["vs"])
            assert out.tolist() == c["out"], (name, c)


NARROW = {"i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16,
          "u32": np.uint32, "u64": np.uint64}


def test_hist_small_integer_types_goldens(goldens):
    # tests/hist/{i8,i16,and8,and16,or8,or16,xor8,xor16,max8,max16,min8,min16}.fut and the
    # unsigned results of max.fut / min.fut
    for bits in (8, 16):
        t, u = f"i{bits}", f"u{bits}"
        for c in goldens[f"hist_add_{t}"]["cases"]:
            assert oracle.rbi("add", t, c["dest"], c["is"], c["vs"]).tolist() == c["out"]
        for op in ("and", "or", "xor"):
            for c in goldens[f"hist_{op}{bits}"]["cases"]:
                assert oracle.hist(op, t, c["n"], c["is"], c["vs"]).tolist() == c["out"], (op, bits, c)
        for op in ("max", "min"):
            for c in goldens[f"hist_{op}{bits}"]["cases"]:
                vs = np.array(c["vs"], NARROW[t])
                zeros = np.zeros(c["n"], NARROW[t])
                assert oracle.rbi(op, t, zeros, c["is"], vs).tolist() == c["out"]
                got = oracle.rbi(op, u, zeros.view(NARROW[u]), c["is"], vs.view(NARROW[u]))
                assert got.view(NARROW[t]).tolist() == c["out_unsigned"], (op, bits, c)
    for op in ("max", "min"):
        for c in goldens[f"hist_{op}_u32"]["cases"]:
            vs = np.array(c["vs"], np.int32).view(np.uint32)
            got = oracle.rbi(op, "u32", np.zeros(c["n"], np.uint32), c["is"], vs)
            assert got.view(np.int32).tolist() == c["out"]


def test_hist_small_integer_types_against_numpy():
    rng = np.random.default_rng(21)
    ufuncs = {"add": np.add, "max": np.maximum, "min": np.minimum, "and": np.bitwise_and,
              "or": np.bitwise_or, "xor": np.bitwise_xor}
    for t, dt in NARROW.items():
        ii = np.iinfo(dt)
        vs = rng.integers(ii.min, ii.max, 5000, dtype=dt, endpoint=True)
        is_ = rng.integers(-3, 40, 5000).astype(np.int32)
        ok = (is_ >= 0) & (is_ < 37)
        for op, uf in ufuncs.items():
            dest = rng.integers(ii.min, ii.max, 37, dtype=dt, endpoint=True)
            want = dest.copy()
            uf.at(want, is_[ok], vs[ok])  # wraps in the element type
            assert np.array_equal(oracle.rbi(op, t, dest, is_, vs), want), (t, op)
            ne = oracle.hist(op, t, 3, np.zeros(0, np.int32), np.zeros(0, dt))
            assert np.all(uf(ne, vs[:3]) == vs[:3]), (t, op)  # the neutral element is neutral


def test_f16_rounding_and_histograms(goldens):
    # f32 -> f16 is round-to-nearest-even: numpy's conversion is the check
    rng = np.random.default_rng(3)
    f = np.concatenate([
        rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        (rng.standard_normal(200000) * 10 ** rng.uniform(-9, 6, 200000)).astype(np.float32),
        np.array([65504, 65519.99, 65520, 2**-24, 2**-25, 2**-25 * 1.0001, 2**-14, 0.0, -0.0,
                  np.inf, -np.inf], np.float32)])
    with np.errstate(all="ignore"):
        want = f.astype(np.float16)
    got = oracle.narrow_f16(f)
    keep = ~np.isnan(f)
    assert np.array_equal(got.view(np.uint16)[keep], want.view(np.uint16)[keep])
    assert np.all(np.isnan(got[~keep]))
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    back = oracle.narrow_f16(oracle.widen(halves.view(np.uint16), "f16"))
    assert np.array_equal(back.view(np.uint16)[~np.isnan(halves)], halves.view(np.uint16)[~np.isnan(halves)])
    # tests/hist/f16.fut and f64.fut
    for c in goldens["hist_f16"]["cases"]:
        for variant in ("lit", "f64acc"):
            out = oracle.rbi("add", "f16", _f(c["dest"]).astype(np.float16), c["is"],
                             _f(c["vs"]).astype(np.float16), variant)
            np.testing.assert_allclose(out.astype(np.float32), _f(c["out"]), rtol=2e-3, equal_nan=True)
    for c in goldens["hist_f64"]["cases"]:
        out = oracle.rbi("add", "f64", _f(c["dest"]).astype(np.float64), c["is"], _f(c["vs"]).astype(np.float64))
        np.testing.assert_allclose(out, _f(c["out"]).astype(np.float64), rtol=1e-6, equal_nan=True)
    # small integers: every partial sum is an f16 value, so all three agree exactly
    vs = rng.integers(0, 4, 3000).astype(np.float16)
    is_ = rng.integers(-2, 9, 3000).astype(np.int32)
    want = np.zeros(8, np.float64)
    ok = (is_ >= 0) & (is_ < 8)
    np.add.at(want, is_[ok], vs[ok].astype(np.float64))
    for variant in ("lit", "f64acc"):
        assert np.array_equal(oracle.hist("add", "f16", 8, is_, vs, variant).astype(np.float64), want)
    # max / min ignore NaN operands like fmaxf / fminf
    vs = np.array([1.5, np.nan, -2, 7, np.nan], np.float16)
    assert oracle.hist("max", "f16", 2, [0, 0, 0, 1, 1], vs).tolist() == [1.5, 7.0]
    assert oracle.hist("min", "f16", 2, [0, 0, 0, 1, 1], vs).tolist() == [-2.0, 7.0]


def test_bitwise_reductions_and_scans_match_numpy():
    rng = np.random.default_rng(9)
    for t, dt in (("i32", np.int32), ("i64", np.int64)):
        xs = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, 1000, dtype=dt)
        for op, uf in (("and", np.bitwise_and), ("or", np.bitwise_or), ("xor", np.bitwise_xor)):
            assert oracle.reduce(op, t, xs) == uf.reduce(xs)
            assert np.array_equal(oracle.scan(op, t, xs), uf.accumulate(xs))
        assert oracle.reduce("and", t, xs[:0]) == -1 and oracle.reduce("xor", t, xs[:0]) == 0


def test_hist_f32_including_nan(goldens):
    for c in goldens["hist_f32"]["cases"]:
        for variant in ("lit", "f64acc"):
            out = oracle.rbi("add", "f32", _f(c["dest"]), c["is"], _f(c["vs"]), variant)
            np.testing.assert_allclose(out, _f(c["out"]), rtol=2e-3, equal_nan=True)


def test_hist_segmented(goldens):
    c = goldens["hist_segmented"]["cases"][0]
    for xs, want in zip(c["xss"], c["out"]):
        got = oracle.hist("add", "i32", c["m"], xs, np.ones(len(xs), np.int32))
        assert got.tolist() == want


def test_segsum_and_segreduce_iota(goldens):
    c = goldens["segsum"]["cases"][0]
    assert oracle.segreduce("add", "f32", c["xss"]).tolist() == c["out"]
    for c in goldens["segreduce_iota"]["cases"]:
        n, m = c["n"], c["m"]
        xss = np.repeat(np.arange(n, dtype=np.int32)[:, None], m, axis=1).reshape(n, m)
        assert oracle.segreduce("add", "i32", xss).tolist() == c["out"]


def test_irregular_segments_with_empty_segment(goldens):
    c = goldens["nonuniform_2d"]["cases"][0]
    sizes = np.array(c["sizes"], dtype=np.int64)
    lens = 3 * sizes
    offsets = np.concatenate(([0], np.cumsum(lens)[:-1]))
    vals = np.concatenate([(np.arange(3)[:, None] + np.arange(s)[None, :]).ravel() for s in sizes])
    out = oracle.segred("add", "i64", offsets, lens, vals.astype(np.int64))
    assert out.tolist() == c["out"]


def test_segscan_operator_against_per_segment_cumsum():
    rng = np.random.default_rng(1)
    n = 5000
    flags = (rng.random(n) < 0.01).astype(np.uint8)
    xs = rng.integers(-1000, 1000, n).astype(np.int64)
    got = oracle.segscan("add", "i64", flags, xs)
    want = np.empty_like(xs)
    starts = [0] + [i for i in range(1, n) if flags[i]] + [n]
    for a, b in zip(starts[:-1], starts[1:]):
        want[a:b] = np.cumsum(xs[a:b])
    assert np.array_equal(got, want)
    # max restarts too, and flags[0] == 0 folds the neutral element in front
    gm = oracle.segscan("max", "f32", flags, xs.astype(np.float32))
    wm = np.empty(n, np.float32)
    for a, b in zip(starts[:-1], starts[1:]):
        wm[a:b] = np.maximum.accumulate(xs[a:b].astype(np.float32))
    assert np.array_equal(gm, wm)


def test_mmm_golden_and_numpy(goldens):
    c = goldens["mmm"]["cases"][0]
    for variant in ("lit", "f64acc"):
        assert oracle.bmm_f32(c["A"], c["B"], variant).tolist() == c["out"]
    rng = np.random.default_rng(2)
    A = rng.standard_normal((3, 17, 29)).astype(np.float32)
    B = rng.standard_normal((3, 29, 13)).astype(np.float32)
    want = np.matmul(A.astype(np.float64), B.astype(np.float64))
    np.testing.assert_allclose(oracle.bmm_f32(A, B, "f64acc"), want, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.bmm_f32(A, B, "lit"), want, rtol=1e-4, atol=1e-4)


def test_f16_bf16_widening_is_exact():
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.widen(bits, "f16")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    gb = oracle.widen(bits, "bf16")
    assert np.array_equal(gb.view(np.uint32), bits.astype(np.uint32) << 16)
    # tests/f16kernel.fut: [1,2,3]f16 sums to 6
    assert float(oracle.widen(np.array([1, 2, 3], np.float16).view(np.uint16), "f16").sum()) == 6.0


def test_radix_sort_is_stable_and_matches_numpy(goldens):
    c = goldens["radixsort"]["cases"][0]
    keys = np.array(c["keys"], np.float32).view(np.uint32)  # positive floats order as u32
    vals = np.array(c["vals"], np.float32)
    ko, vo = oracle.radix_sort(keys, vals.view(np.uint32))
    assert vo.view(np.float32).tolist() == np.array(c["out_vals"], np.float32).tolist()
    rng = np.random.default_rng(3)
    for dt in (np.uint32, np.uint64):
        keys = rng.integers(0, 50, 20000).astype(dt) << dt(20 if dt == np.uint32 else 40)
        idx = np.arange(keys.size, dtype=np.int32)
        ko, vo = oracle.radix_sort(keys, idx)
        perm = np.argsort(keys, kind="stable")
        assert np.array_equal(ko, keys[perm]) and np.array_equal(vo, idx[perm])
        full = rng.integers(0, np.iinfo(dt).max, 10000, dtype=dt)
        assert np.array_equal(oracle.radix_sort(full), np.sort(full))


def test_f64acc_variants_are_close_to_exact_and_lit_drifts():
    rng = np.random.default_rng(4)
    xs = rng.random(1 << 20).astype(np.float32)
    exact = xs.astype(np.float64).cumsum()
    got = oracle.scan("add", "f32", xs, "f64acc")
    np.testing.assert_allclose(got, exact, rtol=1e-7)
    lit = oracle.scan("add", "f32", xs, "lit")
    assert np.array_equal(lit, np.cumsum(xs, dtype=np.float32))  # same left fold
    ex = oracle.scan("add", "f32", xs, "f64acc", exclusive=True)
    assert ex[0] == 0.0 and np.array_equal(ex[1:], got[:-1])


def test_f64acc_reduce_segscan_segred_against_numpy_in_double():
    """The f64-accumulated yardsticks of reduce, segmented scan and segmented
    reduce are sums in double rounded once to f32: numpy's double sums and
    cumulative sums over each segment say the same, bit for bit."""
    rng = np.random.default_rng(14)
    n = 200_003
    xs = rng.random(n).astype(np.float32)
    x64 = xs.astype(np.float64)
    # reduce: one sum in double (math.fsum is the exact sum; both round to the same f32 here)
    got = oracle.reduce("add", "f32", xs, "f64acc")
    assert got == np.float32(np.add.reduce(x64))
    assert abs(float(got) - math.fsum(x64.tolist())) <= 2.0 ** -24 * float(got)
    assert oracle.reduce("add", "f32", xs[:0], "f64acc") == 0.0
    assert oracle.reduce("add", "f32", xs[:1], "f64acc") == xs[0]
    # A dropped element, a sum in f32 or a sum of squares would all fail this.
    assert got != np.float32(np.add.reduce(x64[:-1]))

    # segmented scan: restart at every flag; flags[0] == 0 (the neutral element
    # is folded in front, which changes nothing) and a start on the last element.
    flags = (rng.random(n) < 1 / 700).astype(np.uint8)
    flags[0] = 0
    flags[n - 1] = 1
    flags[1000:1003] = 1  # segments of one element
    starts = np.flatnonzero(flags).tolist()
    bounds = [0] + [s for s in starts if s != 0] + [n]
    want = np.empty(n, np.float32)
    for a, b in zip(bounds[:-1], bounds[1:]):
        want[a:b] = np.cumsum(x64[a:b]).astype(np.float32)
    got = oracle.segscan("add", "f32", flags, xs, "f64acc")
    assert np.array_equal(got, want)
    assert got[n - 1] == xs[n - 1] and got[1001] == xs[1001]
    # no flags at all: the plain scan in double
    assert np.array_equal(oracle.segscan("add", "f32", np.zeros(n, np.uint8), xs, "f64acc"),
                          np.cumsum(x64).astype(np.float32))

    # segmented reduce over (offset, length) pairs: an empty segment gives the
    # neutral element, and elements in a gap between segments belong to nobody.
    lens = np.array([5, 0, 1, 70_000, 0, 3, 100_000], np.int64)
    offsets = np.array([0, 5, 5, 6, 70_006, 70_100, 70_103], np.int64)  # gap: [70006, 70100)
    assert offsets[-1] + lens[-1] <= n
    want = np.array([np.add.reduce(x64[o:o + l]) for o, l in zip(offsets, lens)]).astype(np.float32)
    got = oracle.segred("add", "f32", offsets, lens, xs, "f64acc")
    assert np.array_equal(got, want)
    assert got[1] == 0.0 and got[4] == 0.0 and got[2] == xs[5]
    # segments that tile the array: the reduction of a segment is the scanned
    # value at its last element (Builtins.hs:582-602)
    ends = np.array(bounds[1:], np.int64)
    begs = np.array(bounds[:-1], np.int64)
    tiled = oracle.segred("add", "f32", begs, ends - begs, xs, "f64acc")
    assert np.array_equal(tiled, oracle.segscan("add", "f32", flags, xs, "f64acc")[ends - 1])


def test_transpose():
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(oracle.transpose_f32(x), x.T)


def test_multicore_baseline_agrees_with_oracle():
    rng = np.random.default_rng(5)
    n = 300000
    xs = rng.integers(-1000, 1000, n).astype(np.int32)
    flags = (rng.random(n) < 0.001).astype(np.uint8)
    assert oracle.mc_reduce_add("i32", xs, 4) == oracle.reduce("add", "i32", xs)
    assert np.array_equal(oracle.mc_segscan("i32", None, xs, "add", 4), oracle.scan("add", "i32", xs))
    assert np.array_equal(oracle.mc_segscan("i32", flags, xs, "add", 4),
                          oracle.segscan("add", "i32", flags, xs))
    assert np.array_equal(oracle.mc_segscan("i32", flags, xs, "max", 3),
                          oracle.segscan("max", "i32", flags, xs))
    is_ = rng.integers(-5, 300, n).astype(np.int32)
    assert np.array_equal(oracle.mc_rbi_add_i32(np.zeros(256, np.int32), is_, xs, 4),
                          oracle.rbi("add", "i32", np.zeros(256, np.int32), is_, xs))
    big = oracle.mc_rbi_add_i32(np.zeros(200000, np.int32), is_, xs, 4)  # atomic path
    assert np.array_equal(big, oracle.rbi("add", "i32", np.zeros(200000, np.int32), is_, xs))
    # f32 histograms: max is order-independent (bit-exact); sums differ from the sequential
    # fold only in the order of the additions
    ws = rng.random(n).astype(np.float32)
    dest = rng.random(300).astype(np.float32)
    assert np.array_equal(oracle.mc_rbi_f32("max", dest, is_, ws, 5), oracle.rbi("max", "f32", dest, is_, ws))
    np.testing.assert_allclose(oracle.mc_rbi_f32("add", dest, is_, ws, 5),
                               oracle.rbi("add", "f32", dest, is_, ws, "f64acc"), rtol=1e-5)
    # irregular segmented reduce: scan with flags from the offsets, then a gather
    lens = np.array([5, 0, 1, 70_000, 0, 3, 100_000], np.int64)
    offsets = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int64)
    np.testing.assert_allclose(oracle.mc_segred_add_f32(offsets, lens, ws[: lens.sum()], 3),
                               oracle.segred("add", "f32", offsets, lens, ws[: lens.sum()], "f64acc"),
                               rtol=1e-5)
    # matmul: the same sequential dot product per output as the oracle's literal fold
    A = rng.standard_normal((3, 17, 29)).astype(np.float32)
    B = rng.standard_normal((3, 29, 13)).astype(np.float32)
    Bt = oracle.mc_transpose_f32(B, 3)
    assert np.array_equal(Bt, B.transpose(0, 2, 1))
    Cm = np.full((3, 17, 13), np.nan, np.float32)
    oracle.mc_bmm_rows_f32(A, Bt, Cm, 0, 20, 4)     # a range of rows that crosses a batch boundary
    oracle.mc_bmm_rows_f32(A, Bt, Cm, 20, 51, 4)
    assert np.array_equal(Cm, oracle.bmm_f32(A, B, "lit"))
    # 16-bit inputs: widened where they are used, so the result is the f32 matmul of the widened
    # matrices, bit for bit
    from futhark_amd import datagen as dg
    for kind, bits in (("f16", dg.to_f16_bits), ("bf16", dg.to_bf16_bits)):
        A16, B16 = bits(A), bits(B)
        Bt16 = oracle.mc_transpose_16(B16, 3)
        assert np.array_equal(Bt16, B16.transpose(0, 2, 1))
        Cm = np.full((3, 17, 13), np.nan, np.float32)
        oracle.mc_bmm_rows_16(A16, Bt16, Cm, 0, 30, kind == "bf16", 4)
        oracle.mc_bmm_rows_16(A16, Bt16, Cm, 30, 51, kind == "bf16", 2)
        assert np.array_equal(Cm, oracle.bmm_f32(oracle.widen(A16, kind), oracle.widen(B16, kind), "lit")), kind
    # radix sort: stable, keys and (key, value) pairs, against the sequential oracle
    for dt in (np.uint32, np.uint64):
        keys = rng.integers(0, np.iinfo(dt).max, 50_000, dtype=dt)
        keys[::7] = keys[3]  # ties
        idx = np.arange(keys.size, dtype=np.int32)
        assert np.array_equal(oracle.mc_radix_sort(keys, None, 3), oracle.radix_sort(keys))
        ko, vo = oracle.mc_radix_sort(keys, idx, 5)
        kr, vr = oracle.radix_sort(keys, idx)
        assert np.array_equal(ko, kr) and np.array_equal(vo, vr)


def test_vectorised_reduce_is_a_reduce_per_column():
    """reduce (map2 op) ne xss folds every column on its own: the same as the regular segmented
    reduce of the transposed array, and numpy's wrapping integer reductions along axis 0."""
    rng = np.random.default_rng(5)
    for n, k in [(0, 3), (1, 5), (17, 4), (100, 33)]:
        xi = rng.integers(-2**31, 2**31, (n, k), dtype=np.int64).astype(np.int32)
        for op, f in (("add", np.add), ("max", np.maximum), ("min", np.minimum)):
            got = oracle.vecreduce(op, "i32", xi)
            assert np.array_equal(got, oracle.segreduce(op, "i32", np.ascontiguousarray(xi.T)))
            if n > 0:
                assert np.array_equal(got, f.reduce(xi, axis=0, dtype=np.int32))
        xf = rng.standard_normal((n, k)).astype(np.float32)
        assert np.array_equal(oracle.vecreduce("add", "f32", xf),
                              oracle.segreduce("add", "f32", np.ascontiguousarray(xf.T)))
        np.testing.assert_allclose(oracle.vecreduce("add", "f32", xf, "f64acc"),
                                   xf.astype(np.float64).sum(axis=0), rtol=1e-6, atol=1e-6)


def test_hist_with_vector_operator_and_2d_indices_goldens(goldens):
    # tests/hist/{array,array_novec,equiv,hist2d}.fut; tests/hist/lor.fut with bool as a byte
    for name in ("hist_array", "hist_equiv"):
        for c in goldens[name]["cases"]:
            assert oracle.rbi_vec("add", "i32", c["dest"], c["is"], c["vss"]).tolist() == c["out"]
    for c in goldens["hist2d"]["cases"]:
        assert oracle.rbi_2d("add", "i32", c["dest"], c["is"], c["js"], c["vs"]).tolist() == c["out"]
    for c in goldens["hist_lor"]["cases"]:
        assert oracle.hist("or", "u8", c["n"], c["is"], c["vs"]).tolist() == c["out"]


def test_shaped_hist_against_numpy():
    """The vector form is a plain histogram over bins b * m + c, the 2-D form one over
    i * H1 + j with updates dropped when either coordinate is outside (numpy's unbuffered
    ufunc.at does the in-order read-modify-write)."""
    rng = np.random.default_rng(11)
    H, m, n = 7, 5, 400
    is_ = rng.integers(-2, H + 2, n)
    vss = rng.integers(-2**31, 2**31, (n, m), dtype=np.int64).astype(np.int32)
    dest = rng.integers(-100, 100, (H, m)).astype(np.int32)
    ok = (is_ >= 0) & (is_ < H)
    for op, f in (("add", np.add), ("max", np.maximum), ("min", np.minimum), ("xor", np.bitwise_xor)):
        want = dest.copy()
        f.at(want, is_[ok], vss[ok])
        assert np.array_equal(oracle.rbi_vec(op, "i32", dest, is_, vss), want)
    H0, H1 = 6, 9
    is_, js = rng.integers(-1, H0 + 1, n), rng.integers(-1, H1 + 1, n)
    vs = rng.standard_normal(n)
    dest = rng.standard_normal((H0, H1))
    ok = (is_ >= 0) & (is_ < H0) & (js >= 0) & (js < H1)
    want = dest.copy()
    np.add.at(want, (is_[ok], js[ok]), vs[ok])
    assert np.array_equal(oracle.rbi_2d("add", "f64", dest, is_, js, vs), want)


def test_affine_composition_scan_is_the_iterated_map():
    """Element i of the scan, applied to x, must give what applying the maps 0..i one after the
    other gives (modulo 2^32); the segmented form restarts at flags; the operator does not commute."""
    rng = np.random.default_rng(8)
    n = 300
    abs_ = rng.integers(-2**31, 2**31, (n, 2), dtype=np.int64).astype(np.int32)
    flags = (rng.random(n) < 0.1).astype(np.uint8)
    M = 1 << 32
    for fl in (None, flags):
        inc = oracle.scan_compose_i32(abs_, fl).astype(np.int64)
        exc = oracle.scan_compose_i32(abs_, fl, exclusive=True).astype(np.int64)
        for x0 in (0, 1, 12345):
            x = x0
            for i in range(n):
                if fl is not None and fl[i]:
                    x = x0
                assert (exc[i, 0] * x0 + exc[i, 1]) % M == x % M if fl is None or not fl[i] else True
                x = (int(abs_[i, 0]) * x + int(abs_[i, 1])) % M
                assert (inc[i, 0] * x0 + inc[i, 1]) % M == x
    two = np.array([[2, 3], [5, 7]], np.int32)
    assert oracle.scan_compose_i32(two)[1].tolist() == [10, 22]          # 5 * (2x + 3) + 7
    assert oracle.scan_compose_i32(two[::-1])[1].tolist() == [10, 17]    # 2 * (5x + 7) + 3


def test_tuple_operator_oracles_are_pinned_by_closed_forms():
    """argmax on (value, index) pairs and the fused maps: each against what numpy fixes.
    reduce argmax (zip xs iota) is numpy's argmax (first of equal maxima); the running one
    is maximum.accumulate with the position of its first occurrence; per bin, the maximum
    of the bin's values and the first position holding it."""
    rng = np.random.default_rng(5)
    for n in (1, 2, 17, 1000, 4099):
        xs = rng.integers(-50, 50, n).astype(np.int32)      # many ties
        assert oracle.reduce_argmax_i32(xs).tolist() == [int(xs.max()), int(np.argmax(xs))]
        vis = np.stack([xs, np.arange(n, dtype=np.int32)], axis=1)
        sc = oracle.scan_argmax_i32(vis)
        run = np.maximum.accumulate(xs)
        assert np.array_equal(sc[:, 0], run)
        first = np.array([int(np.argmax(xs[:i + 1])) for i in range(n)]) if n <= 1000 else None
        if first is not None:
            assert np.array_equal(sc[:, 1], first)
        ex = oracle.scan_argmax_i32(vis, exclusive=True)
        assert ex[0].tolist() == [np.iinfo(np.int32).min, np.iinfo(np.int32).max]
        assert np.array_equal(ex[1:], sc[:-1])
        flags = (rng.integers(0, 7, n) == 0).astype(np.uint8)
        seg = oracle.scan_argmax_i32(vis, flags)
        starts = np.flatnonzero(flags).tolist()
        bounds = sorted(set([0] + starts + [n]))
        for a, b in zip(bounds[:-1], bounds[1:]):
            assert np.array_equal(seg[a:b], oracle.scan_argmax_i32(vis[a:b]))
        H = 13
        is_ = rng.integers(-2, H + 2, n).astype(np.int32)
        h = oracle.hist_argmax_i32(H, is_, xs)
        for b in range(H):
            sel = np.flatnonzero(is_ == b)
            want = [np.iinfo(np.int32).min, np.iinfo(np.int32).max] if sel.size == 0 else \
                [int(xs[sel].max()), int(sel[np.argmax(xs[sel])])]
            assert h[b].tolist() == want
    assert oracle.reduce_argmax_i32(np.zeros(0, np.int32)).tolist() == [-2 ** 31, 2 ** 31 - 1]
    # the fold of affine maps applied to a probe value is the maps applied one after the other
    abs_ = rng.integers(-9, 9, (200, 2)).astype(np.int32)
    a, b = (int(v) for v in oracle.reduce_compose_i32(abs_))
    x = 12345
    for fa, fb in abs_.tolist():
        x = (fa * x + fb) % (1 << 32)
    assert (a * 12345 + b) % (1 << 32) == x
    assert oracle.reduce_compose_i32(np.zeros((0, 2), np.int32)).tolist() == [1, 0]
    # sums of squares and running norms against float64 numpy
    xs = rng.standard_normal(5000).astype(np.float32)
    assert abs(float(oracle.sumsq_f32(xs, "f64acc")) - float(np.dot(xs.astype(np.float64), xs.astype(np.float64)))) \
        <= 1e-6 * float(np.dot(xs.astype(np.float64), xs.astype(np.float64)))
    want = np.sqrt(np.cumsum(xs.astype(np.float64) ** 2))
    assert np.all(np.abs(oracle.scan_norm_f32(xs, "f64acc") - want) <= 1e-6 * want)


def test_vector_operator_scan_oracle_is_pinned():
    """vecscan is the scalar scan (pinned by the reference's scan0/exscan0/scan4 vectors above)
    applied per column.  What could go wrong is the axis: a shape that is not square, rows that
    are all alike (closed form (i+1)(j+1)), numpy's own cumulative sum down the rows, and the
    last row against the reduction with the same operator."""
    n, k = 5, 3
    xss = np.tile(np.arange(1, k + 1, dtype=np.int32), (n, 1))
    got = oracle.vecscan("add", "i32", xss)
    assert got.shape == (n, k)
    assert got.tolist() == [[(i + 1) * (j + 1) for j in range(k)] for i in range(n)]
    rng = np.random.default_rng(5)
    yss = rng.integers(-1000, 1000, (37, 11)).astype(np.int64)
    assert np.array_equal(oracle.vecscan("add", "i64", yss), np.cumsum(yss, axis=0))
    assert np.array_equal(oracle.vecscan("max", "i64", yss), np.maximum.accumulate(yss, axis=0))
    assert np.array_equal(oracle.vecscan("add", "i64", yss)[-1], oracle.vecreduce("add", "i64", yss))
    assert oracle.vecscan("add", "i32", np.zeros((0, 4), np.int32)).shape == (0, 4)
    assert oracle.vecscan("add", "i32", np.zeros((4, 0), np.int32)).shape == (4, 0)


def test_rows_fraction_oracle_is_pinned():
    """Closed forms: a row of ones gives (i+1)/k; the last column is 1; rows do not mix
    (a transposed loop would); scaling a row by a power of two changes nothing."""
    k = 8
    ones = np.ones((3, k), np.float32)
    got = oracle.rows_fraction_f32(ones)
    assert np.array_equal(got, np.tile((np.arange(1, k + 1) / k).astype(np.float32), (3, 1)))
    rng = np.random.default_rng(9)
    xss = (rng.random((4, 37)) + 0.5).astype(np.float32)
    got = oracle.rows_fraction_f32(xss, "f64acc")
    want = np.cumsum(xss.astype(np.float64), axis=1) / xss.astype(np.float64).sum(axis=1)[:, None]
    assert np.all(np.abs(got - want) <= 1e-6)
    assert np.all(np.abs(got[:, -1] - 1) <= 1e-6)
    assert np.array_equal(oracle.rows_fraction_f32(xss * np.float32(4)), oracle.rows_fraction_f32(xss))
    one_row = oracle.rows_fraction_f32(xss[2:3])
    assert np.array_equal(one_row[0], oracle.rows_fraction_f32(xss)[2])


def test_two_operator_reduction_oracle_is_pinned():
    xs = np.array([1.5, -2.0, 8.25, 0.5], np.float32)
    assert oracle.reduce_summax_f32(xs).tolist() == [8.25, 8.25]
    assert oracle.reduce_summax_f32(xs[:2]).tolist() == [-0.5, 1.5]
    e = oracle.reduce_summax_f32(np.zeros(0, np.float32))
    assert e[0] == 0 and np.isneginf(e[1])


def test_custom_operators_in_the_segmented_forms():
    """segreduce_argmax_i32, segreduce_compose_i32, scanrows_argmax_i32 and segred_argmax_i32
    against brute force in plain Python (ties go to the smaller index; maps are applied one
    after the other to a probe value) and against the unsegmented functions pinned above."""
    rng = np.random.default_rng(33)
    lo, hi = -2 ** 31, 2 ** 31 - 1
    xss = rng.integers(-5, 5, (23, 17)).astype(np.int32)   # many ties
    got = oracle.segreduce_argmax_i32(xss)
    for r in range(23):
        best = max(range(17), key=lambda j: (int(xss[r, j]), -j))
        assert got[r].tolist() == [int(xss[r, best]), best]
        assert got[r].tolist() == oracle.reduce_argmax_i32(xss[r]).tolist()
    assert oracle.segreduce_argmax_i32(np.zeros((3, 0), np.int32)).tolist() == [[lo, hi]] * 3
    assert oracle.segreduce_argmax_i32(np.zeros((0, 4), np.int32)).shape == (0, 2)

    k = 9
    abs_ = rng.integers(-9, 9, (7 * k, 2)).astype(np.int32)
    got = oracle.segreduce_compose_i32(k, abs_)
    assert got.shape == (7, 2)
    for r in range(7):
        x = 4321
        for fa, fb in abs_[r * k:(r + 1) * k].tolist():
            x = (fa * x + fb) % (1 << 32)
        a, b = (int(v) for v in got[r])
        assert (a * 4321 + b) % (1 << 32) == x
        assert got[r].tolist() == oracle.reduce_compose_i32(abs_[r * k:(r + 1) * k]).tolist()

    vis = np.stack([rng.integers(-4, 4, 6 * k), np.arange(6 * k)], axis=1).astype(np.int32)
    got = oracle.scanrows_argmax_i32(k, vis)
    for r in range(6):
        row = vis[r * k:(r + 1) * k]
        assert np.array_equal(got[r * k:(r + 1) * k], oracle.scan_argmax_i32(row))
        best = (lo, hi)
        for j in range(k):   # the running argmax, by hand
            v, i = int(row[j, 0]), int(row[j, 1])
            if v > best[0] or (v == best[0] and i < best[1]):
                best = (v, i)
            assert got[r * k + j].tolist() == list(best)

    lens = np.array([4, 0, 1, 20, 0, 3], np.int64)
    offsets = np.concatenate(([0], np.cumsum(lens)[:-1])).astype(np.int64)
    vis = np.stack([rng.integers(-4, 4, 40), np.arange(40)], axis=1).astype(np.int32)  # 12 pairs unused
    got = oracle.segred_argmax_i32(offsets, lens, vis)
    for s in range(6):
        seg = vis[offsets[s]:offsets[s] + lens[s]]
        want = [lo, hi] if lens[s] == 0 else oracle.scan_argmax_i32(seg)[-1].tolist()
        assert got[s].tolist() == want
