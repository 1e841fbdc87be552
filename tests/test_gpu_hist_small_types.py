"""GPU parity for histograms over the element types whose updates the
reference emulates with compare-and-swap (8- and 16-bit integers, f16:
src/Futhark/CodeGen/ImpGen/GPU/Base.hs:735-767, rts/c/atomics8.h,
atomics16.h) and over the unsigned 32/64-bit types.  Integers are bit-exact
against the oracle; f16 sums within 1e-2 of the sum accumulated in double, and
exact where every partial sum is an f16 value."""
import ctypes as C

import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu
NP = {"i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16, "u32": np.uint32,
      "u64": np.uint64}
INT_OPS = ("add", "max", "min", "and", "or", "xor")
# (n, H): one LDS range with copies, several ranges, the partitioned path (more than four
# ranges of 32768 bins), and one device atomic per element (more than 255 ranges)
SHAPES = [(0, 5), (100, 7), (100003, 1000), (300001, 65536), (200000, 300000), (50000, 9000000)]


def _vals(t, n, seed):
    ii = np.iinfo(NP[t])
    return np.random.default_rng(seed).integers(ii.min, ii.max, n, dtype=NP[t], endpoint=True)


@pytest.mark.parametrize("t", list(NP))
@pytest.mark.parametrize("op", INT_OPS)
def test_integer_hist_and_rbi(ctx, t, op):
    for n, H in SHAPES:
        if H > 1000000 and op not in ("add", "max"):
            continue
        is_ = dg.hist_indices(60, n, max(H, 1), "uniform", 3)
        vs = _vals(t, n, 61)
        i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
        out = ctx.call(f"hist_{op}_{t}", [f"{t}_1d"], H, i, v)
        assert np.array_equal(out.values(), oracle.hist(op, t, H, is_, vs)), (n, H)
        out.free()
        dest = _vals(t, H, 63)
        d = ctx.new(f"{t}_1d", dest)
        out = ctx.call(f"rbi_{op}_{t}", [f"{t}_1d"], d, i, v)
        assert np.array_equal(out.values(), oracle.rbi(op, t, dest, is_, vs)), (n, H)
        assert np.array_equal(d.values(), dest)  # the input is not consumed
        for h in (out, d, i, v):
            h.free()


@pytest.mark.parametrize("t", ["i8", "u16"])
def test_contended_bins_wrap_like_the_element_type(ctx, t):
    # 2^22 updates into 3 bins: sums wrap many times over
    n = 1 << 22
    is_ = (np.arange(n, dtype=np.int64) % 3).astype(np.int32)
    vs = _vals(t, n, 7)
    i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
    out = ctx.call(f"hist_add_{t}", [f"{t}_1d"], 3, i, v)
    want = np.array([vs[k::3].sum(dtype=np.uint64) for k in range(3)]).astype(NP[t])
    assert np.array_equal(out.values(), want)
    assert np.array_equal(want, oracle.hist("add", t, 3, is_, vs))
    for h in (out, i, v):
        h.free()


def test_reference_goldens(ctx, goldens):
    npx = dict(NP, i32=np.int32)

    def run(entry, t, c, dest=None, view=None):
        """view: the signed type the golden file writes the unsigned values and results in."""
        vs = np.array(c["vs"], npx[view or t]).view(NP[t])
        i, v = ctx.new("i32_1d", np.array(c["is"], np.int32)), ctx.new(f"{t}_1d", vs)
        if dest is None:
            out = ctx.call(f"hist_{entry}_{t}", [f"{t}_1d"], c["n"], i, v)
        else:
            d = ctx.new(f"{t}_1d", np.array(dest, NP[t]))
            out = ctx.call(f"rbi_{entry}_{t}", [f"{t}_1d"], d, i, v)
            d.free()
        got = out.values()
        for h in (out, i, v):
            h.free()
        return got if view is None else got.view(npx[view])

    for bits in (8, 16):
        t, u = f"i{bits}", f"u{bits}"
        for c in goldens[f"hist_add_{t}"]["cases"]:
            assert run("add", t, c, dest=c["dest"]).tolist() == c["out"]
        for op in ("and", "or", "xor"):
            for c in goldens[f"hist_{op}{bits}"]["cases"]:
                assert run(op, t, c).tolist() == c["out"], (op, bits, c)
        for op in ("max", "min"):
            for c in goldens[f"hist_{op}{bits}"]["cases"]:
                zeros = [0] * c["n"]
                assert run(op, t, c, dest=zeros).tolist() == c["out"]
                assert run(op, u, c, dest=zeros, view=t).tolist() == c["out_unsigned"], (op, bits, c)
    for op in ("max", "min"):
        for c in goldens[f"hist_{op}_u32"]["cases"]:
            assert run(op, "u32", c, dest=[0] * c["n"], view="i32").tolist() == c["out"]


def _f(xs):
    return np.array([np.nan if x == "nan" else x for x in xs], dtype=np.float32)


def _f16(ctx, a):
    return ctx.new("f16_1d", np.asarray(a, np.float16).view(np.uint16))


def test_f16_goldens_and_exact_sums(ctx, goldens):
    for c in goldens["hist_f16"]["cases"]:
        d, v = _f16(ctx, _f(c["dest"])), _f16(ctx, _f(c["vs"]))
        i = ctx.new("i32_1d", np.array(c["is"], np.int32))
        out = ctx.call("rbi_add_f16", ["f16_1d"], d, i, v)
        got = out.values().view(np.float16).astype(np.float32)
        np.testing.assert_allclose(got, _f(c["out"]), rtol=2e-3, equal_nan=True)
        for h in (out, d, i, v):
            h.free()
    # small non-negative integers, bins that stay below 2048: every partial sum in any order is
    # an f16 value, so the result is exact
    rng = np.random.default_rng(5)
    for n, H in [(100000, 300), (400000, 70000), (300000, 200000)]:
        is_ = dg.hist_indices(70, n, H, "uniform", 2)
        vs = rng.integers(0, 4, n).astype(np.float16)
        i, v = ctx.new("i32_1d", is_), _f16(ctx, vs)
        out = ctx.call("hist_add_f16", ["f16_1d"], H, i, v)
        got = out.values().view(np.float16)
        want = oracle.hist("add", "f16", H, is_, vs, "f64acc")
        assert want.max() < 2048
        assert np.array_equal(got, want), (n, H)
        for h in (out, i, v):
            h.free()


def test_f16_sums_within_tolerance_and_minmax_exact(ctx):
    n, H = 1 << 20, 4096  # 256 values of [0,1) per bin
    is_ = dg.hist_indices(71, n, H, "uniform", 1)
    vs = dg.uniform_f32(72, n).astype(np.float16)
    i, v = ctx.new("i32_1d", is_), _f16(ctx, vs)
    out = ctx.call("hist_add_f16", ["f16_1d"], H, i, v)
    got = out.values().view(np.float16).astype(np.float64)
    want = oracle.hist("add", "f16", H, is_, vs, "f64acc").astype(np.float64)
    lit = oracle.hist("add", "f16", H, is_, vs, "lit").astype(np.float64)
    rel = np.abs(got - want) / np.maximum(np.abs(want), 1e-6)
    assert rel.max() <= 1e-2, rel.max()  # tolerance for 16-bit floats
    # rounding once per block and bin is closer to the exact sums than rounding per element
    assert np.abs(got - want).mean() <= np.abs(lit - want).mean()
    out.free()
    # max and min do not depend on the order: bit-exact, NaN operands ignored, negative values
    ws = (dg.normal_f32(73, n) * 100).astype(np.float16)
    ws[::97] = np.nan
    w = _f16(ctx, ws)
    for op in ("max", "min"):
        out = ctx.call(f"hist_{op}_f16", ["f16_1d"], H, i, w)
        want = oracle.hist(op, "f16", H, is_, ws)
        assert np.array_equal(out.values(), want.view(np.uint16)), op
        out.free()
    # a destination that holds NaN: fmax / fmin replace it by the other operand
    dest = np.full(H, np.nan, np.float16)
    d = _f16(ctx, dest)
    out = ctx.call("rbi_max_f16", ["f16_1d"], d, i, w)
    want = oracle.rbi("max", "f16", dest, is_, ws)
    assert np.array_equal(out.values(), want.view(np.uint16))
    for h in (out, d, i, v, w):
        h.free()


def test_destination_cells_that_share_a_word_with_foreign_bytes(ctx):
    """The kernel library called directly: dest starts at an odd address inside
    a larger buffer; the bytes before and after it must come back unchanged."""
    from futhark_amd import lib_path
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_seghist.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p,
                             C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_size_t]
    k.fa_seghist_scratch_bytes.restype = C.c_size_t
    k.fa_seghist_scratch_bytes.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int64]
    FA_I8, FA_I16, FA_ADD = 8, 10, 0
    rng = np.random.default_rng(11)
    n = 200003
    for t, dt, code, lead in (("i8", np.int8, FA_I8, 1), ("i8", np.int8, FA_I8, 3),
                              ("i16", np.int16, FA_I16, 1)):
        for H in (5, 1001):
            is_ = rng.integers(-2, H + 2, n).astype(np.int32)
            vs = rng.integers(-100, 100, n).astype(dt)
            host = rng.integers(-100, 100, lead + H + 5).astype(dt)
            buf = ctx.new("u8_1d", host.view(np.uint8))
            d_is, d_vs = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
            sb = k.fa_seghist_scratch_bytes(code, 0, n, H)
            scratch = ctx.new("u8_1d", np.zeros(max(sb, 256), np.uint8))
            dest_ptr = buf.device_ptr + lead * host.itemsize
            print(f"fa_seghist {t} lead={lead} H={H}", flush=True)
            rc = k.fa_seghist(ctx.stream, code, FA_ADD, d_is.device_ptr, 0, d_vs.device_ptr, n,
                              dest_ptr, H, scratch.device_ptr, sb)
            assert rc == 0
            got = buf.values().view(dt)
            want = host.copy()
            want[lead:lead + H] = oracle.rbi("add", t, host[lead:lead + H], is_, vs)
            assert np.array_equal(got, want), (t, lead, H)
            for h in (buf, d_is, d_vs, scratch):
                h.free()
