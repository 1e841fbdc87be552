"""GPU parity for the bitwise operators (and, or, xor on i32/i64) through every
SegOp entry point, bit-exact against the oracle; histogram cases of
tests/hist/{and,or,xor,and64,xor64}.fut of the reference."""
import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu
NP = {"i32": np.int32, "i64": np.int64}
OPS = ("and", "or", "xor")


def _bits(t, n, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(np.iinfo(NP[t]).min, np.iinfo(NP[t]).max, n, dtype=NP[t], endpoint=True)
    # `and` over many random words is 0 and `or` is -1 almost surely: thin out the
    # bits so that long reductions stay informative
    if n > 64:
        x |= rng.integers(0, 2, n).astype(NP[t]) * NP[t](-1) if seed % 2 else NP[t](0)
    return x


@pytest.mark.parametrize("t", ["i32", "i64"])
@pytest.mark.parametrize("op", OPS)
def test_reduce_scan_segscan_segred(ctx, t, op):
    for n in [0, 1, 63, 4097, 100003, (1 << 20) + 7]:
        xs = _bits(t, n, 100 + n % 7)
        a = ctx.new(f"{t}_1d", xs)
        assert ctx.call(f"reduce_{op}_{t}", [NP[t]], a) == oracle.reduce(op, t, xs)
        for entry, excl in (("scan", False), ("exscan", True)):
            out = ctx.call(f"{entry}_{op}_{t}", [f"{t}_1d"], a)
            assert np.array_equal(out.values(), oracle.scan(op, t, xs, exclusive=excl)), (entry, n)
            out.free()
        if n > 0:
            offsets, lens, flags = dg.segments(7, n, 300)
            f = ctx.new("u8_1d", flags)
            out = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, a)
            assert np.array_equal(out.values(), oracle.segscan(op, t, flags, xs)), n
            out.free(); f.free()
            o, l = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens)
            out = ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, a)
            assert np.array_equal(out.values(), oracle.segred(op, t, offsets, lens, xs)), n
            for h in (out, o, l):
                h.free()
        a.free()
    xss = _bits(t, 37 * 1000, 5).reshape(37, 1000)
    m = ctx.new(f"{t}_2d", xss)
    out = ctx.call(f"segreduce_{op}_{t}", [f"{t}_1d"], m)
    assert np.array_equal(out.values(), oracle.segreduce(op, t, xss))
    out.free(); m.free()


@pytest.mark.parametrize("t", ["i32", "i64"])
@pytest.mark.parametrize("op", OPS)
def test_hist_and_rbi(ctx, t, op):
    for n, H in [(0, 5), (100, 7), (100003, 1000), (300001, 65536), (200000, 300000)]:
        is_ = dg.hist_indices(40, n, max(H, 1), "uniform", 3)
        vs = _bits(t, n, 41)
        i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)
        out = ctx.call(f"hist_{op}_{t}", [f"{t}_1d"], H, i, v)
        assert np.array_equal(out.values(), oracle.hist(op, t, H, is_, vs)), (n, H)
        out.free()
        dest = _bits(t, H, 43)
        d = ctx.new(f"{t}_1d", dest)
        out = ctx.call(f"rbi_{op}_{t}", [f"{t}_1d"], d, i, v)
        assert np.array_equal(out.values(), oracle.rbi(op, t, dest, is_, vs)), (n, H)
        for h in (out, d, i, v):
            h.free()


def test_reference_goldens(ctx, goldens):
    for name in ("hist_and", "hist_or", "hist_xor", "hist_and64", "hist_xor64"):
        op, t = name[5:].rstrip("64"), goldens[name]["type"]
        for c in goldens[name]["cases"]:
            i = ctx.new("i32_1d", np.array(c["is"], np.int32))
            v = ctx.new(f"{t}_1d", np.array(c["vs"], NP[t]))
            out = ctx.call(f"hist_{op}_{t}", [f"{t}_1d"], c["n"], i, v)
            assert out.values().tolist() == c["out"], (name, c)
            for h in (out, i, v):
                h.free()
