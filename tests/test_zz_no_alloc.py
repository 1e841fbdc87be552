"""fa_segscan_static, the scan entry point that allocates nothing (its look-back
scratch is a fixed array inside the library), against the CPU oracle and against
fa_segscan through the generated-library API on the same inputs: integers and
max bit-exact, f32 sums within 1e-5 of the f64-accumulated oracle (the look-back
folds tile aggregates in an order that depends on timing).  Two calls in a row
per case, the second on a smaller input, so that what the first left in the
shared scratch is in the way of the second."""
import ctypes as C

import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg, lib_path

pytestmark = pytest.mark.gpu

FA = {"i32": 0, "i64": 1, "f32": 2}
OP = {"add": 0, "max": 1}
NP = {"i32": np.int32, "i64": np.int64, "f32": np.float32}
FA_ESCRATCH = -3


def _lib():
    k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
    k.fa_segscan_static.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int64,
                                    C.c_int, C.c_void_p]
    k.fa_segscan_static_max_n.restype = C.c_int64
    k.fa_segscan_static_max_n.argtypes = [C.c_int]
    k.fa_segscan_tile_elems.restype = C.c_int64
    k.fa_segscan_tile_elems.argtypes = [C.c_int]
    return k


def _data(t, n, aid):
    if t == "f32":
        return dg.uniform_f32(aid, n)
    return dg.uniform_int(aid, n, -1000, 1000, NP[t])


@pytest.mark.parametrize("t,op", [("i32", "add"), ("f32", "add"), ("f32", "max"), ("i64", "add")])
def test_static_scan_matches_pooled_scan(ctx, t, op):
    k = _lib()
    assert k.fa_segscan_static_init() == 0
    for seg in (False, True):
        for excl in (0, 1):
            for n in ((1 << 22) + 12345, 70001):   # hundreds of tiles, then a few
                xs = _data(t, n, 5 + excl)
                flags = (dg.raw_u64(9, n) % np.uint64(700) == 0).astype(np.uint8)
                a, f = ctx.new(f"{t}_1d", xs), ctx.new("u8_1d", flags)
                if seg:
                    if excl:
                        continue  # the program has no exclusive segmented scan to compare with
                    want = ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, a)
                else:
                    want = ctx.call(f"{'ex' if excl else ''}scan_{op}_{t}", [f"{t}_1d"], a)
                out = ctx.new(f"{t}_1d", np.zeros(n, NP[t]))
                print(f"fa_segscan_static {t} {op} seg={seg} excl={excl} n={n}", flush=True)
                rc = k.fa_segscan_static(ctx.stream, FA[t], OP[op], a.device_ptr,
                                         f.device_ptr if seg else None, n, excl, out.device_ptr)
                assert rc == 0
                got, ref = out.values(), want.values()
                variant = "f64acc" if (t, op) == ("f32", "add") else "lit"
                if seg:
                    truth = oracle.segscan(op, t, flags, xs, variant)
                else:
                    truth = oracle.scan(op, t, xs, variant, exclusive=bool(excl))
                if t == "f32" and op == "add":
                    for other in (truth, ref):
                        assert np.all(np.abs(got.astype(np.float64) - other) <= 1e-5 * np.abs(other))
                else:
                    assert np.array_equal(got, truth)
                    assert np.array_equal(got, ref)
                for h in (a, f, out, want):
                    h.free()


def test_static_scan_rejects_what_its_scratch_cannot_hold(ctx):
    k = _lib()
    for t in ("i32", "i64"):
        limit = k.fa_segscan_static_max_n(FA[t])
        # the documented figure: 256 KiB of descriptors, one per tile
        assert limit == 16384 * k.fa_segscan_tile_elems(FA[t]) == {"i32": 234881024, "i64": 117440512}[t]
        a = ctx.new(f"{t}_1d", np.zeros(16, NP[t]))
        # rejected before anything is launched, so the short buffers are never touched
        assert k.fa_segscan_static(ctx.stream, FA[t], 0, a.device_ptr, None, limit + 1, 0,
                                   a.device_ptr) == FA_ESCRATCH
        a.free()
