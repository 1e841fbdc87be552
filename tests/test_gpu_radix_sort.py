"""GPU parity: stable LSD radix sort through the generated-library API.
Bit-exact against the CPU oracle (itself pinned to numpy's stable sort)."""
import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu
SIZES = [0, 1, 2, 63, 64, 65, 511, 8191, 8192, 8193, 100003, (1 << 20) + 5]


@pytest.mark.parametrize("kt", ["u32", "u64"])
def test_keys_only(ctx, kt):
    for n in SIZES:
        keys = dg.uniform_u32(70, n) if kt == "u32" else dg.uniform_u64(71, n)
        out = ctx.call(f"radix_sort_{kt}", [f"{kt}_1d"], ctx.new(f"{kt}_1d", keys))
        got = out.values()
        assert np.array_equal(got, np.sort(keys, kind="stable")), n
        assert np.array_equal(got, oracle.radix_sort(keys))


def _sort_pairs(ctx, kt, keys, vals):
    """The entry point returns one opaque tuple; its two components are projected out and the
    tuple freed (the components live on)."""
    k, v = ctx.new(f"{kt}_1d", keys), ctx.new("i32_1d", vals)
    tup = ctx.call(f"radix_sort_pairs_{kt}_i32", [f"tup2_arr1d_{kt}_arr1d_i32"], k, v)
    ko, vo = tup.project(0), tup.project(1)
    for h in (tup, k, v):
        h.free()
    return ko, vo


def test_opaque_tuple_new_project_store_restore(ctx):
    """Call sequences of tests_lib/c/test_project.c (new, then project twice) and
    test_restore.c (store with p == NULL for the size, then into a buffer, then restore)."""
    keys = np.array([5, 1, 5, 0, 1, 9], np.uint32)
    vals = np.arange(6, dtype=np.int32)
    name = "tup2_arr1d_u32_arr1d_i32"
    k, v = ctx.new("u32_1d", keys), ctx.new("i32_1d", vals)
    tup = ctx.new_opaque(name, k, v)
    k.free(); v.free()                          # the tuple holds its own references
    for _ in range(2):
        a = tup.project(0)
        assert a.values().tolist() == keys.tolist()
        a.free()
    blob = tup.store()
    # two values of the binary data format, one after the other
    assert len(blob) == 2 * (7 + 8) + 6 * 4 + 6 * 4
    assert blob[:7] == b"b\x02\x01 u32" and blob[15 + 24:15 + 24 + 7] == b"b\x02\x01 i32"
    back = ctx.restore_opaque(name, blob)
    assert back.project(0).values().tolist() == keys.tolist()
    assert back.project(1).values().tolist() == vals.tolist()
    out = ctx.call("radix_sort_pairs_u32_i32", [name], back.project(0), back.project(1))
    assert out.project(0).values().tolist() == [0, 1, 1, 5, 5, 9]
    assert out.project(1).values().tolist() == [3, 1, 4, 0, 2, 5]
    with pytest.raises(Exception):
        ctx.restore_opaque(name, b"b\x02\x01 i32" + blob[7:])   # wrong element type
    with pytest.raises(Exception):
        ctx.restore_opaque("tup2_arr1d_u64_arr1d_i32", blob)      # another tuple type
    for h in (tup, back, out):
        h.free()


@pytest.mark.parametrize("kt", ["u32", "u64"])
def test_pairs_are_stable(ctx, kt):
    for n in SIZES:
        # few distinct keys: stability decides the permutation
        raw = dg.uniform_u32(72, n).astype(np.uint64)
        keys = (raw % np.uint64(37)).astype(np.uint32 if kt == "u32" else np.uint64)
        keys = keys << (keys.dtype.type(13) if kt == "u32" else keys.dtype.type(45))
        vals = np.arange(n, dtype=np.int32)
        ko, vo = _sort_pairs(ctx, kt, keys, vals)
        gk, gv = ko.values(), vo.values()
        perm = np.argsort(keys, kind="stable")
        assert np.array_equal(gk, keys[perm]) and np.array_equal(gv, vals[perm].astype(np.int32)), n
        wk, wv = oracle.radix_sort(keys, vals)
        assert np.array_equal(gk, wk) and np.array_equal(gv, wv)


def test_reference_golden(ctx, goldens):
    c = goldens["radixsort"]["cases"][0]
    keys = np.array(c["keys"], np.float32).view(np.uint32)  # positive floats order as their bits
    vals = np.array(c["vals"], np.float32).view(np.int32)
    ko, vo = _sort_pairs(ctx, "u32", keys, vals)
    assert vo.values().view(np.float32).tolist() == np.array(c["out_vals"], np.float32).tolist()


def test_config5_full_size_keys(ctx):
    n = 1 << 26
    keys = dg.uniform_u32(80, n)
    out = ctx.call("radix_sort_u32", ["u32_1d"], ctx.new("u32_1d", keys))
    got = out.values()
    assert np.all(got[1:] >= got[:-1])                      # sorted
    assert np.array_equal(got, oracle.radix_sort(keys))      # the same multiset, same order


def test_config5_full_size_pairs(ctx):
    n = 1 << 26
    keys = dg.uniform_u64(81, n)
    vals = np.arange(n, dtype=np.int32)
    ko, vo = _sort_pairs(ctx, "u64", keys, vals)
    gk, gv = ko.values(), vo.values()
    assert np.all(gk[1:] >= gk[:-1])
    assert np.array_equal(keys[gv], gk)                      # vo is the sorting permutation
    ties = gk[1:] == gk[:-1]
    assert np.all(gv[1:][ties] > gv[:-1][ties])              # ties keep input order
    wk, wv = oracle.radix_sort(keys, vals)
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)


def test_more_than_two_to_the_31_keys(ctx):
    """Positions are unsigned 32-bit numbers, so the sort takes more than 2^31 keys.  The CPU
    does not sort 8 GiB in the time a test has: the result is checked for order and, against the
    input, for the same multiset (counts of the high and of the low 16 bits, sum and xor), in
    pieces that keep the temporaries small."""
    n = (1 << 31) + 12345
    rng = np.random.default_rng(7)
    keys = rng.integers(0, 1 << 32, n, dtype=np.uint32)
    a = ctx.new("u32_1d", keys)
    out = ctx.call("radix_sort_u32", ["u32_1d"], a)
    a.free()
    got = out.values()
    out.free()
    ctx.clear_caches()  # 25 GiB of device buffers go back to the driver
    assert got.shape == (n,)

    def summary(x):
        hi = np.zeros(1 << 16, np.int64)
        lo = np.zeros(1 << 16, np.int64)
        total, parity = 0, 0
        step = 1 << 26
        for i in range(0, n, step):
            p = x[i:i + step]
            hi += np.bincount(p >> 16, minlength=1 << 16)
            lo += np.bincount(p & 0xFFFF, minlength=1 << 16)
            total = (total + int(p.sum(dtype=np.uint64))) & ((1 << 64) - 1)
            parity ^= int(np.bitwise_xor.reduce(p))
        return hi, lo, total, parity

    step = 1 << 26
    for i in range(0, n - 1, step):
        p = got[i:i + step + 1]
        assert np.all(p[:-1] <= p[1:]), i
    want, have = summary(keys), summary(got)
    assert np.array_equal(want[0], have[0]) and np.array_equal(want[1], have[1])
    assert want[2:] == have[2:]


def test_sort_with_64_bit_positions(segops_lib):
    """From 2^32 - 1 keys on the sort counts, scans and scatters with 64-bit positions; the
    tuning parameter segops.sort_wide_positions switches to them at any size, so every key and
    value type goes through that path at sizes the oracle sorts (tests/test_gpu_beyond_2p31.py
    sorts 2^32 + 4099 u32 keys through it).  Bit-exact, ties in input order."""
    from futhark_amd import Context
    with Context(segops_lib, tuning={"segops.sort_wide_positions": 1}) as c:
        for n in [1, 64, 8191, 8193, 100003, (1 << 21) + 5]:
            for kt in ("u32", "u64"):
                keys = dg.uniform_u32(72, n) if kt == "u32" else dg.uniform_u64(73, n)
                if n > 1000:
                    keys[::3] = keys[0]          # many ties
                out = c.call(f"radix_sort_{kt}", [f"{kt}_1d"], c.new(f"{kt}_1d", keys))
                assert np.array_equal(out.values(), oracle.radix_sort(keys)), (kt, n)
                out.free()
                vals = np.arange(n, dtype=np.int32)
                ko, vo = _sort_pairs(c, kt, keys, vals)
                wk, wv = oracle.radix_sort(keys, vals)
                assert np.array_equal(ko.values(), wk) and np.array_equal(vo.values(), wv), (kt, n)
                ko.free(); vo.free()
