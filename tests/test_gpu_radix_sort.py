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


@pytest.mark.parametrize("kt", ["u32", "u64"])
def test_pairs_are_stable(ctx, kt):
    for n in SIZES:
        # few distinct keys: stability decides the permutation
        raw = dg.uniform_u32(72, n).astype(np.uint64)
        keys = (raw % np.uint64(37)).astype(np.uint32 if kt == "u32" else np.uint64)
        keys = keys << (keys.dtype.type(13) if kt == "u32" else keys.dtype.type(45))
        vals = np.arange(n, dtype=np.int32)
        ko, vo = ctx.call(f"radix_sort_pairs_{kt}_i32", [f"{kt}_1d", "i32_1d"],
                          ctx.new(f"{kt}_1d", keys), ctx.new("i32_1d", vals))
        gk, gv = ko.values(), vo.values()
        perm = np.argsort(keys, kind="stable")
        assert np.array_equal(gk, keys[perm]) and np.array_equal(gv, vals[perm].astype(np.int32)), n
        wk, wv = oracle.radix_sort(keys, vals)
        assert np.array_equal(gk, wk) and np.array_equal(gv, wv)


def test_reference_golden(ctx, goldens):
    c = goldens["radixsort"]["cases"][0]
    keys = np.array(c["keys"], np.float32).view(np.uint32)  # positive floats order as their bits
    vals = np.array(c["vals"], np.float32).view(np.int32)
    ko, vo = ctx.call("radix_sort_pairs_u32_i32", ["u32_1d", "i32_1d"], ctx.new("u32_1d", keys),
                      ctx.new("i32_1d", vals))
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
    ko, vo = ctx.call("radix_sort_pairs_u64_i32", ["u64_1d", "i32_1d"], ctx.new("u64_1d", keys),
                      ctx.new("i32_1d", vals))
    gk, gv = ko.values(), vo.values()
    assert np.all(gk[1:] >= gk[:-1])
    assert np.array_equal(keys[gv], gk)                      # vo is the sorting permutation
    ties = gk[1:] == gk[:-1]
    assert np.all(gv[1:][ties] > gv[:-1][ties])              # ties keep input order
    wk, wv = oracle.radix_sort(keys, vals)
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
