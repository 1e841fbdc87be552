"""The C runtime under the entry points, through the public API only: pooled
device memory (rts/c/gpu.h:245-331, free_list.h), error reporting
(docs/c-api.rst:37-58,153-166), contexts side by side, device selection,
profiling report and logging."""
import json
import threading

import numpy as np
import pytest

from futhark_amd import Context, FutharkError

pytestmark = pytest.mark.gpu


def test_out_of_memory_is_reported_and_does_not_stick(segops_lib):
    with Context(segops_lib) as c:
        small = c.call("iota_i64", ["i64_1d"], 1000)
        small.free()                                      # a pooled block the retry loop may release
        with pytest.raises(FutharkError) as e:
            c.call("iota_i64", ["i64_1d"], 1 << 40)       # 8 TiB
        assert e.value.code == 3                          # FUTHARK_OUT_OF_MEMORY
        assert "Failed to allocate memory in space 'device'" in e.value.message
        assert c.get_error() is None                      # reading the message cleared it
        out = c.call("iota_i64", ["i64_1d"], 1000)        # the context is still usable
        assert out.values()[-1] == 999
        out.free()
        with pytest.raises(FutharkError, match="Range 0..<-1 is invalid") as e:
            c.call("iota_i64", ["i64_1d"], -1)
        assert e.value.code == 2                          # FUTHARK_PROGRAM_ERROR


def test_freed_blocks_are_reused_and_clear_caches_returns_them(segops_lib):
    with Context(segops_lib) as c:
        a = c.call("iota_i64", ["i64_1d"], 1 << 20)
        p = a.device_ptr
        a.free()
        b = c.call("iota_i64", ["i64_1d"], 1 << 20)       # same size, same tag: the pooled block
        assert b.device_ptr == p
        assert b.values()[12345] == 12345
        b.free()
        c.clear_caches()
        d = c.call("iota_i64", ["i64_1d"], 1 << 20)
        assert d.values()[-1] == (1 << 20) - 1
        d.free()


def test_values_are_reference_counted_through_aliases(segops_lib):
    with Context(segops_lib) as c:
        k = c.new("u32_1d", np.array([3, 1, 2], np.uint32))
        v = c.new("i32_1d", np.array([0, 1, 2], np.int32))
        t = c.new_opaque("tup2_arr1d_u32_arr1d_i32", k, v)
        alias = t.project(0)
        assert alias.device_ptr == k.device_ptr           # an alias, not a copy
        k.free(); t.free()                                # two of three references gone
        junk = c.new("u32_1d", np.array([9, 9, 9], np.uint32))   # would reuse a freed block
        assert junk.device_ptr != alias.device_ptr
        assert alias.values().tolist() == [3, 1, 2]
        for h in (alias, junk, v):
            h.free()


def test_two_contexts_and_two_threads(segops_lib):
    xs = np.arange(100000, dtype=np.int32)
    results = {}

    def work(name, scale):
        with Context(segops_lib) as c:
            a = c.new("i32_1d", (xs.astype(np.int64) * scale).astype(np.int32))
            for _ in range(20):
                results[name] = int(c.call("reduce_add_i32", [np.int32], a))
            a.free()

    ts = [threading.Thread(target=work, args=(f"t{s}", s)) for s in (1, 2, 3)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    base = int(xs.astype(np.int64).sum())
    wrap = lambda x: int(np.array(x, np.int64).astype(np.int32))   # i32 addition wraps
    assert results == {f"t{s}": wrap(base * s) for s in (1, 2, 3)}


def test_device_selection(segops_lib):
    with Context(segops_lib, device="#0") as c:
        assert c.call("reduce_add_i32", [np.int32], c.new("i32_1d", np.ones(10, np.int32))) == 10
    with pytest.raises(FutharkError):
        Context(segops_lib, device="#7")                  # one GPU on the box
    with pytest.raises(FutharkError):
        Context(segops_lib, device="no such device name")


def test_profiling_report_and_pause(segops_lib):
    with Context(segops_lib, profiling=True) as c:
        a = c.new("f32_1d", np.ones(4096, np.float32))
        c.call("scan_add_f32", ["f32_1d"], a).free()
        c.L.futhark_context_pause_profiling(c.ptr)
        c.call("reduce_add_f32", [np.float32], a)
        c.L.futhark_context_unpause_profiling(c.ptr)
        c.call("exscan_add_f32", ["f32_1d"], a).free()
        rep = json.loads(c.report())
        names = [e["name"] for e in rep["events"]]
        assert names.count("segscan") == 2 and not any("segred" in n for n in names), names
        assert all(e["duration"] > 0 and isinstance(e["details"], dict) for e in rep["events"])
        assert rep["memory"]["device"] >= 2 * 4096 * 4      # peak: the input and one result
        assert json.loads(c.report())["events"] == []     # a report empties the event list
        a.free()
    with Context(segops_lib) as c:                        # profiling off: nothing is recorded
        a = c.new("f32_1d", np.ones(16, np.float32))
        c.call("scan_add_f32", ["f32_1d"], a).free()
        assert json.loads(c.report())["events"] == []
        a.free()


def test_debugging_log_goes_to_the_logging_file(segops_lib, tmp_path):
    import ctypes as C
    libc = C.CDLL(None)
    libc.fopen.restype = C.c_void_p
    libc.fopen.argtypes = [C.c_char_p, C.c_char_p]
    libc.fclose.argtypes = [C.c_void_p]
    path = tmp_path / "log.txt"
    f = libc.fopen(str(path).encode(), b"w")
    assert f
    with Context(segops_lib, debugging=True) as c:
        segops_lib.lib.futhark_context_set_logging_file.argtypes = [C.c_void_p, C.c_void_p]
        segops_lib.lib.futhark_context_set_logging_file(c.ptr, f)
        a = c.new("i32_1d", np.ones(100, np.int32))
        c.call("scan_add_i32", ["i32_1d"], a).free()
        a.free()
    libc.fclose(f)
    text = path.read_text()
    assert "Allocating" in text and "segscan" in text


def test_tuning_parameters_select_other_code_paths_with_the_same_results(segops_lib):
    """The three tuning parameters are thresholds inside the kernel library.  Values far from
    the defaults push small inputs down the paths that large inputs take."""
    import oracle
    rng = np.random.default_rng(12)
    tuning = {"segops.hist_lds_bins_max": 256, "segops.segred_small_threshold": 16,
              "segops.matmul_pad_min_work": 1}
    with Context(segops_lib, profiling=True, tuning=tuning) as c:
        # 3000 bins > 4 ranges of 256: the partitioned histogram
        is_ = rng.integers(-5, 3005, 200000).astype(np.int32)
        vs = rng.integers(-1000, 1000, 200000).astype(np.int32)
        out = c.call("hist_add_i32", ["i32_1d"], 3000, c.new("i32_1d", is_), c.new("i32_1d", vs))
        assert np.array_equal(out.values(), oracle.hist("add", "i32", 3000, is_, vs))
        # 700 bins: three LDS ranges in one launch
        out = c.call("hist_max_i32", ["i32_1d"], 700, c.new("i32_1d", is_ % 700), c.new("i32_1d", vs))
        assert np.array_equal(out.values(), oracle.hist("max", "i32", 700, is_ % 700, vs))
        # rows of 100 > 16: whole blocks per row; rows of 40000 in pieces
        for m, k in [(300, 100), (3, 40000)]:
            xss = rng.integers(-1000, 1000, (m, k)).astype(np.int64)
            out = c.call("segreduce_add_i64", ["i64_1d"], c.new("i64_2d", xss))
            assert np.array_equal(out.values(), xss.sum(axis=1))
        # a 200 x 200 x 30 product on padded operands (1.2 M multiply-adds: below the default)
        A = rng.standard_normal((1, 200, 30)).astype(np.float32)
        B = rng.standard_normal((1, 30, 200)).astype(np.float32)
        out = c.call("bmm_f32", ["f32_3d"], c.new("f32_3d", A), c.new("f32_3d", B))
        np.testing.assert_allclose(out.values(), A.astype(np.float64) @ B.astype(np.float64), rtol=1e-4, atol=1e-5)
        ev = [e for e in json.loads(c.report())["events"] if e["name"] == "segmap_matmul"]
        assert ev[0]["details"]["padded"] is True
    with Context(segops_lib, profiling=True) as c:    # back to the defaults
        out = c.call("bmm_f32", ["f32_3d"], c.new("f32_3d", A), c.new("f32_3d", B))
        np.testing.assert_allclose(out.values(), A.astype(np.float64) @ B.astype(np.float64), rtol=1e-4, atol=1e-5)
        ev = [e for e in json.loads(c.report())["events"] if e["name"] == "segmap_matmul"]
        assert ev[0]["details"]["padded"] is False
    # two contexts alive at once keep their own values, whichever was created or used last
    with Context(segops_lib, profiling=True, tuning=tuning) as c1, Context(segops_lib, profiling=True) as c2:
        for c in (c1, c2, c1, c2):
            out = c.call("bmm_f32", ["f32_3d"], c.new("f32_3d", A), c.new("f32_3d", B))
            np.testing.assert_allclose(out.values(), A.astype(np.float64) @ B.astype(np.float64), rtol=1e-4, atol=1e-5)
        for c, padded in ((c1, True), (c2, False)):
            ev = [e for e in json.loads(c.report())["events"] if e["name"] == "segmap_matmul"]
            assert len(ev) == 2 and all(e["details"]["padded"] is padded for e in ev)
    with pytest.raises(KeyError):
        Context(segops_lib, tuning={"segops.no_such_parameter": 1})


def test_scalar_results_arrive_at_the_synchronisation(segops_lib):
    """A scalar result may be used after futhark_context_sync (docs/c-api.rst:578-581).  Entry
    points that return one do not wait for the device: many calls are queued back to back, each
    with its own destination, and one synchronisation delivers all of them - also more calls than
    the runtime has pinned slots for (64), which it must drain by itself on the way."""
    import ctypes as C
    import oracle
    from futhark_amd import datagen as dg
    with Context(segops_lib) as c:
        L = c.L
        arrays, want = [], []
        for i in range(150):
            xs = dg.uniform_int(100 + i, 1000 + 37 * i, -1000, 1000, np.int32)
            arrays.append(c.new("i32_1d", xs))
            want.append(int(oracle.reduce("add", "i32", xs)))
        outs = (C.c_int32 * len(arrays))(*([-1] * len(arrays)))
        for i, a in enumerate(arrays):
            rc = L.futhark_entry_reduce_add_i32(c.ptr, C.byref(outs, 4 * i), a.ptr)
            assert rc == 0
        c.sync()
        assert list(outs) == want
        # the same destination twice before one synchronisation: the later call wins
        one = C.c_int32(-1)
        assert L.futhark_entry_reduce_add_i32(c.ptr, C.byref(one), arrays[3].ptr) == 0
        assert L.futhark_entry_reduce_add_i32(c.ptr, C.byref(one), arrays[4].ptr) == 0
        c.sync()
        assert one.value == want[4]
        f = c.new("f32_1d", np.arange(1, 5, dtype=np.float32))
        sq = C.c_float(-1.0)
        assert L.futhark_entry_sumsq_f32(c.ptr, C.byref(sq), f.ptr) == 0
        c.sync()
        assert sq.value == 30.0
        for a in arrays + [f]:
            a.free()


def test_scans_under_both_ways_of_picking_ticket_counters(segops_lib):
    """The blocks of the single-pass scan pick their ticket counter by block index while the
    context is alone in the process (no arrival atomic), by order of arrival otherwise or when
    `segops.scan_arrival_tickets` says so.  Same results either way: a context of its own with
    the parameter set, a second context alive beside it (both then take the order of arrival),
    and hundreds of tiles, a few tiles and fewer tiles than counters."""
    import oracle
    from futhark_amd import datagen as dg

    def check(c):
        for n in (5, 40000, 100003, (1 << 22) + 77):
            xs = dg.uniform_int(7, n, -1000, 1000, np.int32)
            flags = (dg.raw_u64(9, n) % np.uint64(900) == 0).astype(np.uint8)
            a, f = c.new("i32_1d", xs), c.new("u8_1d", flags)
            out = c.call("scan_add_i32", ["i32_1d"], a)
            assert np.array_equal(out.values(), oracle.scan("add", "i32", xs)), n
            out.free()
            out = c.call("segscan_max_i32", ["i32_1d"], f, a)
            assert np.array_equal(out.values(), oracle.segscan("max", "i32", flags, xs)), n
            for h in (out, a, f):
                h.free()

    with Context(segops_lib, tuning={"segops.scan_arrival_tickets": 1}) as c1:
        check(c1)
        with Context(segops_lib) as c2:      # two contexts alive: neither assumes the device is its own
            check(c2)
            check(c1)
    with Context(segops_lib) as c3:
        check(c3)
