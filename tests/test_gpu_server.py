"""The server executable driven over its pipe the way `futhark bench/test` drive
a compiled program (docs/server-protocol.rst): values go in and out as files in
the binary data format, results are checked against the oracle.  Replies and
error texts are those of rts/c/server.h."""
import os
import subprocess
from pathlib import Path

import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg
from futhark_amd import values as fv
from futhark_amd.server import SERVER, Server, ServerFailure


def test_server_without_a_device_fails_at_start():
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    proc = subprocess.run([str(SERVER)], input="", capture_output=True, text=True, timeout=60)
    assert proc.returncode == 1
    assert "Error during context initialisation" in proc.stderr
    assert "%%% OK" not in proc.stdout


def test_print_params_needs_no_device():
    proc = subprocess.run([str(SERVER), "--print-params"], capture_output=True, text=True,
                          timeout=60)
    assert proc.returncode == 0
    assert "segops.hist_lds_bins_max (shared_memory)" in proc.stdout.splitlines()


pytestmark_gpu = pytest.mark.gpu


@pytest.fixture(scope="module")
def srv():
    with Server("-P") as s:
        yield s


@pytest.mark.gpu
def test_introspection(srv):
    types = srv.cmd("types")
    assert {"i32", "[]f32", "[][]f32", "[][][]f16", "([]u32, []i32)"} <= set(types)
    entries = srv.cmd("entry_points")
    assert len(entries) == (4 * 3 + 2 * 3) * 16 + (6 * 6 + 3) * 4 + 26 and "segscan_add_f32" in entries
    from futhark_amd import manifest
    m = manifest.manifest()            # the server and the manifest describe the same API
    assert set(entries) == set(m["entry_points"])
    assert set(types) == set(m["types"]) | {"i32", "i64", "f32", "f64"}
    for name, e in m["entry_points"].items():   # every entry point, whatever its number of inputs
        assert srv.cmd("inputs", name) == [("*" if i["unique"] else "") + i["type"] for i in e["inputs"]]
        assert srv.cmd("output", name) == [("*" if e["output"]["unique"] else "") + e["output"]["type"]]
        assert [l.split()[0] for l in srv.cmd("tuning_params", name)] == e["tuning_params"]
    assert srv.cmd("inputs", "segscan_add_f32") == ["[]u8", "[]f32"]
    assert srv.cmd("output", "segscan_add_f32") == ["*[]f32"]
    assert srv.cmd("inputs", "rbi_add_i32") == ["*[]i32", "[]i32", "[]i32"]
    assert srv.cmd("inputs", "hist_max_f32") == ["i64", "[]i32", "[]f32"]
    assert srv.cmd("kind", "[]f32") == ["array"] and srv.cmd("kind", "i64") == ["primitive"]
    assert srv.cmd("kind", "([]u64, []i32)") == ["record"]
    assert srv.cmd("rank", "[][][]f16") == ["3"] and srv.cmd("elemtype", "[][][]f16") == ["f16"]
    assert srv.cmd("fields", "([]u32, []i32)") == ["0 []u32", "1 []i32"]
    assert srv.cmd("tuning_params", "hist_add_i32") == ["segops.hist_lds_bins_max shared_memory"]
    assert srv.cmd("tuning_param_class", "segops.segred_small_threshold") == ["threshold"]
    assert srv.cmd("attributes", "scan_add_i32") == []
    with pytest.raises(ServerFailure, match="Unknown entry point: nope"):
        srv.cmd("inputs", "nope")
    with pytest.raises(ServerFailure, match="Not an array type"):
        srv.cmd("rank", "i32")
    with pytest.raises(ServerFailure, match="Empty line"):
        srv.cmd()


@pytest.mark.gpu
def test_restore_call_store_segscan(srv, tmp_path):
    n = 300_007
    offsets, lens, flags = dg.segments(11, n, 700)
    xs = dg.uniform_f32(12, n)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    fv.write_binary(fin, [flags, xs, offsets, lens])
    srv.cmd("restore", fin, "flags", "[]u8", "xs", "[]f32", "offs", "[]i64", "lens", "[]i64")
    assert srv.cmd("type", "xs") == ["[]f32"] and srv.cmd("shape", "flags") == [str(n)]
    usec = srv.call("segscan_add_f32", "scanned", "flags", "xs")
    assert usec > 0
    srv.call("segred_add_f32", "sums", "offs", "lens", "xs")
    srv.call("reduce_max_f32", "top", "xs")
    srv.cmd("store", fout, "scanned", "sums", "top")
    scanned, sums, top = fv.read_binary(fout, [("f32", 1), ("f32", 1), ("f32", 0)])
    ref = oracle.segscan("add", "f32", flags, xs, "f64acc")
    assert np.allclose(scanned, ref, rtol=1e-5, atol=0)
    assert np.allclose(sums, oracle.segred("add", "f32", offsets, lens, xs, "f64acc"), rtol=1e-5)
    assert top == xs.max()
    # errors leave the server usable and create nothing
    with pytest.raises(ServerFailure, match="Variable already exists: sums"):
        srv.call("segred_add_f32", "sums", "offs", "lens", "xs")
    with pytest.raises(ServerFailure, match=r"Wrong input type.  Expected \[\]u8, got \[\]f32."):
        srv.call("segscan_add_f32", "bad", "xs", "xs")
    with pytest.raises(ServerFailure, match="Unknown variable: ghost"):
        srv.call("scan_add_f32", "bad", "ghost")
    with pytest.raises(ServerFailure, match="Unknown variable: bad"):
        srv.cmd("type", "bad")
    with pytest.raises(ServerFailure, match="invalid sizes"):
        srv.call("segscan_add_f32", "bad", "flags", "sums")
    with pytest.raises(ServerFailure, match="Unknown variable: bad"):
        srv.cmd("type", "bad")
    srv.cmd("rename", "sums", "totals")
    assert srv.cmd("type", "totals") == ["[]f32"]
    srv.cmd("free", "flags", "xs", "offs", "lens", "scanned", "totals", "top")
    with pytest.raises(ServerFailure, match="Unknown variable: xs"):
        srv.cmd("free", "xs")


@pytest.mark.gpu
def test_restore_errors(srv, tmp_path):
    f = tmp_path / "v.bin"
    fv.write_binary(f, [np.arange(5, dtype=np.int32), np.arange(3, dtype=np.int32)])
    with pytest.raises(ServerFailure, match="Failed to open"):
        srv.cmd("restore", tmp_path / "missing.bin", "a", "[]i32")
    with pytest.raises(ServerFailure, match="Failed to restore variable a"):
        srv.cmd("restore", f, "a", "[]f32")
    with pytest.raises(ServerFailure, match="Expected EOF after reading 1 values"):
        srv.cmd("restore", f, "a", "[]i32")
    srv.cmd("free", "a")
    srv.cmd("restore", f, "a", "[]i32", "b", "[]i32")
    assert srv.cmd("shape", "b") == ["3"]
    srv.cmd("free", "a", "b")


@pytest.mark.gpu
def test_scalars_new_array_index(srv, tmp_path):
    f = tmp_path / "s.bin"
    fv.write_binary(f, [np.array(7, np.int64), np.array(5, np.int32), np.array(-2, np.int32)])
    srv.cmd("restore", f, "k", "i64", "a", "i32", "b", "i32")
    srv.cmd("new_array", "arr", "[]i32", 3, "a", "b", "a")
    srv.cmd("index", "elem", "arr", 1)
    srv.call("replicate_i32", "rep", "k", "a")
    srv.call("iota_i64", "io", "k")
    srv.call("reduce_add_i32", "tot", "rep")
    out = tmp_path / "o.bin"
    srv.cmd("store", out, "arr", "elem", "rep", "io", "tot")
    arr, elem, rep, io, tot = fv.read_binary(
        out, [("i32", 1), ("i32", 0), ("i32", 1), ("i64", 1), ("i32", 0)])
    assert arr.tolist() == [5, -2, 5] and elem == -2 and rep.tolist() == [5] * 7
    assert io.tolist() == list(range(7)) and tot == 35
    with pytest.raises(ServerFailure, match="Index out of bounds"):
        srv.cmd("index", "oob", "arr", 3)
    with pytest.raises(ServerFailure, match="Expected 2 values, but got 1."):
        srv.cmd("new_array", "x", "[]i32", 2, "a")
    with pytest.raises(ServerFailure, match=r"Value 0 mismatch: expected type i32, got i64"):
        srv.cmd("new_array", "x", "[]i32", 1, "k")
    srv.cmd("free", "k", "a", "b", "arr", "elem", "rep", "io", "tot")


@pytest.mark.gpu
def test_entry_with_four_inputs(srv, tmp_path, goldens):
    """reduce_by_index_2d takes the most inputs of all entries (tests/hist/hist2d.fut:2-3)."""
    c = goldens["hist2d"]["cases"][0]
    f = tmp_path / "h.bin"
    fv.write_binary(f, [np.array(c["dest"], np.int32), np.array(c["is"], np.int64),
                        np.array(c["js"], np.int64), np.array(c["vs"], np.int32)])
    srv.cmd("restore", f, "dest", "[][]i32", "is", "[]i64", "js", "[]i64", "vs", "[]i32")
    srv.call("rbi_2d_add_i32", "h2", "dest", "is", "js", "vs")
    out = tmp_path / "o.bin"
    srv.cmd("store", out, "h2")
    (h2,) = fv.read_binary(out, [("i32", 2)])
    assert h2.tolist() == c["out"]
    assert srv.cmd("inputs", "rbi_2d_add_i32") == ["*[][]i32", "[]i64", "[]i64", "[]i32"]
    srv.cmd("free", "dest", "is", "js", "vs", "h2")


@pytest.mark.gpu
def test_pair_sort_record_and_hist(srv, tmp_path):
    n = 100_000
    keys = dg.uniform_u32(21, n) % np.uint32(5000)
    vals = np.arange(n, dtype=np.int32)
    idx = dg.hist_indices(22, n, 1000, "uniform")
    f = tmp_path / "p.bin"
    fv.write_binary(f, [keys, vals, np.array(1000, np.int64), idx])
    srv.cmd("restore", f, "keys", "[]u32", "vals", "[]i32", "h", "i64", "is", "[]i32")
    srv.call("radix_sort_pairs_u32_i32", "sorted", "keys", "vals")
    assert srv.cmd("type", "sorted") == ["([]u32, []i32)"]
    srv.cmd("project", "sk", "sorted", "0")
    srv.cmd("project", "sv", "sorted", "1")
    srv.call("hist_add_i32", "hist", "h", "is", "vals")
    out = tmp_path / "o.bin"
    srv.cmd("store", out, "sorted", "sk", "sv", "hist")
    k1, v1, k2, v2, hist = fv.read_binary(
        out, [("u32", 1), ("i32", 1), ("u32", 1), ("i32", 1), ("i32", 1)])
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(k1, keys[order]) and np.array_equal(v1, vals[order])
    assert np.array_equal(k2, k1) and np.array_equal(v2, v1)
    assert np.array_equal(hist, oracle.rbi("add", "i32", np.zeros(1000, np.int32), idx, vals))
    # a record built from its fields (cmd_new, rts/c/server.h:1220-1271) holds copies of them
    srv.cmd("new", "rec", "([]u32, []i32)", "keys", "vals")
    srv.cmd("store", out, "rec")
    rk, rv = fv.read_binary(out, [("u32", 1), ("i32", 1)])
    assert np.array_equal(rk, keys) and np.array_equal(rv, vals)
    with pytest.raises(ServerFailure, match="1 fields expected but 2 values provided."):
        srv.cmd("new", "r2", "([]u32, []i32)", "keys")
    with pytest.raises(ServerFailure, match=r"Field 1 mismatch: expected type \[\]i32, got \[\]u32"):
        srv.cmd("new", "r2", "([]u32, []i32)", "keys", "keys")
    with pytest.raises(ServerFailure, match="Not a record type"):
        srv.cmd("new", "r2", "[]u32", "keys")
    with pytest.raises(ServerFailure, match="Variable already exists: rec"):
        srv.cmd("new", "rec", "([]u32, []i32)", "keys", "vals")
    srv.cmd("free", "rec")
    with pytest.raises(ServerFailure, match="No such field"):
        srv.cmd("project", "x", "sorted", "2")
    with pytest.raises(ServerFailure, match="Not a sum type"):
        srv.cmd("variants", "i32")
    srv.cmd("free", "keys", "vals", "h", "is", "sorted", "sk", "sv", "hist")


@pytest.mark.gpu
def test_profiling_report_and_clear(srv):
    import json
    srv.cmd("unpause_profiling")
    report = json.loads("\n".join(srv.cmd("report")))
    assert "events" in report and "memory" in report
    srv.cmd("pause_profiling")
    srv.cmd("clear")
    srv.cmd("set_tuning_param", "segops.hist_lds_bins_max", 1024)
    with pytest.raises(ServerFailure, match="Failed to set tuning parameter nope to 3"):
        srv.cmd("set_tuning_param", "nope", 3)


@pytest.mark.gpu
def test_unknown_command_ends_the_server():
    s = Server()
    s.proc.stdin.write("frobnicate\n")
    s.proc.stdin.flush()
    assert s.proc.wait(timeout=60) == 1
    assert "Unknown command: frobnicate" in s.proc.stderr.read()
