"""futhark_amd/bin/segops, the command-line executable of the program
(src/Futhark/CodeGen/Backends/GenericC/CLI.hs): arguments on standard input in
either value syntax, the result on standard output, run times in a file."""
import subprocess
from pathlib import Path

import numpy as np
import pytest

import oracle
from futhark_amd import values as fv

pytestmark = pytest.mark.gpu
CLI = Path(__file__).resolve().parent.parent / "futhark_amd" / "bin" / "segops"


def run(args, stdin=b"", check=True):
    p = subprocess.run([str(CLI), *args], input=stdin, capture_output=True, timeout=120)
    if check:
        assert p.returncode == 0, p.stderr.decode()
    return p


def test_text_in_text_out():
    p = run(["-e", "scan_add_i32"], b"[1, 2, 3, 4]  -- the argument\n")
    assert p.stdout.decode() == "[1i32, 3i32, 6i32, 10i32]\n"
    p = run(["-e", "reduce_max_f32"], b"[1.5, -2, f32.nan, 7.25f32]")
    assert p.stdout.decode() == "7.25f32\n"
    p = run(["--entry-point=hist_add_i64"], b"4i64 [0, 3, 3, 9, -1] [10i64, 20i64, 30i64, 40i64, 50i64]")
    assert p.stdout.decode() == "[10i64, 0i64, 0i64, 50i64]\n"
    p = run(["-e", "scan_add_f64"], b"empty([0]f64)")
    assert p.stdout.decode() == "empty([0]f64)\n"
    p = run(["-e", "seghist_add_i32"], b"10i64 [[1,2,3],[2,3,4],[3,4,5]] [[1,1,1],[1,1,1],[1,1,1]]")
    rows = ["[" + ", ".join(f"{int(j in r)}i32" for j in range(10)) + "]"
            for r in ([1, 2, 3], [2, 3, 4], [3, 4, 5])]
    assert p.stdout.decode() == "[" + ", ".join(rows) + "]\n"      # tests/hist/segmented.fut:3-7


def test_entries_with_shaped_operators_take_the_inputs_of_the_reference_tests():
    # tests/hist/array.fut:3-4
    p = run(["-e", "rbi_vec_add_i32"],
            b"[[1,2,3],[4,5,6]] [0i64,0i64,2i64,1i64] [[0,1,2],[0,1,2],[0,1,2],[0,1,2]]")
    assert p.stdout.decode() == "[[1i32, 4i32, 7i32], [4i32, 6i32, 8i32]]\n"
    # tests/hist/hist2d.fut:2-3, four inputs
    p = run(["-e", "rbi_2d_add_i32"],
            b"[[1,2,3],[4,5,6],[7,8,9]] [1i64, 1i64] [1i64, -1i64] [42, 1337]")
    assert p.stdout.decode() == "[[1i32, 2i32, 3i32], [4i32, 47i32, 6i32], [7i32, 8i32, 9i32]]\n"
    p = run(["-e", "vecreduce_add_i32"], b"[[1,2,3],[4,5,6]]")
    assert p.stdout.decode() == "[5i32, 7i32, 9i32]\n"
    p = run(["-e", "scan_compose_i32"], b"[[2,3],[5,7],[1,1]]")   # 5(2x+3)+7 = 10x+22, then +1
    assert p.stdout.decode() == "[[2i32, 3i32], [10i32, 22i32], [10i32, 23i32]]\n"


def test_tuple_result_prints_one_field_per_line():
    p = run(["-e", "radix_sort_pairs_u32_i32"], b"[5u32, 1u32, 5u32, 0u32] [0, 1, 2, 3]")
    assert p.stdout.decode() == "[0u32, 1u32, 5u32, 5u32]\n[3i32, 1i32, 0i32, 2i32]\n"


def test_binary_in_and_out_runs_and_runtime_file(tmp_path):
    rng = np.random.default_rng(2)
    flags = (rng.random(100000) < 0.01).astype(np.uint8)
    vs = rng.standard_normal(100000).astype(np.float32)
    inp = tmp_path / "in.bin"
    fv.write_binary(inp, [flags, vs])
    times = tmp_path / "times.txt"
    p = run(["-e", "segscan_max_f32", "-b", "-r", "3", "-t", str(times)], inp.read_bytes())
    out = tmp_path / "out.bin"
    out.write_bytes(p.stdout)
    (got,) = fv.read_binary(out, [("f32", 1)])
    assert np.array_equal(got, oracle.segscan("max", "f32", flags, vs))
    runs = [int(l) for l in times.read_text().split()]
    assert len(runs) == 3 and all(0 < t < 10_000_000 for t in runs)   # the warm-up run is not timed
    p = run(["-e", "segscan_max_f32", "-n"], inp.read_bytes())
    assert p.stdout == b""
    # a mix: first argument binary, second textual
    mixed = tmp_path / "mixed"
    fv.write_binary(mixed, [np.array([1, 0, 1], np.uint8)])
    p = run(["-e", "segscan_add_i32"], mixed.read_bytes() + b" [5, 6, 7]")
    assert p.stdout.decode() == "[5i32, 11i32, 7i32]\n"


def test_errors():
    p = run(["-e", "nope"], check=False)
    assert p.returncode == 1 and b"No entry point 'nope'.  Select another with --entry-point." in p.stderr
    assert b"scan_add_i32\n" in p.stderr
    p = run([], check=False)                                          # the default entry point is main
    assert p.returncode == 1 and b"No entry point 'main'" in p.stderr
    p = run(["-e", "scan_add_i32"], b"[1, 2] [3]", check=False)
    assert p.returncode == 1 and b'Expected EOF on stdin after reading input for "scan_add_i32".' in p.stderr
    p = run(["-e", "scan_add_i32"], b"[1.5]", check=False)
    assert p.returncode == 1 and b"Cannot read input #0 of type []i32" in p.stderr
    p = run(["-e", "hist_add_i32"], b"[1] [1] [1]", check=False)
    assert p.returncode == 1 and b"Error when reading input #0 of type i64" in p.stderr
    p = run(["-e", "segscan_add_i32"], b"[1u8, 0u8] [1, 2, 3]", check=False)
    assert p.returncode == 1 and b"invalid sizes" in p.stderr
    p = run(["-r", "0", "-e", "scan_add_i32"], b"[1]", check=False)
    assert p.returncode == 1 and b"Need a positive number of runs, not 0" in p.stderr
    p = run(["--param", "nope=3", "-e", "scan_add_i32"], b"[1]", check=False)
    assert p.returncode == 1 and b"Unknown tuning parameter: nope" in p.stderr
    p = run(["-e", "scan_add_i32", "extra"], b"[1]", check=False)
    assert p.returncode == 1 and b"Excess non-option: extra" in p.stderr


def test_options_that_need_no_input():
    assert run(["--print-params"]).stdout.decode().splitlines() == [
        "segops.hist_lds_bins_max (shared_memory)", "segops.segred_small_threshold (threshold)",
        "segops.matmul_pad_min_work (threshold)", "segops.scan_arrival_tickets (threshold)",
        "segops.sort_wide_positions (threshold)"]
    assert run(["-h"]).stdout.decode().startswith("Usage: ")
    p = run(["-e", "reduce_add_i32", "-P", "--param", "segops.hist_lds_bins_max=1024"], b"[1, 2, 3]")
    assert p.stdout.decode() == "6i32\n" and b'"events"' in p.stderr
