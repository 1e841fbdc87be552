"""Value I/O (csrc/server/values.c) against the binary data format as the
reference documents and produces it: two data files held by the reference's own
tests, encodings built by hand from docs/binary-data-format.rst, round trips,
and the textual form of rts/c/values.h:398-491,724-768."""
import struct
from pathlib import Path

import numpy as np
import pytest

from futhark_amd import values as fv

GOLDEN = Path(__file__).parent / "golden"


def test_reference_file_f32_vector():
    # tests/script/data/input.in of the reference: [1f32, 2f32, 3f32]
    (xs,) = fv.read_binary(GOLDEN / "ref_tests_script_data_input.in", [("f32", 1)])
    assert xs.dtype == np.float32 and np.array_equal(xs, [1.0, 2.0, 3.0])


def test_reference_file_three_values_roundtrips_bit_exact(tmp_path):
    # tests/ad/reducebyindexminmax7.in: (is: [n]i64) (dst: [m][k]f32) (vs: [n][k]f32)
    src = GOLDEN / "ref_tests_ad_reducebyindexminmax7.in"
    is_, dst, vs = fv.read_binary(src, [("i64", 1), ("f32", 2), ("f32", 2)])
    assert is_.shape[0] == vs.shape[0] and dst.shape[1] == vs.shape[1]
    assert np.isfinite(vs).all()
    out = tmp_path / "again.in"
    fv.write_binary(out, [is_, dst, vs])
    assert out.read_bytes() == src.read_bytes()


def _encode(a: np.ndarray, tag: str) -> bytes:
    """The format, straight from the specification."""
    a = np.asarray(a, order="C")  # (ascontiguousarray would make a 0-d value 1-d)
    head = b"b" + bytes([2, a.ndim]) + tag.encode()
    dims = b"".join(struct.pack("<Q", d) for d in a.shape)
    return head + dims + a.astype(a.dtype.newbyteorder("<")).tobytes()


TAGS = {"i8": "  i8", "i16": " i16", "i32": " i32", "i64": " i64", "u8": "  u8", "u16": " u16",
        "u32": " u32", "u64": " u64", "f16": " f16", "f32": " f32", "f64": " f64", "bool": "bool"}


@pytest.mark.parametrize("name", sorted(TAGS))
@pytest.mark.parametrize("shape", [(), (0,), (5,), (2, 3), (3, 0, 2), (2, 1, 4)])
def test_writer_and_reader_match_the_specification(tmp_path, name, shape):
    rng = np.random.default_rng(hash((name, shape)) & 0xffff)
    dt = np.dtype(fv._DTYPES[name])
    if name == "bool":
        a = rng.integers(0, 2, shape).astype(np.bool_)
    elif dt.kind == "f":
        a = (rng.standard_normal(shape) * 100).astype(dt)
    else:
        info = np.iinfo(dt)
        a = rng.integers(info.min, info.max, shape, dtype=dt, endpoint=True)
    a = np.asarray(a, dtype=dt).reshape(shape)
    path = tmp_path / "v.bin"
    fv.write_binary(path, [a])
    assert path.read_bytes() == _encode(a, TAGS[name])
    path.write_bytes(b" \n\t" + _encode(a, TAGS[name]))  # leading whitespace is allowed
    (back,) = fv.read_binary(path, [(name, len(shape))])
    assert back.dtype == dt and back.shape == tuple(shape)
    assert back.tobytes() == a.tobytes()


def test_reader_rejects_what_the_reference_rejects(tmp_path):
    good = _encode(np.arange(4, dtype=np.int32), " i32")
    cases = {
        "version": b"b\x01" + good[2:],
        "type": good[:3] + b" i64" + good[7:],
        "rank": good,          # read as rank 2 below
        "truncated": good[:-3],
        "text": b"[1i32, 2i32]",
        "tag": good[:3] + b"i32 " + good[7:],
    }
    for what, blob in cases.items():
        p = tmp_path / f"{what}.bin"
        p.write_bytes(blob)
        with pytest.raises(fv.ValueError_):
            fv.read_binary(p, [("i32", 2 if what == "rank" else 1)])
    # trailing garbage after the requested values
    p = tmp_path / "extra.bin"
    p.write_bytes(good + b" x")
    with pytest.raises(fv.ValueError_):
        fv.read_binary(p, [("i32", 1)])
    assert len(fv.read_binary(p, [("i32", 1)], expect_eof=False)) == 1


def test_text_form(tmp_path):
    p = tmp_path / "t.txt"

    def text(a):
        fv.write_text(p, [a])
        return p.read_text()

    assert text(np.array([1, 2, 3], np.int32)) == "[1i32, 2i32, 3i32]"
    assert text(np.array([[1, 2], [3, 4]], np.uint8)) == "[[1u8, 2u8], [3u8, 4u8]]"
    assert text(np.array(-7, np.int64)) == "-7i64"
    assert text(np.zeros((0, 3), np.int32)) == "empty([0][3]i32)"
    assert text(np.array([True, False])) == "[true, false]"
    assert text(np.array([1.0, 0.5, 1e10], np.float32)) == "[1f32, 0.5f32, 1e+10f32]"
    assert text(np.array([np.nan, np.inf, -np.inf], np.float64)) == "[f64.nan, f64.inf, -f64.inf]"
    assert text(np.array([0.1], np.float64)) == "[0.10000000000000001f64]"
    assert text(np.array([1.5, -2.0], np.float16)) == "[1.5f16, -2f16]"
    assert text(np.array(2 ** 64 - 1, np.uint64)) == "18446744073709551615u64"


# ------------------------------------------------------------------ textual input
def _read_text(tmp_path, text, specs, **kw):
    p = tmp_path / "in.txt"
    p.write_text(text)
    return fv.read_text(p, specs, **kw)


def test_text_reader_takes_the_inputs_of_the_reference_tests(tmp_path):
    # input blocks as they stand in the reference's test programs
    (a,) = _read_text(tmp_path, "[0i8, 0i8, 0i8, 0i8, 0i8]", [("i8", 1)])          # tests/hist/i8.fut:5
    assert a.dtype == np.int8 and a.tolist() == [0] * 5
    n, is_, img = _read_text(tmp_path, "5i64\n[1, 2, 1, 4, 5]\n[1i8, 1i8, 4i8, 4i8, 4i8]",
                             [("i64", 0), ("i32", 1), ("i8", 1)])                    # tests/hist/and8.fut:24-27
    assert n == 5 and is_.tolist() == [1, 2, 1, 4, 5] and img.tolist() == [1, 1, 4, 4, 4]
    (h,) = _read_text(tmp_path, "[1f16, f16.nan, 3f16, 4f16, 5f16]", [("f16", 1)])    # tests/hist/f16.fut:32
    assert np.isnan(h[1]) and h[[0, 2, 3, 4]].tolist() == [1, 3, 4, 5]
    a, b = _read_text(tmp_path, "empty([0][1]i32) [[1]]", [("i32", 2), ("i32", 2)])   # tests/concat2.fut:10
    assert a.shape == (0, 1) and b.tolist() == [[1]]
    m, xss = _read_text(tmp_path, "10i64 [[1,2,3],[2,3,4],[3,4,5]]", [("i64", 0), ("i32", 2)])
    assert m == 10 and xss.tolist() == [[1, 2, 3], [2, 3, 4], [3, 4, 5]]              # tests/hist/segmented.fut:2


def test_text_reader_syntax(tmp_path):
    out = _read_text(tmp_path, """-- a comment line
        [[1, 2, 3], [4_000, 0x10, -6i32]]  -- trailing comment
        4.5f64 [true, false] [] [[],[]] [1.5, 2,] 017 -0x1F 18446744073709551615u64 255u8 -1u8
        [-f32.inf, f32.inf, f32.nan, 1e-3, -2.5e2f32] 1_0.5f64""",
                     [("i32", 2), ("f64", 0), ("bool", 1), ("u8", 1), ("i64", 2), ("f32", 1),
                      ("i32", 0), ("i16", 0), ("u64", 0), ("u8", 0), ("u8", 0), ("f32", 1), ("f64", 0)])
    assert out[0].tolist() == [[1, 2, 3], [4000, 16, -6]]
    assert out[1] == 4.5 and out[2].tolist() == [True, False]
    assert out[3].shape == (0,) and out[4].shape == (2, 0) and out[5].tolist() == [1.5, 2.0]
    assert out[6] == 15 and out[7] == -31 and out[8] == 2**64 - 1 and out[9] == 255 and out[10] == 255
    f = out[11]
    assert f[0] == -np.inf and f[1] == np.inf and np.isnan(f[2])
    assert f[3] == np.float32(1e-3) and f[4] == -250 and out[12] == 10.5
    for bad, spec in [("[[1, 2], [3]]", ("i32", 2)),           # rows of different length
                      ("[1, 2", ("i32", 1)), ("[1 2]", ("i32", 1)), ("[1, x]", ("i32", 1)),
                      ("[1i64]", ("i32", 1)), ("[[1]]", ("i32", 1)), ("[1]", ("i32", 2)),
                      ("empty([1]i32)", ("i32", 1)), ("empty([0]i64)", ("i32", 1)),
                      ("empty([0]i32)", ("i32", 2)), ("1.5", ("i32", 0)), ("yes", ("bool", 0)),
                      ("0x10u64", ("u64", 0)), ("", ("i32", 0)), ("f64.nan", ("f32", 0))]:
        with pytest.raises(fv.ValueError_):
            _read_text(tmp_path, bad, [spec], expect_eof=False)
    with pytest.raises(fv.ValueError_, match="end of input"):
        _read_text(tmp_path, "1 2", [("i32", 0)])


def test_f16_literals_are_cut_not_rounded(tmp_path):
    """float2halfbits (rts/c/half.h:220-228) drops the low mantissa bits: 1.2 reads as
    0x3ccc where rounding to nearest gives 0x3ccd; values that are f16 numbers read exactly."""
    (h,) = _read_text(tmp_path, "[1.2f16, 0.1f16, 65504f16, 1e5f16, 1e-8f16, 6e-8, -0.5]", [("f16", 1)])
    assert [hex(x) for x in h.view(np.uint16)] == ["0x3ccc", "0x2e66", "0x7bff", "0x7c00", "0x0",
                                                   "0x1", "0xb800"]
    rng = np.random.default_rng(4)
    f = rng.standard_normal(2000).astype(np.float32) * np.float32(10.0) ** rng.integers(-6, 5, 2000)
    (h,) = _read_text(tmp_path, "[" + ", ".join(f"{x:.9g}" for x in f) + "]", [("f16", 1)])
    with np.errstate(over="ignore"):
        rn = f.astype(np.float16)                     # round to nearest
    toward_zero = np.where(np.abs(rn.astype(np.float32)) > np.abs(f),
                           np.nextafter(rn, np.float16(0)), rn)
    assert np.array_equal(h.view(np.uint16), toward_zero.view(np.uint16))


@pytest.mark.parametrize("name", sorted(fv._DTYPES))
def test_text_round_trip_of_every_type_and_rank(tmp_path, name):
    rng = np.random.default_rng(8)
    dt = np.dtype(fv._DTYPES[name])
    for shape in [(), (7,), (3, 4), (2, 3, 2), (0,), (0, 3), (2, 0, 5)]:
        n = int(np.prod(shape, dtype=np.int64))
        if name == "bool":
            a = rng.integers(0, 2, n).astype(np.bool_)
        elif name[0] == "f":
            a = (rng.standard_normal(n) * 1000).astype(dt)
            if n > 2:
                a[0], a[1], a[2] = np.nan, np.inf, -np.inf
        else:
            ii = np.iinfo(dt)
            a = rng.integers(ii.min, ii.max, n, dtype=dt, endpoint=True)
        a = a.reshape(shape)
        p = tmp_path / "v.txt"
        fv.write_text(p, [a])
        (back,) = fv.read_text(p, [(name, len(shape))])
        assert back.shape == a.shape and back.dtype == a.dtype
        assert np.array_equal(back.view(np.uint8 if dt.itemsize == 1 else f"u{dt.itemsize}"),
                              a.view(np.uint8 if dt.itemsize == 1 else f"u{dt.itemsize}")) or \
            (name[0] == "f" and np.array_equal(back, a, equal_nan=True))
        (either,) = fv.read_values(p, [(name, len(shape))])    # the detecting reader takes text ...
        assert np.array_equal(either, back, equal_nan=name[0] == "f")
        fv.write_binary(p, [a])
        (either,) = fv.read_values(p, [(name, len(shape))])    # ... and binary
        assert np.array_equal(either, a, equal_nan=name[0] == "f")


def test_end_of_input_check_leaves_the_next_value_in_the_stream(tmp_path):
    """Asking whether the input has ended must not eat what follows: blanks and comments are
    skipped, a value (also one starting with a minus sign) is still there for the next read."""
    import ctypes as C
    L = fv._get()
    p = tmp_path / "in.txt"
    p.write_text("  -- a comment\n -7i32 -- another\n[1, 2] -- last\n")
    f = fv._open(p, b"rb")
    try:
        got = []
        for name, rank in (("i32", 0), ("i32", 1)):
            assert L.v.fv_end_of_input(f) != 0
            assert L.v.fv_end_of_input(f) != 0   # asking twice changes nothing
            shape, data, err = (C.c_int64 * fv.MAX_RANK)(), C.c_void_p(), C.create_string_buffer(256)
            rc = L.v.fv_read_value(f, L.v.fv_primtype(name.encode()), rank, shape, C.byref(data), err, len(err))
            assert rc == 0, err.value
            n = shape[0] if rank else 1
            got.append(np.frombuffer(C.string_at(data, 4 * n), np.int32).tolist())
            L.c.free(data)
        assert got == [[-7], [1, 2]]
        assert L.v.fv_end_of_input(f) == 0
    finally:
        L.c.fclose(f)
