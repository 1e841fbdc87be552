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
