"""LMAD copies (csrc/kernels/lmad.hip) against the element-by-element copy of
rts/c/copy.h:35-53, restated in oracle/oracle.c and pinned here by numpy's own
strided views; the flat / transpose / general classification against the cases
rts/c/copy.h:55-190 distinguishes."""
import ctypes as C

import numpy as np
import pytest

import oracle

NOTHING, FLAT, TRANSPOSE, GENERAL = 0, 1, 2, 3


def _rm(shape):
    out, acc = [], 1
    for d in reversed(shape):
        out.append(acc)
        acc *= d
    return out[::-1]


def _view_copy(src, src_offset, src_strides, shape):
    """numpy's answer: the strided view, made contiguous."""
    v = np.lib.stride_tricks.as_strided(src[src_offset:], shape=shape,
                                        strides=[s * src.itemsize for s in src_strides])
    return np.ascontiguousarray(v).reshape(-1)


@pytest.mark.parametrize("dt", [np.uint8, np.uint16, np.int32, np.float64])
def test_oracle_against_numpy_views(dt):
    rng = np.random.default_rng(3)
    for shape, perm in [((5,), (0,)), ((3, 4), (1, 0)), ((2, 3, 4), (2, 0, 1)),
                        ((2, 3, 4, 5), (3, 1, 0, 2)), ((4, 1, 6), (2, 1, 0))]:
        n = int(np.prod(shape))
        src = rng.integers(0, 200, n + 7).astype(dt)
        base = tuple(np.array(shape)[list(perm)])          # memory layout of the source
        sstr = [0] * len(shape)
        for pos, d in enumerate(perm):
            sstr[d] = _rm(base)[pos]
        dst = np.zeros(n, dt)
        oracle.lmad_copy(dst, 0, _rm(shape), src, 7, sstr, list(shape))
        assert np.array_equal(dst, _view_copy(src, 7, sstr, shape)), (shape, perm)
    # a slice with a step and a reversed dimension (negative stride), into an offset destination
    src = rng.integers(0, 200, 120).astype(dt)
    dst = np.zeros(40, dt)
    oracle.lmad_copy(dst, 4, [6, 1], src, 90, [-20, 3], [5, 6])
    want = np.zeros(40, dt)
    rows = [src[90 - 20 * i: 90 - 20 * i + 18: 3] for i in range(5)]
    want[4:34] = np.concatenate(rows)
    assert np.array_equal(dst, want)


class _K:
    def __init__(self):
        from futhark_amd import lib_path
        self.k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
        self.k.fa_lmad_copy.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int64, C.c_void_p,
                                        C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int,
                                        C.POINTER(C.c_int)]
        self.k.fa_map_transpose.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                            C.c_int64, C.c_int64, C.c_int64]


def _gpu_copy(ctx, k, dt, dst_len, dst_offset, dst_strides, src, src_offset, src_strides, shape):
    es = np.dtype(dt).itemsize
    sentinel = np.full(dst_len, 0xA5, np.uint8).repeat(es).view(dt) if es > 1 else np.full(dst_len, 0xA5, dt)
    s = ctx.new("u8_1d", src.view(np.uint8))
    d = ctx.new("u8_1d", sentinel.view(np.uint8))
    r = len(shape)
    I64 = C.c_int64 * max(r, 1)
    path = C.c_int(-1)
    rc = k.k.fa_lmad_copy(ctx.stream, es, d.device_ptr, dst_offset, I64(*dst_strides),
                          s.device_ptr, src_offset, I64(*src_strides), I64(*shape), r,
                          C.byref(path))
    assert rc == 0, rc
    got = d.values().view(dt)
    s.free(); d.free()
    want = sentinel.copy()
    oracle.lmad_copy(want, dst_offset, dst_strides, np.ascontiguousarray(src), src_offset,
                     src_strides, shape)
    return got, want, path.value


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.uint8, np.uint16, np.uint32, np.uint64])
def test_copies_match_the_oracle_and_take_the_expected_path(ctx, dt):
    k = _K()
    rng = np.random.default_rng(11)

    def data(n):
        return rng.integers(0, 255, n).astype(dt)

    cases = [
        # (shape, dst_strides, src_strides, expected path)
        ((1000,), [1], [1], FLAT),
        ((7, 9, 11), _rm((7, 9, 11)), _rm((7, 9, 11)), FLAT),
        ((5, 1, 8), [8, 8, 1], [8, 40, 1], FLAT),                       # unit dims may disagree
        ((5, 1, 8), [8, 8, 1], [8, 1, 1], TRANSPOSE),                   # ... or read as an 8x1 transpose
        ((300, 200), [200, 1], [1, 300], TRANSPOSE),                    # dst row-major, src column-major
        ((300, 200), [1, 300], [200, 1], TRANSPOSE),                    # the other way round
        ((6, 70, 90), [6300, 90, 1], [6300, 1, 70], TRANSPOSE),         # mapped over a leading dim
        ((4, 5, 6, 7), [210, 42, 7, 1], [210, 1, 35, 5], TRANSPOSE),    # (5)|(6,7) collapse
        ((3, 2000), [2000, 1], [1, 3], TRANSPOSE),                      # short rows
        ((2000, 5), [5, 1], [1, 2000], TRANSPOSE),                      # short columns
        ((20, 30, 40), _rm((20, 30, 40)), [40, 800, 1], GENERAL),       # permutation of outer dims
        ((10, 12), [12, 1], [24, 2], GENERAL),                          # strided source
        ((10, 12), [30, 2], [12, 1], GENERAL),                          # strided destination
        ((9, 4, 5), _rm((9, 4, 5)), [-20, 5, 1], GENERAL),              # reversed outer dim
        ((0, 5), [5, 1], [5, 1], NOTHING),
        ((), [], [], GENERAL),                                          # scalar: one element
    ]
    for shape, dstr, sstr, want_path in cases:
        n = int(np.prod(shape)) if shape else 1
        # room for any stride pattern above, plus offsets
        span_s = sum((abs(s) * (d - 1)) for s, d in zip(sstr, shape)) + 1 if n else 1
        span_d = sum((abs(s) * (d - 1)) for s, d in zip(dstr, shape)) + 1 if n else 1
        s_off = 3 + (sum((-s) * (d - 1) for s, d in zip(sstr, shape) if s < 0) if n else 0)
        d_off = 5
        src = data(span_s + s_off + 2)
        got, want, path = _gpu_copy(ctx, k, dt, span_d + d_off + 3, d_off, list(dstr), src, s_off,
                                    list(sstr), list(shape))
        assert path == want_path, (shape, dstr, sstr, path)
        assert np.array_equal(got, want), (shape, dstr, sstr)


@pytest.mark.gpu
def test_random_layouts(ctx):
    k = _K()
    rng = np.random.default_rng(5)
    for trial in range(60):
        r = int(rng.integers(1, 6))
        shape = [int(x) for x in rng.integers(1, 9, r)]
        if trial % 7 == 0:
            shape[int(rng.integers(0, r))] = int(rng.integers(40, 200))
        perm_s, perm_d = rng.permutation(r), rng.permutation(r)

        def strides(perm, gap):
            base = [shape[p] for p in perm]
            st = [0] * r
            acc = 1
            for pos in range(r - 1, -1, -1):
                st[perm[pos]] = acc * gap if pos == r - 1 else acc
                acc *= base[pos] * (gap if pos == r - 1 else 1)
            return st
        sstr = strides(perm_s, int(rng.integers(1, 3)))
        dstr = strides(perm_d, 1)
        dt = [np.uint8, np.uint16, np.uint32, np.uint64][trial % 4]
        span_s = sum(s * (d - 1) for s, d in zip(sstr, shape)) + 1
        span_d = sum(s * (d - 1) for s, d in zip(dstr, shape)) + 1
        src = rng.integers(0, 255, span_s + 4).astype(dt)
        got, want, _ = _gpu_copy(ctx, k, dt, span_d + 6, 2, dstr, src, 1, sstr, shape)
        assert np.array_equal(got, want), (shape, dstr, sstr)


@pytest.mark.gpu
@pytest.mark.parametrize("es", [1, 2, 4, 8])
def test_map_transpose_shapes(ctx, es):
    k = _K()
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[es]
    rng = np.random.default_rng(es)
    shapes = [(1, 1, 1), (1, 64, 64), (3, 65, 127), (2, 1, 5000), (2, 5000, 1),
              (1, 17, 4099), (1, 4099, 31), (5, 33, 33), (1, 1000, 1000)]
    if es == 4:
        # more than 65535 tiles down, and more matrices than a launch grid's second dimension holds
        shapes += [(1, 65536 * 64 + 70, 33), (70001, 3, 5), (65600, 40, 34)]
    for batch, rows, cols in shapes:
        x = rng.integers(0, 255, (batch, rows, cols)).astype(dt)
        s = ctx.new("u8_1d", x.reshape(-1).view(np.uint8))
        d = ctx.new("u8_1d", np.zeros(x.size * es, np.uint8))
        assert k.k.fa_map_transpose(ctx.stream, es, d.device_ptr, s.device_ptr, batch, rows, cols) == 0
        got = d.values().view(dt).reshape(batch, cols, rows)
        s.free(); d.free()
        assert np.array_equal(got, x.transpose(0, 2, 1)), (batch, rows, cols)
