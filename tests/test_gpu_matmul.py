"""GPU parity: tiled SegMap (batched matmul) through the generated-library API.

Tolerance: |got - ref| <= tol * sum_k |a_ik||b_kj| per output, ref accumulated in
f64; tol = 1e-5 for f32 inputs and 1e-2 for f16/bf16 inputs (f32 accumulate).
The bound is relative to the magnitude of the summands because a dot product
of zero-mean data can be arbitrarily close to zero."""
import numpy as np
import pytest

import oracle
from futhark_amd import datagen as dg

pytestmark = pytest.mark.gpu


def _inputs(t, b, M, N, K, aid=60):
    sc = 1.0 / np.sqrt(max(K, 1))
    A = dg.normal_f32(aid, b * M * K, sc).reshape(b, M, K)
    B = dg.normal_f32(aid + 1, b * K * N, sc).reshape(b, K, N)
    if t == "f32":
        return A, B, A, B, "f32_3d"
    if t == "f16":
        Ab, Bb = dg.to_f16_bits(A), dg.to_f16_bits(B)
        return Ab, Bb, oracle.widen(Ab, "f16"), oracle.widen(Bb, "f16"), "f16_3d"
    Ab, Bb = dg.to_bf16_bits(A), dg.to_bf16_bits(B)
    return Ab, Bb, oracle.widen(Ab, "bf16"), oracle.widen(Bb, "bf16"), "u16_3d"


def _check(got, Af, Bf, tol):
    ref = np.matmul(Af.astype(np.float64), Bf.astype(np.float64))
    scale = np.matmul(np.abs(Af).astype(np.float64), np.abs(Bf).astype(np.float64))
    err = np.abs(got.astype(np.float64) - ref)
    assert np.all(err <= tol * scale + 1e-30), float((err / (scale + 1e-30)).max())


@pytest.mark.parametrize("t,tol", [("f32", 1e-5), ("f16", 1e-2), ("bf16", 1e-2)])
def test_shapes(ctx, t, tol):
    for b, M, N, K in [(1, 2, 2, 3), (3, 17, 29, 13), (2, 64, 64, 64), (1, 100, 70, 130),
                       (1, 256, 256, 32), (1, 256, 256, 64), (2, 256, 512, 96), (1, 512, 256, 512),
                       (1, 128, 128, 64), (3, 384, 128, 192), (1, 640, 896, 128),  # 128 x 128 tiles
                       (1, 5, 7, 0), (0, 4, 4, 4)]:
        Ain, Bin, Af, Bf, kind = _inputs(t, b, M, N, K)
        out = ctx.call(f"bmm_{t}", ["f32_3d"], ctx.new(kind, Ain), ctx.new(kind, Bin))
        got = out.values()
        assert got.shape == (b, M, N)
        _check(got, Af, Bf, tol)


def test_reference_golden(ctx, goldens):
    c = goldens["mmm"]["cases"][0]
    out = ctx.call("matmul_f32", ["f32_2d"], ctx.new("f32_2d", np.array(c["A"], np.float32)),
                   ctx.new("f32_2d", np.array(c["B"], np.float32)))
    assert out.values().tolist() == c["out"]


def test_structured_operands_catch_transposition(ctx):
    # A = row index, B = one-hot columns: any swap of operands or indices shows.
    M = N = 256
    K = 64
    A = (np.arange(M)[:, None] * 0.5 + np.arange(K)[None, :] * 0.125).astype(np.float32)
    B = np.zeros((K, N), np.float32)
    B[np.arange(N) % K, np.arange(N)] = 1.0
    B[(np.arange(N) * 7 + 3) % K, np.arange(N)] += 2.0
    want = A.astype(np.float64) @ B.astype(np.float64)
    for t, kind in (("f32", "f32_3d"), ("f16", "f16_3d"), ("bf16", "u16_3d")):
        cvt = {"f32": lambda x: x, "f16": dg.to_f16_bits, "bf16": dg.to_bf16_bits}[t]
        out = ctx.call(f"bmm_{t}", ["f32_3d"], ctx.new(kind, cvt(A)[None]), ctx.new(kind, cvt(B)[None]))
        got = out.values()[0]
        if t == "bf16":  # A is not exactly representable in bf16
            Aw = oracle.widen(dg.to_bf16_bits(A), "bf16").astype(np.float64)
            np.testing.assert_allclose(got, Aw @ B.astype(np.float64), rtol=1e-6)
        else:
            np.testing.assert_allclose(got, want, rtol=1e-6)


@pytest.mark.parametrize("t,tol", [("f32", 1e-5), ("f16", 1e-2), ("bf16", 1e-2)])
@pytest.mark.parametrize("b,m", [(1, 4096), (64, 512)])
def test_config4_full_size(ctx, t, tol, b, m):
    Ain, Bin, Af, Bf, kind = _inputs(t, b, m, m, m, 64)
    out = ctx.call(f"bmm_{t}", ["f32_3d"], ctx.new(kind, Ain), ctx.new(kind, Bin))
    got = out.values()
    # full oracle on a sample of rows (the CPU triple loop over 4096^3 takes minutes)
    rows = np.array([0, 1, 31, 32, 127, 128, 255, 256, m // 2 + 3, m - 1])
    for q in (0, b - 1):
        _check(got[q][rows], Af[q][rows], Bf[q], tol)
    # size-independent property: linearity in the row sums, C 1 = A (B 1)
    lhs = got.astype(np.float64).sum(axis=2)
    rhs = np.matmul(Af.astype(np.float64), Bf.astype(np.float64).sum(axis=2)[..., None])[..., 0]
    scale = np.matmul(np.abs(Af).astype(np.float64), np.abs(Bf).astype(np.float64).sum(axis=2)[..., None])[..., 0]
    assert np.all(np.abs(lhs - rhs) <= tol * scale)


@pytest.mark.parametrize("t,tol", [("f32", 1e-5), ("f16", 1e-2), ("bf16", 1e-2)])
def test_ragged_shapes_through_padded_operands(ctx, t, tol):
    """Shapes that are no multiples of the MFMA tile but large enough to run on
    zero-padded copies; every output element is checked, and the report says
    which way the product went."""
    import json
    from futhark_amd import Context
    with Context(ctx.so, profiling=True) as c:
        shapes = [(1, 300, 500, 200, True), (3, 257, 255, 129, True), (1, 1000, 1000, 1000, True),
                  (4, 256, 256, 100, True), (1, 511, 256, 192, True), (1, 2011, 515, 777, True),
                  (1, 255, 256, 64, False),     # too little work to pay for the copies
                  (1, 2000, 3, 2000, False)]    # padding would multiply the work by 85
        for b, M, N, K, _ in shapes:
            Ain, Bin, Af, Bf, kind = _inputs(t, b, M, N, K, 66)
            out = c.call(f"bmm_{t}", ["f32_3d"], c.new(kind, Ain), c.new(kind, Bin))
            got = out.values()
            assert got.shape == (b, M, N)
            _check(got, Af, Bf, tol)
            out.free()
        ev = [e for e in json.loads(c.report())["events"] if e["name"] == "segmap_matmul"]
        assert [e["details"]["padded"] for e in ev] == [p for *_, p in shapes], ev


def test_padded_operands_with_more_than_65535_rows(ctx):
    """K beyond the 65535 a launch grid's second dimension holds, and off the
    k-step: the copy into padded operands must walk rows, not give a launch error."""
    b, M, N, K = 1, 300, 260, 70001
    Ain, Bin, Af, Bf, kind = _inputs("f16", b, M, N, K, 68)
    out = ctx.call("bmm_f16", ["f32_3d"], ctx.new(kind, Ain), ctx.new(kind, Bin))
    got = out.values()
    assert got.shape == (b, M, N)
    _check(got, Af, Bf, 1e-2)
    # M beyond it as well (f32, tall and thin, large enough for the padded path)
    b, M, N, K = 1, 70003, 250, 60
    Ain, Bin, Af, Bf, kind = _inputs("f32", b, M, N, K, 69)
    got = ctx.call("bmm_f32", ["f32_3d"], ctx.new(kind, Ain), ctx.new(kind, Bin)).values()
    _check(got, Af, Bf, 1e-5)


def test_more_tile_rows_than_a_launch_grid_holds(ctx):
    """M / 128 above 65535 tile rows (f16, one matrix): the product goes out in bands of rows.
    The rows of A repeat with period 384, so every row of C repeats too: the first period is
    checked against the oracle and the rest against the first period."""
    M, N, K, period = 65537 * 128, 128, 64, 384
    Ain, Bin, Af, Bf, kind = _inputs("f16", 1, period, N, K, 70)
    reps = M // period + 1
    A_all = np.tile(Ain[0], (reps, 1))[:M][None]
    out = ctx.call("bmm_f16", ["f32_3d"], ctx.new(kind, np.ascontiguousarray(A_all)), ctx.new(kind, Bin))
    got = out.values()[0]
    out.free()
    assert got.shape == (M, N)
    _check(got[:period][None], Af, Bf, 1e-2)
    first = got[:period]
    whole = (M // period) * period
    assert np.array_equal(got[:whole].reshape(-1, period, N), np.broadcast_to(first, (M // period, period, N)))
    assert np.array_equal(got[whole:], first[: M - whole])
