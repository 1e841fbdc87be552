"""Every entry point of the program, once, through both of its callers: the C API (ctypes) and
the server's table (restore / call / store over the pipe).  The two must return the same bytes,
and a handful of families are also checked against the oracle, so a wrongly wired entry (argument
order, array rank, element type, number of inputs) cannot hide behind the entries the other tests
happen to use.  Values are small whole numbers, so that float sums are exact in any order."""
import json
from pathlib import Path

import numpy as np
import pytest

import oracle
from futhark_amd import values as fv
from futhark_amd.capi import OPAQUE_PAIRS
from futhark_amd.server import Server

pytestmark = pytest.mark.gpu

MANIFEST = json.loads((Path(__file__).resolve().parent.parent / "include" / "segops.json").read_text())
NP = {"i8": np.int8, "u8": np.uint8, "i16": np.int16, "u16": np.uint16, "i32": np.int32,
      "u32": np.uint32, "i64": np.int64, "u64": np.uint64, "f16": np.float16, "f32": np.float32,
      "f64": np.float64}
N = 37


def _vals(rng, t, shape):
    dt = NP[t]
    lo = 0 if t[0] == "u" else -5
    return rng.integers(lo, 9, shape).astype(dt)


def make_inputs(name, e, rng):
    """One numpy value per input of the entry, with shapes that fit together."""
    types = [i["type"] for i in e["inputs"]]
    el = lambda ty: ty.lstrip("[]")
    fam = name.split("_")[0]
    if name in ("segreduce_compose_i32", "scanrows_argmax_i32"):
        return [np.array(4, np.int64), _vals(rng, "i32", (36, 2))]       # nine rows of four
    if name == "segred_argmax_i32":
        return [np.array([0, 10, 10, 30], np.int64), np.array([10, 0, 20, 7], np.int64),
                _vals(rng, "i32", (N, 2))]
    if name.startswith("rbi_vec"):
        t = el(types[0])
        return [_vals(rng, t, (5, 3)), rng.integers(-1, 6, N).astype(np.int64), _vals(rng, t, (N, 3))]
    if name.startswith("rbi_2d"):
        t = el(types[0])
        return [_vals(rng, t, (4, 5)), rng.integers(-1, 5, N).astype(np.int64),
                rng.integers(-1, 6, N).astype(np.int64), _vals(rng, t, N)]
    if name.endswith("compose_i32") or name == "scan_argmax_i32":
        ab = _vals(rng, "i32", (N, 2))
        return ([(rng.random(N) < 0.2).astype(np.uint8)] if fam == "segscan" else []) + [ab]
    if name == "hist_argmax_i32":
        return [np.array(5, np.int64), rng.integers(-1, 7, N).astype(np.int32), _vals(rng, "i32", N)]
    if name in ("sumsq_f32", "scan_norm_f32", "reduce_summax_f32"):
        return [_vals(rng, "f32", N)]
    if name == "rows_fraction_f32":
        return [np.abs(_vals(rng, "f32", (6, 7))) + np.float32(1)]
    if fam in ("reduce", "scan", "exscan"):
        return [_vals(rng, el(types[0]), N)]
    if fam == "segscan":
        return [(rng.random(N) < 0.2).astype(np.uint8), _vals(rng, el(types[1]), N)]
    if fam == "segred":
        lens = np.array([10, 0, 20, 7], np.int64)
        return [np.array([0, 10, 10, 30], np.int64), lens, _vals(rng, el(types[2]), N)]
    if fam in ("segreduce", "scanrows", "vecreduce", "vecscan"):
        return [_vals(rng, el(types[0]), (6, 7))]
    if fam == "hist":
        return [np.array(5, np.int64), rng.integers(-1, 7, N).astype(NP[el(types[1])]),
                _vals(rng, el(types[2]), N)]
    if fam == "rbi":
        t = el(types[0])
        return [_vals(rng, t, 5), rng.integers(-1, 7, N).astype(NP[el(types[1])]), _vals(rng, t, N)]
    if fam == "seghist":
        return [np.array(5, np.int64), rng.integers(-1, 7, (3, N)).astype(np.int32),
                _vals(rng, el(types[2]), (3, N))]
    if fam == "bmm":
        t = el(types[0])
        a, b = rng.integers(-3, 4, (2, 4, 8)), rng.integers(-3, 4, (2, 8, 4))
        if t == "f32":
            return [a.astype(np.float32), b.astype(np.float32)]
        if t == "f16":
            return [a.astype(np.float16), b.astype(np.float16)]
        bf16 = lambda x: (x.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        return [bf16(a), bf16(b)]
    if fam == "matmul":
        return [rng.integers(-3, 4, (4, 8)).astype(np.float32), rng.integers(-3, 4, (8, 4)).astype(np.float32)]
    if fam == "radix":
        k = NP[el(types[0])]
        keys = rng.integers(0, 50, N).astype(k)
        return [keys] + ([np.arange(N, dtype=np.int32)] if len(types) == 2 else [])
    if fam == "iota":
        return [np.array(9, np.int64)]
    if fam == "replicate":
        return [np.array(9, np.int64), np.array(-4, np.int32)]
    if fam == "transpose":
        return [_vals(rng, "f32", (3, 5))]
    raise AssertionError(f"no inputs known for entry point {name}")


def _kind(ty):
    """Manifest type -> what Context.call / Context.new name it."""
    if ty.startswith("("):
        a, b = [x.strip().lstrip("[]") for x in ty.strip("()").split(",")]
        return next(k for k, v in OPAQUE_PAIRS.items() if v == (a, b))
    rank = ty.count("[]")
    return f"{ty.lstrip('[]')}_{rank}d" if rank else NP[ty]


def _spec(ty):
    """Manifest type -> the (element type, rank) pairs fv.read_binary wants."""
    if ty.startswith("("):
        return [(x.strip().lstrip("[]"), x.count("[]")) for x in ty.strip("()").split(",")]
    return [(ty.lstrip("[]"), ty.count("[]"))]


def _bits(x):
    x = np.asarray(x)
    return x.view(np.uint16) if x.dtype == np.float16 else x


@pytest.fixture(scope="module")
def server():
    s = Server()
    yield s
    s.close()


def test_every_entry_point_through_the_c_api_and_the_server(ctx, server, tmp_path):
    rng = np.random.default_rng(1)
    checked = 0
    for name, e in MANIFEST["entry_points"].items():
        ins = make_inputs(name, e, rng)
        assert len(ins) == len(e["inputs"]), name
        # -- the server: restore, call, store
        f_in, f_out = tmp_path / "in.bin", tmp_path / "out.bin"
        fv.write_binary(f_in, ins)
        names = [f"in{i}" for i in range(len(ins))]
        server.cmd("restore", f_in, *[w for n_, i in zip(names, e["inputs"]) for w in (n_, i["type"])])
        server.call(name, "out", *names)
        server.cmd("store", f_out, "out")
        via_server = fv.read_binary(f_out, _spec(e["output"]["type"]))
        server.cmd("free", "out", *names)
        # -- the C API
        args, held = [], []
        for x, i in zip(ins, e["inputs"]):
            k = _kind(i["type"])
            if isinstance(k, str):
                held.append(ctx.new(k, _bits(x)))
                args.append(held[-1])
            else:
                args.append(x.item())
        out = ctx.call(name, [_kind(e["output"]["type"])], *args)
        if e["output"]["type"].startswith("("):
            fields = [out.project(0), out.project(1)]
            via_api = [f.values() for f in fields]
            for f in fields:
                f.free()
            out.free()
        elif e["output"]["type"].startswith("["):
            via_api = [out.values()]
            out.free()
        else:
            via_api = [np.asarray(out)]
        for h in held:
            h.free()
        assert len(via_api) == len(via_server), name
        for a, b in zip(via_api, via_server):
            a, b = _bits(a), _bits(b)
            assert a.shape == b.shape and a.tobytes() == b.tobytes(), name
        # -- a few families against the oracle as well (exact: whole numbers)
        fam, parts = name.split("_")[0], name.split("_")
        if fam in ("vecreduce", "segreduce") and parts[1] not in ("argmax", "compose") \
                and parts[2] in ("i32", "i64", "f32", "f64"):
            want = getattr(oracle, fam)(parts[1], parts[2], ins[0])
            assert np.array_equal(via_api[0], want), name
        if name.startswith("rbi_2d"):
            assert np.array_equal(via_api[0], oracle.rbi_2d(parts[2], parts[3], *ins)), name
        if name.startswith("rbi_vec"):
            assert np.array_equal(via_api[0], oracle.rbi_vec(parts[2], parts[3], *ins)), name
        if fam in ("hist", "rbi") and parts[1] != "argmax" and parts[-1] == "i64" and len(parts) == 4 \
                and parts[2] in ("i32", "i64", "f32", "f64"):
            # the []i64 forms against the oracle, which takes 32-bit indices
            narrow = [ins[0], ins[1].astype(np.int32), ins[2]]
            want = oracle.hist(parts[1], parts[2], int(ins[0]), *narrow[1:]) if fam == "hist" \
                else oracle.rbi(parts[1], parts[2], *narrow)
            assert np.array_equal(via_api[0], want), name
        if name in ("segreduce_argmax_i32", "segreduce_compose_i32", "scanrows_argmax_i32",
                    "segred_argmax_i32"):
            assert np.array_equal(via_api[0], getattr(oracle, name)(*[x.item() if x.ndim == 0 else x
                                                                      for x in ins])), name
        checked += 1
    assert checked == len(MANIFEST["entry_points"]) > 300
