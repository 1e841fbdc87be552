#!/usr/bin/env python3
"""Benchmark of the SegOp hot path on one MI355X.

Default workload: segmented inclusive scan with (+) over 2^26 f32 values in
irregular segments (geometric lengths, mean 1024, u8 start flags) -- the
configuration the headline metric is quoted on.  One step = one
futhark_entry_* call (one pass of the path over the resident input) followed
by freeing its result; inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is whole-job throughput in GB/s over the
algorithmic bytes of the workload; `roofline` prices the dominant kernel with
HIP events recorded on the context's stream; `cpu_baseline` times the
futhark-multicore-style CPU restatement (oracle/multicore.c) on the host cores.
Other workloads (--workload) report the same fields for the other SegOps.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}


def make_workload(name: str, ctx):
    """Returns dict(step, bytes, unit_work, dtype, kernel, cpu, describe, bound)."""
    from futhark_amd import datagen as dg
    import oracle

    w = {}
    if name.startswith("segscan_") or name.startswith("segred_"):
        kind, op, t, sz = name.split("_")
        n = 1 << int(sz[2:])
        w["elements"] = n
        es = 4 if t == "f32" else 8
        offsets, lens, flags = dg.segments(32, n, 1024)
        xs = dg.uniform_f32(33, n) if t == "f32" else dg.uniform_int(34, n, -(1 << 20), 1 << 20, np.int64)
        v = ctx.new(f"{t}_1d", xs)
        if kind == "segscan":
            f = ctx.new("u8_1d", flags)

            def step():
                ctx.call(f"segscan_{op}_{t}", [f"{t}_1d"], f, v).free()
            w["bytes"] = n * (2 * es + 1)
            w["kernel"] = "segscan"
            if t in ("f32", "i64"):
                w["cpu"] = lambda out=np.empty_like(xs): oracle.mc_segscan(t, flags, xs, op, out=out)
                # the sequential `futhark c` fold (the oracle proper) on the first 2^24 elements
                w["cpu_seq"] = (lambda: oracle.segscan(op, t, flags[:1 << 24], xs[:1 << 24]),
                                (1 << 24) * (2 * es + 1))
        else:
            o, l = ctx.new("i64_1d", offsets), ctx.new("i64_1d", lens)

            def step():
                ctx.call(f"segred_{op}_{t}", [f"{t}_1d"], o, l, v).free()
            w["bytes"] = n * es + len(offsets) * (8 + es)
            w["kernel"] = "segred_irregular"
            if t == "f32" and op == "add":
                tmp = (np.empty(n, np.uint8), np.empty(n, np.float32))
                w["cpu"] = lambda: oracle.mc_segred_add_f32(offsets, lens, xs, tmp=tmp)
                w["cpu_how"] = ("segmented scan with flags written from the offsets, then one read "
                                "per segment (what flattening makes of it)")
        w.update(step=step, dtype=t, bound="hbm", keep=[v],
                 describe=f"{kind} ({op}) over 2^{sz[2:]} {t}, {len(offsets)} irregular segments "
                          f"(geometric, mean 1024), u8 flags / i64 offsets")
    elif name.startswith("reduce_") or name.startswith("scan_"):
        kind, op, t, sz = name.split("_")
        n = 1 << int(sz[2:])
        w["elements"] = n
        es = 4
        xs = dg.uniform_f32(17, n) if t == "f32" else dg.uniform_int(16, n, -1000, 1000)
        a = ctx.new(f"{t}_1d", xs)
        if kind == "reduce":
            nt = np.float32 if t == "f32" else np.int32

            import ctypes as C
            entry = getattr(ctx.L, f"futhark_entry_reduce_{op}_{t}")
            result = np.zeros(1, nt)
            result_p = result.ctypes.data_as(C.c_void_p)

            def step():
                # The scalar arrives at the synchronisation that ends the timed loop
                # (docs/c-api.rst:578-581), like the arrays of the other workloads.
                ctx.check(entry(ctx.ptr, result_p, a.ptr))
            w["result"] = result
            w["bytes"] = n * es
            w["kernel"] = "segred_nonseg"
            w["cpu"] = lambda: oracle.mc_reduce_add(t, xs)
        else:
            def step():
                ctx.call(f"scan_{op}_{t}", [f"{t}_1d"], a).free()
            w["bytes"] = 2 * n * es
            w["kernel"] = "segscan"
            w["cpu"] = lambda out=np.empty_like(xs): oracle.mc_segscan(t, None, xs, op, out=out)
        w.update(step=step, dtype=t, bound="hbm", keep=[a],
                 describe=f"{kind} ({op}) over 2^{sz[2:]} {t}")
    elif name.startswith("hist_"):
        # hist_add_i32_H65536_uniform_2p27
        _, op, t, hs, dist, sz = name.split("_")
        n, H = 1 << int(sz[2:]), int(hs[1:])
        w["elements"] = n
        is_ = dg.hist_indices(48, n, H, dist)
        if t == "f16":
            vs, es = dg.to_f16_bits(dg.uniform_f32(50, n)), 2
        elif t[0] == "f":
            vs = dg.uniform_f32(50, n).astype(np.dtype(f"float{t[1:]}"))
            es = vs.itemsize
        else:
            dt = np.dtype(("int" if t[0] == "i" else "uint") + t[1:])
            lo, hi = (-1000, 1000) if dt.itemsize >= 4 and t[0] == "i" else (0, 100)
            vs = dg.uniform_int(49, n, lo, hi).astype(dt)
            es = dt.itemsize
        i, v = ctx.new("i32_1d", is_), ctx.new(f"{t}_1d", vs)

        def step():
            ctx.call(f"hist_{op}_{t}", [f"{t}_1d"], H, i, v).free()
        w.update(step=step, bytes=n * (4 + es) + 2 * H * es, kernel="seghist", dtype=t, bound="hbm",
                 keep=[i, v], describe=f"hist ({op}) of 2^{sz[2:]} {t} into {H} bins, {dist} i32 "
                                       f"indices, 1% out of range")
        if t == "i32" and op == "add":
            w["cpu"] = lambda: oracle.mc_rbi_add_i32(np.zeros(H, np.int32), is_, vs)
        elif t == "f32" and op in ("add", "max"):
            ne = np.float32(0.0 if op == "add" else -np.inf)
            w["cpu"] = lambda: oracle.mc_rbi_f32(op, np.full(H, ne, np.float32), is_, vs)
        w["cpu_how"] = "a private sub-histogram per task, then a reduce over the tasks per bin"
    elif name.startswith("rbivec_"):
        # rbivec_add_i32_H256x16_2p23: 2^23 updates of 16-element vectors into [256][16] bins
        _, op, t, hs, sz = name.split("_")
        n = 1 << int(sz[2:])
        H, m = (int(x) for x in hs[1:].split("x"))
        w["elements"] = n * m
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        is_ = dg.hist_indices(52, n, H, "uniform").astype(np.int64)
        vss = (dg.uniform_f32(53, n * m) if t[0] == "f" else dg.uniform_int(54, n * m, -1000, 1000)
               ).astype(dt).reshape(n, m)
        d, i, v = ctx.new(f"{t}_2d", np.zeros((H, m), dt)), ctx.new("i64_1d", is_), ctx.new(f"{t}_2d", vss)

        def step():
            ctx.call(f"rbi_vec_{op}_{t}", [f"{t}_2d"], d, i, v).free()
        es = dt().itemsize
        w.update(step=step, bytes=n * 8 + n * m * es + 2 * H * m * es, kernel="seghist_shaped",
                 dtype=t, bound="hbm", keep=[d, i, v],
                 describe=f"reduce_by_index with operator map2 {op}: 2^{sz[2:]} vectors of {m} {t} "
                          f"into [{H}][{m}] bins, uniform i64 indices, 1% out of range")
    elif name.startswith("rbi2d_"):
        # rbi2d_add_i32_256x256_2p27: reduce_by_index_2d into [256][256] bins
        _, op, t, hs, sz = name.split("_")
        n = 1 << int(sz[2:])
        H0, H1 = (int(x) for x in hs.split("x"))
        w["elements"] = n
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        is_ = dg.hist_indices(55, n, H0, "uniform").astype(np.int64)
        js = dg.hist_indices(56, n, H1, "uniform").astype(np.int64)
        vs = (dg.uniform_f32(57, n) if t[0] == "f" else dg.uniform_int(58, n, -1000, 1000)).astype(dt)
        d = ctx.new(f"{t}_2d", np.zeros((H0, H1), dt))
        i, j, v = ctx.new("i64_1d", is_), ctx.new("i64_1d", js), ctx.new(f"{t}_1d", vs)

        def step():
            ctx.call(f"rbi_2d_{op}_{t}", [f"{t}_2d"], d, i, j, v).free()
        es = dt().itemsize
        w.update(step=step, bytes=n * (16 + es) + 2 * H0 * H1 * es, kernel="seghist_shaped", dtype=t,
                 bound="hbm", keep=[d, i, j, v],
                 describe=f"reduce_by_index_2d ({op}) of 2^{sz[2:]} {t} into [{H0}][{H1}] bins, "
                          f"uniform i64 index pairs, 1% out of range per coordinate")
    elif name.startswith("sort_"):
        # sort_u32_2p26 | sort_u64i32_2p26
        _, kt, sz = name.split("_")
        n = 1 << int(sz[2:])
        w["elements"] = n
        if kt == "u32":
            keys = dg.uniform_u32(80, n)
            k = ctx.new("u32_1d", keys)
            w["cpu"] = lambda: oracle.mc_radix_sort(keys)

            def step():
                ctx.call("radix_sort_u32", ["u32_1d"], k).free()
            w.update(bytes=4 * 12 * n, keep=[k])
        else:
            keys, idx = dg.uniform_u64(81, n), np.arange(n, dtype=np.int32)
            k = ctx.new("u64_1d", keys)
            vv = ctx.new("i32_1d", idx)
            w["cpu"] = lambda: oracle.mc_radix_sort(keys, idx)

            def step():
                ctx.call("radix_sort_pairs_u64_i32", ["tup2_arr1d_u64_arr1d_i32"], k, vv).free()
            w.update(bytes=8 * 32 * n, keep=[k, vv])
        w["cpu_how"] = ("per 8-bit digit a histogram per task, an exclusive scan of the [digit][task] "
                        "counts and a stable scatter; each pass includes a copy of the unsorted input")
        w.update(step=step, kernel="radix_sort", dtype=kt, bound="hbm",
                 describe=f"stable LSD radix sort, 8-bit digits, 2^{sz[2:]} {kt}")
    elif name.startswith("bmm_"):
        # bmm_f16_1x4096 | bmm_f32_64x512
        _, t, shape = name.split("_")
        b, m = (int(x) for x in shape.split("x"))
        sc = 1.0 / np.sqrt(m)
        A = dg.normal_f32(64, b * m * m, sc).reshape(b, m, m)
        B = dg.normal_f32(65, b * m * m, sc).reshape(b, m, m)
        if t == "f32":
            a, bb = ctx.new("f32_3d", A), ctx.new("f32_3d", B)
            # CPU: a bounded sample of the rows of C (all of B is needed for any row)
            rows = min(b * m, max(16, (1 << 31) // (m * m)))
            Bt = oracle.mc_transpose_f32(B)
            Cs = np.empty((b, m, m), np.float32)
            w["cpu"] = lambda: oracle.mc_bmm_rows_f32(A, Bt, Cs, 0, rows)
            w["cpu_work"] = 2 * rows * m * m
            w["cpu_how"] = (f"rows 0..{rows - 1} of the {b * m} rows of C: parallel over rows, sequential "
                            f"loops over columns and k, B transposed once beforehand (not timed)")
        else:
            bits = dg.to_f16_bits if t == "f16" else dg.to_bf16_bits
            A16, B16 = bits(A), bits(B)
            kind = "f16_3d" if t == "f16" else "u16_3d"
            a, bb = ctx.new(kind, A16), ctx.new(kind, B16)
            rows = min(b * m, max(16, (1 << 29) // (m * m)))
            Bt16 = oracle.mc_transpose_16(B16)
            Cs = np.empty((b, m, m), np.float32)
            w["cpu"] = lambda: oracle.mc_bmm_rows_16(A16, Bt16, Cs, 0, rows, t == "bf16")
            w["cpu_work"] = 2 * rows * m * m
            w["cpu_how"] = (f"rows 0..{rows - 1} of the {b * m} rows of C: parallel over rows, sequential "
                            f"loops over columns and k, every {t} element widened to f32 where it is used, "
                            f"B transposed once beforehand (not timed)")

        def step():
            ctx.call(f"bmm_{t}", ["f32_3d"], a, bb).free()
        w.update(step=step, flops=2 * b * m * m * m, kernel="segmap_matmul", dtype=t, bound="mfma",
                 keep=[a, bb], describe=f"batched matmul b={b} M=N=K={m}, {t} in, f32 accumulate")
    elif name.startswith("scanrows_"):
        # scanrows_add_f32_65536x1024: map (scan op ne) xss
        _, op, t, shape = name.split("_")
        m, k = (int(x) for x in shape.split("x"))
        w["elements"] = m * k
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        xss = (dg.uniform_f32(38, m * k) if t[0] == "f" else dg.uniform_int(39, m * k, -1000, 1000)
               ).astype(dt).reshape(m, k)
        a = ctx.new(f"{t}_2d", xss)

        def step():
            ctx.call(f"scanrows_{op}_{t}", [f"{t}_2d"], a).free()
        w.update(step=step, bytes=2 * m * k * dt().itemsize, kernel="segscan_rows", dtype=t,
                 bound="hbm", keep=[a], describe=f"scan ({op}) of every row of [{m}][{k}]{t}")
    elif name.startswith("vecscan_"):
        # vecscan_add_f32_65536x1024: scan (map2 op) (replicate k ne) xss, xss : [n][k]
        _, op, t, shape = name.split("_")
        n, k = (int(x) for x in shape.split("x"))
        w["elements"] = n * k
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        xss = (dg.uniform_f32(38, n * k) if t[0] == "f" else dg.uniform_int(39, n * k, -1000, 1000)
               ).astype(dt).reshape(n, k)
        a = ctx.new(f"{t}_2d", xss)

        def step():
            ctx.call(f"vecscan_{op}_{t}", [f"{t}_2d"], a).free()
        w.update(step=step, bytes=2 * n * k * dt().itemsize, kernel="vecscan", dtype=t, bound="hbm",
                 keep=[a], describe=f"scan with vectorised operator (map2 {op}) of [{n}][{k}]{t}")
    elif name.startswith("rowsfraction_"):
        # rowsfraction_f32_65536x1024: reduce, scan and map over every row inside one block
        _, t, shape = name.split("_")
        m, k = (int(x) for x in shape.split("x"))
        w["elements"] = m * k
        xss = (dg.uniform_f32(38, m * k) + np.float32(0.01)).reshape(m, k)
        a = ctx.new("f32_2d", xss)

        def step():
            ctx.call("rows_fraction_f32", ["f32_2d"], a).free()
        w.update(step=step, bytes=2 * m * k * 4, kernel="intrablock_rows", dtype=t, bound="hbm",
                 keep=[a], describe=f"row sums, row scans and a division inside a block, [{m}][{k}]{t}")
    elif name.startswith("segreduce_"):
        # segreduce_add_f32_65536x1024: regular segments, map (reduce op ne) xss
        _, op, t, shape = name.split("_")
        m, k = (int(x) for x in shape.split("x"))
        w["elements"] = m * k
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        xss = (dg.uniform_f32(36, m * k) if t[0] == "f" else dg.uniform_int(37, m * k, -1000, 1000)
               ).astype(dt).reshape(m, k)
        a = ctx.new(f"{t}_2d", xss)

        def step():
            ctx.call(f"segreduce_{op}_{t}", [f"{t}_1d"], a).free()
        w.update(step=step, bytes=m * k * dt().itemsize + m * dt().itemsize, kernel="segred_regular",
                 dtype=t, bound="hbm", keep=[a],
                 describe=f"regular segmented reduce ({op}) of [{m}][{k}]{t}")
    elif name.startswith("vecreduce_"):
        # vecreduce_add_f32_65536x1024: reduce (map2 op) (replicate k ne) xss, xss : [n][k]
        _, op, t, shape = name.split("_")
        n, k = (int(x) for x in shape.split("x"))
        w["elements"] = n * k
        dt = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "f64": np.float64}[t]
        xss = (dg.uniform_f32(38, n * k) if t[0] == "f" else dg.uniform_int(39, n * k, -1000, 1000)
               ).astype(dt).reshape(n, k)
        a = ctx.new(f"{t}_2d", xss)

        def step():
            ctx.call(f"vecreduce_{op}_{t}", [f"{t}_1d"], a).free()
        w.update(step=step, bytes=n * k * dt().itemsize + k * dt().itemsize, kernel="segred_columns",
                 dtype=t, bound="hbm", keep=[a],
                 describe=f"reduce with vectorised operator (map2 {op}) of [{n}][{k}]{t}")
    elif name.startswith("transpose_"):
        # transpose_f32_8192x8192
        _, t, shape = name.split("_")
        rows, cols = (int(x) for x in shape.split("x"))
        w["elements"] = rows * cols
        x = ctx.new("f32_2d", dg.uniform_f32(90, rows * cols).reshape(rows, cols))

        def step():
            ctx.call("transpose_f32", ["f32_2d"], x).free()
        w.update(step=step, bytes=2 * rows * cols * 4, kernel="map_transpose_4b", dtype=t, bound="hbm",
                 keep=[x], describe=f"transpose of [{rows}][{cols}]{t} (map_transpose_4b)")
    elif name.startswith("mfma_peak_"):
        # mfma_peak_f16: registers-only MFMA rate on operands distributed like bmm_*_1x4096's
        import ctypes as C
        from futhark_amd import lib_path
        t = name.split("_")[2]
        m = 4096
        vals = dg.normal_f32(64, 4096, 1.0 / np.sqrt(m))
        bits = dg.to_f16_bits(vals) if t == "f16" else dg.to_bf16_bits(vals)
        ops = ctx.new("u16_1d", bits)
        sink = ctx.new("f32_1d", np.zeros(4, np.float32))
        k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
        k.fa_mfma_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                    C.POINTER(C.c_double)]
        hip = C.CDLL("libamdhip64.so")
        blocks, iters = 256, 2000
        flop = C.c_double(0.0)
        code = {"f16": 6, "bf16": 7}[t]
        ev0, ev1 = C.c_void_p(), C.c_void_p()
        assert hip.hipEventCreate(C.byref(ev0)) == 0 and hip.hipEventCreate(C.byref(ev1)) == 0
        durations = []

        def step():
            timed = not w.get("paused", True)
            if timed:
                hip.hipEventRecord(ev0, C.c_void_p(ctx.stream))
            rc = k.fa_mfma_probe(ctx.stream, code, ops.device_ptr, blocks, iters, sink.device_ptr,
                                 C.byref(flop))
            assert rc == 0, rc
            if timed:
                hip.hipEventRecord(ev1, C.c_void_p(ctx.stream))
                hip.hipEventSynchronize(ev1)
                ms = C.c_float(0.0)
                hip.hipEventElapsedTime(C.byref(ms), ev0, ev1)
                durations.append(ms.value * 1e3)
        step()
        ctx.sync()
        w.update(step=step, flops=flop.value, kernel="mfma_probe", dtype=t, bound="mfma",
                 keep=[ops, sink], own_events=durations,
                 describe=f"registers-only MFMA 32x32x16 {t} (f32 accumulate), {blocks} blocks x 4 waves x "
                          f"{iters} rounds of 16 MFMAs, operands N(0,1)/sqrt({m})")
    else:
        raise SystemExit(f"unknown workload {name}")
    return w


def run_via_server(name: str, steps: int, warmup: int):
    """`futhark bench` protocol: restore inputs once, then time `call` (entry + sync, as the
    server measures it: rts/c/server.h:386-391) with the result freed between runs."""
    import tempfile
    from futhark_amd import datagen as dg
    from futhark_amd import values as fv
    from futhark_amd.server import Server

    kind, op, t, sz = name.split("_")
    n = 1 << int(sz[2:])
    if kind in ("segscan", "segred"):
        offsets, lens, flags = dg.segments(32, n, 1024)
        xs = dg.uniform_f32(33, n) if t == "f32" else dg.uniform_int(34, n, -(1 << 20), 1 << 20, np.int64)
        if kind == "segscan":
            arrays, types = [flags, xs], ["[]u8", f"[]{t}"]
        else:
            arrays, types = [offsets, lens, xs], ["[]i64", "[]i64", f"[]{t}"]
    elif kind in ("scan", "reduce"):
        xs = dg.uniform_f32(17, n) if t == "f32" else dg.uniform_int(16, n, -1000, 1000)
        arrays, types = [xs], [f"[]{t}"]
    else:
        raise SystemExit("--via-server covers scan/reduce/segscan/segred workloads")
    names = [f"in{i}" for i in range(len(arrays))]
    with tempfile.TemporaryDirectory() as d, Server() as srv:
        path = f"{d}/inputs.bin"
        fv.write_binary(path, arrays)
        srv.cmd("restore", path, *[w for pair in zip(names, types) for w in pair])
        runtimes = []
        for i in range(warmup + steps):
            us = srv.call(f"{kind}_{op}_{t}", "out", *names)
            srv.cmd("free", "out")
            if i >= warmup:
                runtimes.append(us)
    return {"entry": f"{kind}_{op}_{t}", "runs": steps,
            "runtime_us_mean": round(float(np.mean(runtimes)), 1),
            "runtime_us_min": int(np.min(runtimes))}


# HBM bytes per step measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by the same
# counters on a 256 MiB copy).  The figure is read from the summary of that run,
# profiles/<kernel>_<workload>.txt, which ends its traffic section with a line
# "TRAFFIC_BYTES_PER_STEP <workload> <bytes>"; a workload without such a summary reports null.
def measured_traffic_bytes(workload: str):
    for f in sorted((ROOT / "profiles").glob("*.txt")):
        for line in f.read_text().splitlines():
            p = line.split()
            if len(p) == 3 and p[0] == "TRAFFIC_BYTES_PER_STEP" and p[1] == workload:
                return float(p[2])
    return None


# What the default run measures besides the headline workload: every BASELINE configuration at
# its full size (reduce / scan / segmented reduce at 2^26, histograms at 2^27 into 256, 65 536 and
# 2^22 bins, both sorts at 2^26, the matmuls of config 4) and the MFMA rate this GPU sustains on
# registers alone, which bounds what a matmul kernel can reach here.
SUITE = [
    "reduce_add_f32_2p26", "scan_add_f32_2p26", "scan_add_i32_2p24", "reduce_add_i32_2p24",
    "segred_add_f32_2p26", "segscan_add_i64_2p26",
    "hist_add_i32_H256_uniform_2p27", "hist_add_i32_H65536_uniform_2p27",
    "hist_add_i32_H4194304_uniform_2p27", "hist_add_i32_H4194304_zipf_2p27",
    "hist_add_f32_H256_uniform_2p27", "hist_add_f32_H256_zipf_2p27", "hist_add_f32_H65536_uniform_2p27",
    "hist_max_f32_H65536_uniform_2p27",
    "sort_u32_2p26", "sort_u64i32_2p26",
    "bmm_f16_1x4096", "bmm_bf16_1x4096", "bmm_f32_1x4096", "bmm_f16_64x512", "bmm_f32_64x512",
    "mfma_peak_f16", "mfma_peak_bf16",
]


def measure(ctx, w, steps: int, warmup: int, prewarm_seconds: float):
    """Times one workload.  Two loops of the same K steps: the first with profiling paused gives
    the wall time per step (`ms_per_step`, what `value` is computed from); the second records a HIP
    event pair around every launch on the context's stream and is timed by the wall clock as well
    (`ms_per_step_profiled`), so that the mean event interval of the dominant kernel (`kernel_us`)
    and a wall time over the very same steps stand side by side."""
    step = w["step"]
    ctx.L.futhark_context_pause_profiling(ctx.ptr)
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < prewarm_seconds:
        for _ in range(10):
            step()
        ctx.sync()
    for _ in range(warmup):
        step()
    ctx.sync()

    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    ctx.report()  # drop whatever was recorded before
    ctx.L.futhark_context_unpause_profiling(ctx.ptr)
    w["paused"] = False
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    ms_profiled = (time.perf_counter() - t0) * 1e3 / steps
    w["paused"] = True
    ctx.L.futhark_context_pause_profiling(ctx.ptr)
    report = json.loads(ctx.report())
    durs = [e["duration"] for e in report["events"] if e["name"] == w["kernel"]]
    if "own_events" in w:  # a workload outside the program library times its launches itself
        durs = list(w["own_events"])
        del w["own_events"][:]
    # events of one step (a step may launch the kernel more than once: count per step)
    per_step = len(durs) / steps if durs else 0
    kernel_us = float(np.sum(durs)) / steps if durs else float("nan")
    kernel_us_min = float(np.min(durs)) * per_step if durs else float("nan")
    kernel_us_ci95 = (float(1.96 * np.std(durs, ddof=1) / np.sqrt(len(durs))) * per_step
                      if len(durs) > 1 else 0.0)

    if w["bound"] == "hbm":
        work, unit, peak, scale = w["bytes"], "GB/s", HBM_PEAK_GBS, 1e9
    else:
        work, unit, peak, scale = w["flops"], "TFLOP/s", MFMA_PEAK_TFLOPS[w["dtype"]], 1e12
    value = work / (ms_per_step * 1e-3) / scale
    achieved = work / (kernel_us * 1e-6) / scale
    return {
        "value": round(value, 3), "unit": unit, "ms_per_step": round(ms_per_step, 5),
        "ms_per_step_profiled": round(ms_profiled, 5), "work": work,
        "roofline": {"bound": w["bound"], "achieved": round(achieved, 3), "peak": peak,
                     "unit": unit, "frac": round(achieved / peak, 4),
                     "traffic": measured_traffic_bytes(w["name"]),
                     "kernel": w["kernel"], "kernel_us": round(kernel_us, 3),
                     "kernel_us_min": round(kernel_us_min, 3),
                     "kernel_us_ci95": round(kernel_us_ci95, 3)},
    }


def cpu_baseline(w, seconds: float):
    """Times the futhark-multicore-style restatement of the workload (oracle/multicore.c) on the
    host cores for about `seconds`; None for a workload that has none."""
    if "cpu" not in w:
        return None
    import oracle
    hbm = w["bound"] == "hbm"
    work = w.get("cpu_work", w["bytes"] if hbm else w["flops"])
    w["cpu"]()  # warm-up
    reps, t_cpu = 0, 0.0
    start = time.perf_counter()
    while t_cpu < seconds and reps < 100000:
        w["cpu"]()
        reps += 1
        t_cpu = time.perf_counter() - start
    scale, unit = (1e9, "GB/s") if hbm else (1e12, "TFLOP/s")
    how = w.get("cpu_how")
    whole = "cpu_work" not in w
    cpu = {"value": round(work * reps / t_cpu / scale, 6 if not hbm else 3), "unit": unit,
           "cores": oracle.mc_threads(), "kind": "port",
           "sample": f"{reps} passes of " + ("the full workload" if whole else "a bounded part of the workload")
                     + " with the futhark-multicore-style restatement in oracle/multicore.c"
                     + (f" ({how})" if how else "") + f", {t_cpu:.1f} s"}
    if "cpu_seq" in w:
        fn, nbytes = w["cpu_seq"]
        fn()
        t_s = time.perf_counter()
        fn()
        cpu["single_thread"] = {"value": round(nbytes / (time.perf_counter() - t_s) / 1e9, 3),
                                "unit": "GB/s", "sample": "one pass of oracle/oracle.c (the "
                                "sequential futhark c fold) over the first 2^24 elements"}
    return cpu


def release(ctx, w) -> None:
    """Frees a workload's resident inputs and what the pool kept for it."""
    for a in w.get("keep", []):
        a.free()
    w.clear()
    ctx.clear_caches()


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="segscan_add_f32_2p26")
    ap.add_argument("--prewarm-seconds", type=float, default=0.5,
                    help="untimed passes before the W warm-up steps, until this much time has "
                         "passed: the GPU leaves its idle power state only after a few hundred "
                         "milliseconds of work, and a short MFMA run measured before that reads "
                         "up to 40%% slow")
    ap.add_argument("--via-server", action="store_true",
                    help="additionally drive the same workload through futhark_amd/bin/"
                         "segops-server the way `futhark bench` does (values restored from a "
                         "binary data file, K `call`s) and report the runtimes the server prints; "
                         "scan/reduce/segscan/segred workloads only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--no-suite", action="store_true",
                    help="measure the named workload only (profiling runs); by default the "
                         "other BASELINE configurations are measured after it and reported "
                         "under `suite` in the same JSON line")
    ap.add_argument("--suite-steps", type=int, default=20)
    ap.add_argument("--suite-cpu-seconds", type=float, default=1.5,
                    help="CPU baseline time per workload of the suite (the headline workload "
                         "gets --cpu-seconds)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run the plain copy kernel (fa_copy, 256 MiB) a few times, so "
                         "that a rocprofv3 --pmc run of this command holds a dispatch of known "
                         "traffic to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--param", action="append", default=[], metavar="NAME=VALUE",
                    help="a tuning parameter of the program (as futhark bench passes them), "
                         "e.g. segops.hist_lds_bins_max=16384; may be given several times")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path "
                         "(the reference is single-device); run with --gpus 1")

    from futhark_amd import Context

    tuning = {k: int(v) for k, v in (p.split("=", 1) for p in args.param)}
    ctx = Context(profiling=True, tuning=tuning or None)
    ctx.L.futhark_context_pause_profiling(ctx.ptr)
    w = make_workload(args.workload, ctx)
    w["name"] = args.workload
    m = measure(ctx, w, args.steps, args.warmup, args.prewarm_seconds)

    cpu = None if args.no_cpu_baseline else cpu_baseline(w, args.cpu_seconds)

    server = None
    if args.via_server:
        server = run_via_server(args.workload, args.steps, args.warmup)

    if args.calibrate_copy:
        import ctypes as C
        from futhark_amd import lib_path
        k = C.CDLL(str(lib_path("libfuthark_amd_kernels.so")))
        k.fa_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        nbytes = 256 << 20
        src = ctx.new("u8_1d", np.zeros(nbytes, np.uint8))
        dst = ctx.new("u8_1d", np.zeros(nbytes, np.uint8))
        for _ in range(5):
            assert k.fa_copy(ctx.stream, dst.device_ptr, src.device_ptr, nbytes) == 0
        ctx.sync()
        src.free()
        dst.free()

    bound, dtype, describe = w["bound"], w["dtype"], w["describe"]
    elements = w.get("elements")
    metric = "achieved GB/s" if bound == "hbm" else "achieved TFLOP/s"
    out = {
        "metric": f"{metric} ({args.workload}), 1xMI355X",
        "value": m["value"], "unit": m["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": m["ms_per_step"],
        "ms_per_step_profiled": m["ms_per_step_profiled"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": describe, "name": args.workload,
                   "algorithmic_bytes_per_step" if bound == "hbm" else "flop_per_step": m["work"],
                   **({"elements_per_s": round(elements / (m["ms_per_step"] * 1e-3), 1)}
                      if elements else {})},
        "roofline": m["roofline"],
        "cpu_baseline": cpu,
    }
    if server is not None:
        out["server"] = server

    if not args.no_suite:
        release(ctx, w)
        suite = {}
        for name in SUITE:
            if name == args.workload:
                continue
            t_w = time.perf_counter()
            sw = make_workload(name, ctx)
            sw["name"] = name
            sm = measure(ctx, sw, args.suite_steps, 3, 0.3 if sw["bound"] == "mfma" else 0.1)
            entry = {"value": sm["value"], "unit": sm["unit"], "ms_per_step": sm["ms_per_step"],
                     "ms_per_step_profiled": sm["ms_per_step_profiled"], "dtype": sw["dtype"],
                     "workload": sw["describe"], "work_per_step": sm["work"],
                     "roofline": sm["roofline"]}
            if "elements" in sw:
                entry["elements_per_s"] = round(sw["elements"] / (sm["ms_per_step"] * 1e-3), 1)
            if not args.no_cpu_baseline:
                sw.pop("cpu_seq", None)
                entry["cpu_baseline"] = cpu_baseline(sw, args.suite_cpu_seconds)
            suite[name] = entry
            release(ctx, sw)
            print(f"[bench] {name}: {sm['value']} {sm['unit']}, kernel {sm['roofline']['kernel_us']} us, "
                  f"frac {sm['roofline']['frac']} ({time.perf_counter() - t_w:.1f} s)",
                  file=sys.stderr, flush=True)
        out["suite"] = suite
        out["suite_steps"] = args.suite_steps
    print(json.dumps(out))
    ctx.close()


if __name__ == "__main__":
    main()
