"""The manifest of the `segops` library: the JSON description of its C API that
`futhark hip --library` writes next to the header (docs/c-api.rst:794-871,
schema docs/manifest.schema.json; filled in by
src/Futhark/CodeGen/Backends/GenericC/EntryPoints.hs:210-221 for entry points
and GenericC/Types.hs:242-250,1185-1214 for types).  The serialiser itself is
the Hackage package futhark-manifest 1.9.0.0, which is not part of the
reference tree: key names follow the schema file.

`python -m futhark_amd.manifest` writes include/segops.json.
"""
from __future__ import annotations

import json
from pathlib import Path

from .capi import ARRAY_TYPES, HIST_ONLY_TYPES, NUM_TYPES, OPAQUE_PAIRS, ops_for

ROOT = Path(__file__).resolve().parent.parent
BACKEND = "hip"
VERSION = "segops for gfx950, C API of Futhark 0.28.0"
HIST_PARAM = "segops.hist_lds_bins_max"
SEGRED_PARAM = "segops.segred_small_threshold"
MATMUL_PARAM = "segops.matmul_pad_min_work"
SCAN_PARAM = "segops.scan_arrival_tickets"
SORT_PARAM = "segops.sort_wide_positions"


def _array_type_name(kind: str) -> str:
    elem, rank = kind.rsplit("_", 1)
    return "[]" * int(rank[0]) + elem


def _entry(name, out_type, inputs, tuning=(), out_unique=True):
    return name, {
        "cfun": f"futhark_entry_{name}",
        "tuning_params": list(tuning),
        "attributes": [],
        "output": {"type": out_type, "unique": out_unique and out_type.startswith(("[", "("))},
        "inputs": [{"name": n, "type": t.lstrip("*"), "unique": t.startswith("*")} for n, t in inputs],
    }


def entry_points() -> dict:
    eps = []
    for t in NUM_TYPES:
        for op in ops_for(t):
            a = f"[]{t}"
            eps += [
                _entry(f"reduce_{op}_{t}", t, [("xs", a)]),
                _entry(f"scan_{op}_{t}", a, [("xs", a)], [SCAN_PARAM]),
                _entry(f"exscan_{op}_{t}", a, [("xs", a)], [SCAN_PARAM]),
                _entry(f"segscan_{op}_{t}", a, [("flags", "[]u8"), ("vs", a)], [SCAN_PARAM]),
                _entry(f"segred_{op}_{t}", a, [("offsets", "[]i64"), ("lens", "[]i64"), ("vs", a)]),
                _entry(f"segreduce_{op}_{t}", a, [("xss", "[]" + a)], [SEGRED_PARAM]),
                _entry(f"vecreduce_{op}_{t}", a, [("xss", "[]" + a)]),
                _entry(f"scanrows_{op}_{t}", "[]" + a, [("xss", "[]" + a)], [SCAN_PARAM]),
                _entry(f"vecscan_{op}_{t}", "[]" + a, [("xss", "[]" + a)]),
                _entry(f"seghist_{op}_{t}", "[]" + a,
                       [("k", "i64"), ("iss", "[][]i32"), ("vss", "[]" + a)], [HIST_PARAM]),
                _entry(f"rbi_vec_{op}_{t}", "[]" + a,
                       [("dest", "*[]" + a), ("is", "[]i64"), ("vss", "[]" + a)], [HIST_PARAM]),
                _entry(f"rbi_2d_{op}_{t}", "[]" + a,
                       [("dest", "*[]" + a), ("is", "[]i64"), ("js", "[]i64"), ("vs", a)],
                       [HIST_PARAM]),
            ]
    for t in list(NUM_TYPES) + list(HIST_ONLY_TYPES):
        for op in ops_for(t):
            a = f"[]{t}"
            for ix, it in (("", "[]i32"), ("_i64", "[]i64")):
                eps += [
                    _entry(f"hist_{op}_{t}{ix}", a, [("k", "i64"), ("is", it), ("vs", a)], [HIST_PARAM]),
                    _entry(f"rbi_{op}_{t}{ix}", a, [("dest", "*" + a), ("is", it), ("vs", a)], [HIST_PARAM]),
                ]
    eps += [
        _entry("bmm_f32", "[][][]f32", [("A", "[][][]f32"), ("B", "[][][]f32")], [MATMUL_PARAM]),
        _entry("bmm_f16", "[][][]f32", [("A", "[][][]f16"), ("B", "[][][]f16")], [MATMUL_PARAM]),
        _entry("scan_compose_i32", "[][]i32", [("abs", "[][]i32")], [SCAN_PARAM]),
        _entry("exscan_compose_i32", "[][]i32", [("abs", "[][]i32")], [SCAN_PARAM]),
        _entry("segscan_compose_i32", "[][]i32", [("flags", "[]u8"), ("abs", "[][]i32")], [SCAN_PARAM]),
        _entry("reduce_argmax_i32", "[]i32", [("xs", "[]i32")]),
        _entry("scan_argmax_i32", "[][]i32", [("vis", "[][]i32")]),
        _entry("hist_argmax_i32", "[][]i32", [("k", "i64"), ("is", "[]i32"), ("xs", "[]i32")]),
        _entry("reduce_compose_i32", "[]i32", [("abs", "[][]i32")]),
        _entry("sumsq_f32", "f32", [("xs", "[]f32")]),
        _entry("scan_norm_f32", "[]f32", [("xs", "[]f32")]),
        _entry("reduce_summax_f32", "[]f32", [("xs", "[]f32")]),
        _entry("rows_fraction_f32", "[][]f32", [("xss", "[][]f32")]),
        _entry("segreduce_argmax_i32", "[][]i32", [("xss", "[][]i32")]),
        _entry("segreduce_compose_i32", "[][]i32", [("k", "i64"), ("abs", "[][]i32")]),
        _entry("scanrows_argmax_i32", "[][]i32", [("k", "i64"), ("vis", "[][]i32")]),
        _entry("segred_argmax_i32", "[][]i32", [("offsets", "[]i64"), ("lens", "[]i64"), ("vis", "[][]i32")]),
        _entry("bmm_bf16", "[][][]f32", [("A", "[][][]u16"), ("B", "[][][]u16")], [MATMUL_PARAM]),
        _entry("matmul_f32", "[][]f32", [("A", "[][]f32"), ("B", "[][]f32")], [MATMUL_PARAM]),
        _entry("radix_sort_u32", "[]u32", [("keys", "[]u32")], [SORT_PARAM]),
        _entry("radix_sort_u64", "[]u64", [("keys", "[]u64")], [SORT_PARAM]),
    ]
    for k, v in OPAQUE_PAIRS.values():
        eps.append(_entry(f"radix_sort_pairs_{k}_{v}", f"([]{k}, []{v})",
                          [("keys", f"[]{k}"), ("vals", f"[]{v}")], [SORT_PARAM]))
    eps += [
        _entry("transpose_f32", "[][]f32", [("xss", "[][]f32")]),
        _entry("iota_i64", "[]i64", [("n", "i64")]),
        _entry("replicate_i32", "[]i32", [("n", "i64"), ("x", "i32")]),
    ]
    return dict(eps)


def types() -> dict:
    out = {}
    for kind in ARRAY_TYPES:
        elem, rank = kind.rsplit("_", 1)
        out[_array_type_name(kind)] = {
            "kind": "array",
            "ctype": f"struct futhark_{kind} *",
            "rank": int(rank[0]),
            "elemtype": elem,
            "ops": {op: f"futhark_{op}_{kind}"
                    for op in ("free", "shape", "values", "values_raw", "new", "new_raw", "index")},
        }
    for name, (k, v) in OPAQUE_PAIRS.items():
        out[f"([]{k}, []{v})"] = {
            "kind": "opaque",
            "ctype": f"struct futhark_opaque_{name} *",
            "ops": {op: f"futhark_{op}_opaque_{name}" for op in ("free", "store", "restore")},
            "record": {
                "new": f"futhark_new_opaque_{name}",
                "fields": [
                    {"name": "0", "type": f"[]{k}", "project": f"futhark_project_opaque_{name}_0"},
                    {"name": "1", "type": f"[]{v}", "project": f"futhark_project_opaque_{name}_1"},
                ],
            },
        }
    return out


def manifest() -> dict:
    return {"backend": BACKEND, "version": VERSION, "entry_points": entry_points(), "types": types()}


def write(path: Path | None = None) -> Path:
    path = path or ROOT / "include" / "segops.json"
    path.write_text(json.dumps(manifest(), indent=1, sort_keys=True) + "\n")
    return path


if __name__ == "__main__":
    print(write())
