"""include/segops.json, the manifest of the library: shaped as
docs/manifest.schema.json of the reference demands (the rules are restated in
_check_* below; tests_lib/c/validatemanifest.py runs a JSON-schema validator,
which this image does not have), in step with its generator, and naming only
functions that libsegops.so really exports."""
import json
import subprocess
from pathlib import Path

from futhark_amd import lib_path, manifest

ROOT = Path(__file__).resolve().parent.parent
PRIMS = {"i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "f16", "f32", "f64", "bool"}


def _exports(path):
    out = subprocess.check_output(["nm", "-D", "--defined-only", str(path)], text=True)
    return {l.split()[-1] for l in out.splitlines() if l.strip()}


def _only(obj, allowed):
    assert isinstance(obj, dict) and set(obj) <= set(allowed), (set(obj) - set(allowed))


def _strs(obj, *keys):
    for k in keys:
        if k in obj:
            assert isinstance(obj[k], str), (k, obj[k])


def _check_entry(e):
    _strs(e, "cfun", "doc")
    for k in ("tuning_params", "attributes"):
        assert all(isinstance(x, str) for x in e.get(k, []))
    _only(e["output"], {"type", "unique"})
    assert isinstance(e["output"]["type"], str) and isinstance(e["output"]["unique"], bool)
    for i in e["inputs"]:
        _only(i, {"name", "type", "unique"})
        assert isinstance(i["name"], str) and isinstance(i["type"], str) and isinstance(i["unique"], bool)


def _check_type(t):
    if t["kind"] == "array":
        assert isinstance(t["ctype"], str) and isinstance(t["rank"], int) and t["elemtype"] in PRIMS
        _only(t["ops"], {"free", "shape", "values", "values_raw", "new", "new_raw", "index"})
        _strs(t["ops"], *t["ops"])
    else:
        assert t["kind"] == "opaque"
        assert {"kind", "ctype", "ops"} <= set(t)
        assert any(k in t for k in ("record", "sum", "record_array", "opaque_array"))
        _only(t["ops"], {"free", "store", "restore"})
        _strs(t["ops"], *t["ops"])
        _only(t["record"], {"new", "fields"})
        for f in t["record"]["fields"]:
            _strs(f, "name", "type", "project")


def test_manifest_file_is_what_the_generator_writes():
    on_disk = json.loads((ROOT / "include" / "segops.json").read_text())
    assert on_disk == manifest.manifest()


def test_manifest_has_the_shape_the_schema_demands():
    m = manifest.manifest()
    _only(m, {"backend", "version", "entry_points", "types"})
    assert {"backend", "entry_points", "types"} <= set(m)
    assert m["backend"] == "hip" and isinstance(m["version"], str)
    for e in m["entry_points"].values():
        _check_entry(e)
    for t in m["types"].values():
        _check_type(t)
    # every type an entry point mentions is a primitive or described under "types"
    known = PRIMS | set(m["types"])
    for name, e in m["entry_points"].items():
        for ty in [e["output"]["type"]] + [i["type"] for i in e["inputs"]]:
            assert ty in known, (name, ty)
    for t in m["types"].values():
        if t["kind"] == "opaque":
            assert all(f["type"] in known for f in t["record"]["fields"])


def test_every_function_the_manifest_names_is_exported_and_every_entry_is_listed():
    m = manifest.manifest()
    exported = _exports(lib_path())
    named = {e["cfun"] for e in m["entry_points"].values()}
    for t in m["types"].values():
        named |= set(t["ops"].values())
        if t["kind"] == "opaque":
            named.add(t["record"]["new"])
            named |= {f["project"] for f in t["record"]["fields"]}
    assert not named - exported, sorted(named - exported)
    entries = {s for s in exported if s.startswith("futhark_entry_")}
    assert entries == {e["cfun"] for e in m["entry_points"].values()}
    tuning = {p for e in m["entry_points"].values() for p in e["tuning_params"]}
    assert tuning == {"segops.hist_lds_bins_max", "segops.segred_small_threshold",
                      "segops.matmul_pad_min_work", "segops.scan_arrival_tickets",
                      "segops.sort_wide_positions"}
