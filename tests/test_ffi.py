"""The embedding C ABI (include/clpeak_ffi.h) through ctypes, against the stand-in device.

These restate the reference's own bridge tests (app/test/ffi_integration_test.dart:28-104: version
and catalog, a quick run that streams events and saves XML, bad arguments, cancellation) and add the
parts of the protocol that file leaves to the header (src/ffi/clpeak_ffi.h:40-82): string ownership,
the busy code, numbers in the classic locale with four decimals.
"""
import ctypes as C
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# the embedding ABI built from the host layer's own sources against the pretend device (tests/host_double)
HOSTLIB = os.path.join(ROOT, "tests", "host_double", "libclpeak_host_double.so")
SHIPPED = os.path.join(ROOT, "clpeak_amd", "libclpeak_host.so")
HEADER = os.path.join(ROOT, "include", "clpeak_ffi.h")

CALLBACK = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)
RUN_OK, RUN_BAD_ARGS, RUN_CANCELLED, RUN_BUSY = 0, -1, -2, -3


@pytest.fixture(scope="module", autouse=True)
def _host_double():
    from conftest import ensure_host_double
    ensure_host_double()


@pytest.fixture(scope="module")
def ffi(_host_double):
    lib = C.CDLL(HOSTLIB)
    lib.clpeak_version.restype = C.c_char_p
    lib.clpeak_copy_backend_catalog_json.restype = C.c_void_p
    lib.clpeak_free_string.argtypes = [C.c_void_p]
    lib.clpeak_free_string.restype = None
    lib.clpeak_launch.argtypes = [C.c_int, C.POINTER(C.c_char_p), CALLBACK, C.c_void_p]
    lib.clpeak_launch.restype = C.c_int
    lib.clpeak_request_cancel.restype = None
    lib.clpeak_load_result_file_json.argtypes = [C.c_char_p]
    lib.clpeak_load_result_file_json.restype = C.c_void_p
    return lib


def take_string(lib, p):
    """Decode a malloc'd string and give it back to the library, as the contract demands."""
    s = C.string_at(p).decode("utf-8")
    lib.clpeak_free_string(p)
    return s


def launch(lib, args, on_event=None):
    """Run with argv = ["clpeak", *args]; returns (rc, raw event strings)."""
    raw = []

    def cb(_user, p):
        raw.append(take_string(lib, p))
        if on_event:
            on_event(json.loads(raw[-1]))

    argv = [b"clpeak"] + [a.encode() for a in args]
    arr = (C.c_char_p * len(argv))(*argv)
    keep = CALLBACK(cb)
    rc = lib.clpeak_launch(len(argv), arr, keep, None)
    return rc, raw


def test_header_symbols_are_exported(ffi):
    declared = re.findall(r"CLPEAK_FFI_EXPORT[^;]*?\b(clpeak_\w+)\s*\(", open(HEADER).read())
    assert sorted(declared) == sorted(["clpeak_version", "clpeak_copy_backend_catalog_json", "clpeak_free_string",
                                       "clpeak_launch", "clpeak_request_cancel", "clpeak_load_result_file_json"])
    for name in declared:
        getattr(ffi, name)


def test_version_and_catalog(ffi, monkeypatch):
    assert ffi.clpeak_version()
    monkeypatch.setenv("CLPEAK_FAKE_DEVICES", "2")
    doc = json.loads(take_string(ffi, ffi.clpeak_copy_backend_catalog_json()))
    (be,) = doc["backends"]
    assert be["name"] == "ROCm" and be["available"] is True
    devs = be["platforms"][0]["devices"]
    assert [d["index"] for d in devs] == [0, 1]
    assert devs[0] == {"index": 0, "name": "Fake MI355X", "type": "GPU", "driver": "7.2.0", "computeUnits": 256,
                       "clockMHz": 2400, "globalMemBytes": 288 << 30, "fp16": True, "fp64": True}
    monkeypatch.setenv("CLPEAK_FAKE_DEVICES", "0")
    doc = json.loads(take_string(ffi, ffi.clpeak_copy_backend_catalog_json()))
    assert doc == {"backends": [{"name": "ROCm", "available": False, "platforms": []}]}


def test_quick_run_streams_events_and_saves_xml(ffi, tmp_path):
    xml = tmp_path / "run.xml"
    rc, raw = launch(ffi, ["--small-shapes", "-i", "1", "--xml-file", str(xml)])
    events = [json.loads(r) for r in raw]
    assert rc == RUN_OK
    assert events[-1] == {"t": "done", "status": 0, "cancelled": False}
    kinds = [e["t"] for e in events]
    assert kinds[0] == "backend_begin" and kinds[1] == "device" and kinds[-2] == "backend_end" and kinds[-3] == "device_end"
    assert kinds.count("test_begin") == kinds.count("test_end")
    dev = events[1]
    assert dev["backend"] == "ROCm" and dev["device"] == "Fake MI355X" and dev["device_index"] == 0
    assert [p["k"] for p in dev["props"]] == ["Arch", "HIP", "CUs", "Wave", "VRAM"]
    metrics = [e for e in events if e["t"] == "metric"]
    assert metrics and metrics[0]["backend"] == "ROCm"
    assert any(m["status"] == "ok" and m["value"] > 0 for m in metrics)
    assert {"category", "test", "display", "metric", "unit", "value", "status", "reason", "sub", "desc", "minfo"} <= set(metrics[0])
    # the fields the GUI's event model decodes, and the row key it builds from them (app/test/models_test.dart:107-131)
    m0 = metrics[0]
    assert {"backend", "platform", "device", "driver", "category", "test", "display", "metric", "unit", "value", "status",
            "reason", "sub"} <= set(m0)
    assert isinstance(m0["sub"], bool) and isinstance(m0["value"], float) and m0["reason"] == ""
    key = "/".join(m0[k] for k in ("backend", "platform", "device", "category", "test", "metric"))
    assert key == "ROCm/ROCm/Fake MI355X/fp_compute/single_precision_compute/float"
    # what a test measures arrives on test_begin, a reading's own note rides the row
    begin = next(e for e in events if e["t"] == "test_begin" and e["test"] == "global_memory_bandwidth")
    assert begin["desc"] and begin["unit"] == "gbps" and begin["category"] == "bandwidth"
    assert all(m["minfo"] for m in metrics if m["test"] == "global_memory_bandwidth")
    # numbers: classic locale, four decimals, in the raw text
    for r in raw:
        if '"t":"metric"' in r:
            assert re.search(r'"value":-?\d+\.\d{4}[,}]', r), r
    # the saved file round-trips through the native loader
    assert xml.exists()
    doc = json.loads(take_string(ffi, ffi.clpeak_load_result_file_json(str(xml).encode())))
    skipped_all = sum(len(e["metrics"]) for e in events if e["t"] == "test_skipped")
    assert len(doc["entries"]) == len(metrics) + skipped_all
    assert doc["format_version"] == 2 and doc["devices"][0]["device"] == "Fake MI355X"
    row = next(e for e in doc["entries"] if e["test"] == "global_memory_bandwidth" and e["metric"] == "float4")
    assert row["description"] == begin["desc"] and row["metric_description"]


def test_bad_args_are_rejected_without_side_effects(ffi, tmp_path):
    xml = tmp_path / "never.xml"
    for args in (["--bogus-flag"], ["--help"], ["--version"], ["--list-devices"], ["--iters"], ["--xml-file", str(xml), "--iters", "x"]):
        rc, raw = launch(ffi, args)
        events = [json.loads(r) for r in raw]
        assert rc == RUN_BAD_ARGS, args
        assert [e["t"] for e in events] == ["note", "done"], args
        assert events[0]["message"].startswith("clpeak:")
        assert events[1] == {"t": "done", "status": RUN_BAD_ARGS, "cancelled": False}
    assert not xml.exists()


def test_cancel_stops_the_run_and_still_saves(ffi, tmp_path):
    xml = tmp_path / "partial.xml"
    seen = {"metrics": 0}

    def on_event(e):
        if e["t"] == "metric":
            seen["metrics"] += 1
            if seen["metrics"] == 3:
                ffi.clpeak_request_cancel()     # any thread may call this; here: the run's own

    rc, raw = launch(ffi, ["--small-shapes", "--xml-file", str(xml)], on_event)
    events = [json.loads(r) for r in raw]
    assert rc == RUN_CANCELLED
    assert events[-1] == {"t": "done", "status": RUN_CANCELLED, "cancelled": True}
    # the running test finishes, the remaining ones are skipped silently
    assert [e["test"] for e in events if e["t"] == "test_begin"] == ["single_precision_compute"]
    doc = json.loads(take_string(ffi, ffi.clpeak_load_result_file_json(str(xml).encode())))
    assert [e["test"] for e in doc["entries"]] == ["single_precision_compute"] * 3
    # the flag resets at the start of the next launch
    rc, raw = launch(ffi, ["--small-shapes", "--kernel-launch-latency"])
    assert rc == RUN_OK and json.loads(raw[-1])["cancelled"] is False


def test_second_launch_while_running_is_busy_and_silent(ffi):
    inner = {}

    def on_event(e):
        if e["t"] == "device" and "rc" not in inner:
            inner["rc"], inner["raw"] = launch(ffi, ["--small-shapes"])

    rc, raw = launch(ffi, ["--small-shapes", "--kernel-launch-latency"], on_event)
    assert inner["rc"] == RUN_BUSY and inner["raw"] == []
    assert rc == RUN_OK and json.loads(raw[-1])["t"] == "done"


def test_skipped_backend_runs_nothing(ffi):
    rc, raw = launch(ffi, ["--no-rocm"])
    assert rc == RUN_OK and [json.loads(r)["t"] for r in raw] == ["done"]


def test_load_result_file_rejects_garbage(ffi, tmp_path):
    assert ffi.clpeak_load_result_file_json(None) is None
    assert ffi.clpeak_load_result_file_json(str(tmp_path / "missing.xml").encode()) is None
    bad = tmp_path / "bad.json"
    bad.write_text("{not json")
    assert ffi.clpeak_load_result_file_json(str(bad).encode()) is None


def test_loads_a_result_file_the_reference_wrote(ffi):
    """clpeak_load_result_file_json on a file from the reference's results/ (tests/golden, copied as data):
    every row arrives with the keys the GUI's model reads, values and skip reasons intact."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_results_amd_threadripper.xml")
    doc = json.loads(take_string(ffi, ffi.clpeak_load_result_file_json(path.encode())))
    assert doc["format_version"] == 2 and len(doc["entries"]) == 192
    first = doc["entries"][0]
    assert (first["backend"], first["category"], first["test"], first["metric"], first["unit"]) == \
        ("Vulkan", "fp_compute", "single_precision_compute", "float", "gflops")
    assert abs(first["value"] - 229.0884) < 1e-3 and "status" not in first      # measured rows carry a value, skipped ones a status
    assert first["device"] == "llvmpipe (LLVM 22.1.8, 256 bits)" and first["display"] == "Single-precision compute"
    skipped = [e for e in doc["entries"] if e.get("status") == "unsupported"]
    assert skipped and all(e["reason"] and "value" not in e for e in skipped)
    assert any(e["reason"].startswith("VK_KHR_shader_bfloat16") for e in skipped)
    assert ffi.clpeak_load_result_file_json(b"/nonexistent/file.xml") is None


def test_arguments_the_gui_builds_for_a_partial_selection(ffi):
    """What RunConfig.toArgs (app/lib/src/model/run_config.dart:96-144) hands to clpeak_launch when the user has
    deselected one category, two backends and one of two ROCm devices, and changed both time budgets: a
    --no-<backend> per deselected backend, a device list, a positive flag per remaining category (crypto and
    string included) and both --max-time flags.  The run must start, and run what those flags select."""
    args = ["--no-opencl", "--no-vulkan", "--rocm-device", "0", "--no-cpu",
            "--fp-compute", "--int-compute", "--crypto", "--string", "--bandwidth",
            "--max-time", "200", "--max-time-cpu", "500"]
    rc, raw = launch(ffi, ["--small-shapes", "-i", "1"] + args)
    events = [json.loads(r) for r in raw]
    assert rc == RUN_OK and events[-1] == {"t": "done", "status": 0, "cancelled": False}
    tags = {e["test"] for e in events if e["t"] == "test_begin"}
    assert "single_precision_compute" in tags and "integer_compute" in tags and "global_memory_bandwidth" in tags
    assert "kernel_launch_latency" not in tags             # latency was the deselected category


@pytest.mark.parametrize("args, runs", [
    (["--cuda"], False),                                   # another backend named alone: this one stays out
    (["--cuda", "--rocm"], True),
    (["--no-cuda", "--no-metal", "--no-oneapi"], True),
    (["--aes"], False),                                    # a test of another backend: allow-list with nothing of ours in it
    (["--aes", "--mfma"], True),
    (["--no-aes", "--no-cache-bandwidth", "--use-event-timer"], True),
    (["--cl-platform", "0", "--cl-device", "0,1", "--vk-device", "1", "--cuda-device", "0", "--mtl-device", "0", "--oneapi-device", "2"], True),
    (["--crypto"], False),                                 # a category with no test here
])
def test_flags_of_the_other_backends_parse_with_their_meaning(ffi, args, runs):
    rc, raw = launch(ffi, ["--small-shapes", "-i", "1"] + args)
    events = [json.loads(r) for r in raw]
    assert rc == RUN_OK, (args, events[:1])
    began = [e for e in events if e["t"] == "test_begin"]
    assert bool(began) == runs, (args, [e["test"] for e in began])


@pytest.mark.parametrize("args", [["--max-time-cpu"], ["--max-time-cpu", "0"], ["--max-time", "0"], ["--iters", "0"],
                                  ["--cuda-device", "a"], ["--cl-platform"], ["--integer-compute-wide"]])
def test_malformed_values_of_those_flags_are_still_refused(ffi, args):
    rc, raw = launch(ffi, args)
    assert rc == RUN_BAD_ARGS and json.loads(raw[0])["message"].startswith("clpeak:")
