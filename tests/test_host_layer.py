"""Host layer (C++ Peak / logger / result store / CLI) on a machine without a GPU: the CLI runs
against the stand-in device, so row set, order, gating, degrade paths and the dump formats are
all exercised; no kernel runs."""
import ctypes as C
import json
import os
import re
import subprocess
import xml.etree.ElementTree as ET

import numpy as np
import pytest

from oracle import pyoracle as orc
from oracle import workloads as wl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# the host layer's own sources linked against the pretend device (tests/host_double), not the program that ships
CLI = os.path.join(ROOT, "tests", "host_double", "clpeak-mi355-double")
HOSTLIB = os.path.join(ROOT, "clpeak_amd", "libclpeak_host.so")


@pytest.fixture(scope="module", autouse=True)
def _host_double():
    from conftest import ensure_host_double
    ensure_host_double()


def run_cli(*args, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([CLI, "--small-shapes", *args], capture_output=True, text=True, env=e, timeout=120)


# The rows a ROCm device reports, in order: (test tag, unit, metrics).  Tags, units and metric
# names are the reference's (src/rocm/*.cpp); the tags marked + are rows this backend adds.
EXPECTED_ROWS = [
    ("single_precision_compute", "gflops", ["float", "float2", "float4"]),
    ("half_precision_compute", "gflops", ["half", "half2"]),
    ("double_precision_compute", "gflops", ["double", "double2", "double4"]),
    ("mixed_precision_compute", "gflops", ["mp"]),
    ("bfloat16_compute", "gflops", ["bf16"]),
    ("wmma_fp16", "tflops", ["wmma_fp16"]), ("wmma_bf16", "tflops", ["wmma_bf16"]),
    ("wmma_fp8_e4m3", "tflops", ["wmma_fp8_e4m3"]), ("wmma_fp8_e5m2", "tflops", ["wmma_fp8_e5m2"]),
    ("rocwmma-fp", "tflops", ["rocwmma_fp16"]),
    ("mfma_fp16", "tflops", ["mfma_fp16"]), ("mfma_fp16_32x32x16", "tflops", ["mfma_fp16_32x32x16"]),  # +
    ("mfma_bf16", "tflops", ["mfma_bf16"]), ("mfma_bf16_32x32x16", "tflops", ["mfma_bf16_32x32x16"]),  # +
    ("mfma_fp8", "tflops", ["mfma_fp8"]), ("mfma_bf8", "tflops", ["mfma_bf8"]),                          # +
    ("mfma_mxfp6_e2m3", "tflops", ["mfma_mxfp6_e2m3"]), ("mfma_mxfp6_e3m2", "tflops", ["mfma_mxfp6_e3m2"]),  # +
    ("mfma_mxfp4", "tflops", ["mfma_mxfp4"]),
    ("smfmac_fp16", "tflops", ["smfmac_fp16"]), ("smfmac_bf16", "tflops", ["smfmac_bf16"]),
    ("smfmac_fp8", "tflops", ["smfmac_fp8"]), ("smfmac_bf8", "tflops", ["smfmac_bf8"]),                  # +
    ("rocblas-fp", "tflops", ["fp32", "fp64", "fp16", "bf16"]),
    ("hipblaslt-fp8", "tflops", ["fp8_e4m3", "fp8_e5m2", "mxf4_e2m1"]),
    ("integer_compute", "gops", ["int", "int2", "int4"]),
    ("integer_compute_int8_dp", "gops", ["int8_dp", "int8_dp2", "int8_dp4", "int8_dp8"]),
    ("wmma_int8", "tops", ["wmma_int8"]), ("rocwmma-int", "tops", ["rocwmma_int8"]),
    ("mfma_int8", "tops", ["mfma_int8"]), ("smfmac_int8", "tops", ["smfmac_int8"]),
    ("rocblas-int", "tops", ["int8"]),
    ("global_memory_bandwidth", "gbps", ["float", "float2", "float4"]),
    ("local_memory_bandwidth", "gbps", ["float", "float2", "float4"]),
    ("image_memory_bandwidth", "gbps", ["float4"]),
    ("transfer_bandwidth", "gbps", ["h2d_pinned", "d2h_pinned"]),
    ("kernel_launch_latency", "us", ["dispatch", "roundtrip"]),
]
CATEGORY_OF_UNIT = {"gflops": "fp_compute", "tflops": "fp_compute", "gops": "int_compute", "tops": "int_compute",
                    "gbps": "bandwidth", "us": "latency"}


def parse_xml(path):
    root = ET.parse(path).getroot()
    rows = []
    for run in root.findall("run"):
        for cat in run.findall("category"):
            for test in cat.findall("test"):
                rows.append((cat.get("name"), test.get("name"), test.get("unit"),
                             [(m.get("name"), m.get("status"), m.text) for m in test.findall("metric")]))
    return root, rows


def test_full_run_row_contract_and_xml(tmp_path):
    x = tmp_path / "out.xml"
    r = run_cli("--xml-file", str(x))
    assert r.returncode == 0, r.stderr
    root, rows = parse_xml(x)
    assert root.get("format_version") == "2" and root.get("os") == "Linux x64"
    run = root.find("run")
    assert run.get("backend") == "ROCm" and run.get("platform") == "ROCm" and run.get("device") == "Fake MI355X"
    assert [p.get("name") for p in run.findall("prop")] == ["Arch", "HIP", "CUs", "Wave", "VRAM"]
    assert [(t, u, [m[0] for m in ms]) for _, t, u, ms in rows] == EXPECTED_ROWS
    for cat, _, unit, _ in rows:
        assert cat == CATEGORY_OF_UNIT[unit]
    # measured values carry exactly 4 decimals
    vals = [m[2] for _, _, _, ms in rows for m in ms if m[1] is None]
    assert len(vals) == 49 and all(re.fullmatch(r"-?\d+\.\d{4}", v) for v in vals)
    # rows that are deliberate skips keep the reference's status
    status = {(t, m[0]): m[1] for _, t, _, ms in rows for m in ms}
    assert status[("kernel_launch_latency", "dispatch")] == "unsupported"
    assert status[("image_memory_bandwidth", "float4")] == "unsupported"
    assert status[("wmma_fp16", "wmma_fp16")] == "unsupported"
    assert status[("rocblas-fp", "bf16")] is None and status[("rocblas-fp", "fp32")] is None and status[("rocblas-fp", "fp64")] is None
    assert status[("hipblaslt-fp8", "fp8_e4m3")] is None


def test_text_table_format():
    r = run_cli("--single-precision-compute", "--global-memory-bandwidth")
    out = r.stdout
    assert "Single-precision compute (GFLOPS)" in out and "Global memory bandwidth (GBPS)" in out
    assert re.search(r"^\s+float    : \d+\.\d\d$", out, re.M) and re.search(r"^\s+float4   : \d+\.\d\d$", out, re.M)
    assert "MFMA" not in out and "latency" not in out.lower()
    # the reference's layout (README.md:90-97, src/common/logger_text.cpp:58-100): device one step in, properties and
    # test headers at two, readings at three; property keys padded to 17 characters
    lines = out.splitlines()
    assert lines[0] == "Backend: ROCm" and lines[1] == "  Device 0: Fake MI355X"
    assert lines[2] == "    Driver version   : 7.2.0" and "    CUs              : 256" in lines
    assert "    Single-precision compute (GFLOPS)" in lines
    assert any(re.fullmatch(r"      float    : \d+\.\d\d", ln) for ln in lines)


def test_describe_prints_wrapped_notes_under_headers_and_readings():
    """--describe (src/common/logger_text.cpp:129-135, 238-243, 266-299): the test's description under its header,
    one step in from it, wrapped to 80 columns and followed by a blank line; each reading's note on the line(s)
    below the reading, flush with the value column; without the flag none of that text appears."""
    plain = run_cli("--single-precision-compute", "--kernel-launch-latency").stdout
    out = run_cli("--describe", "--single-precision-compute", "--kernel-launch-latency").stdout
    lines = out.splitlines()
    h = lines.index("    Single-precision compute (GFLOPS)")
    assert lines[h + 1].startswith("      Vector-ALU rate") and lines[h + 2].startswith("      ") and lines[h + 3] == ""
    desc = " ".join(ln.strip() for ln in lines[h + 1:h + 3])
    assert desc.endswith("nothing but registers involved.")
    assert all(len(ln) <= 80 for ln in lines)
    f = next(i for i, ln in enumerate(lines) if re.fullmatch(r"      float    : \d+\.\d\d", ln))
    assert lines[f + 1].startswith(" " * (6 + 8 + 3) + "One value per lane at a time.")
    # a skipped reading carries its note too
    d = next(i for i, ln in enumerate(lines) if ln.startswith("      dispatch  : [unsupported] "))
    assert lines[d + 1].startswith(" " * (6 + 9 + 3)) and lines[d + 1].strip()
    assert "Vector-ALU rate" not in plain and "One value per lane" not in plain
    reading = re.compile(r"      \S+ +: (\d|\[)")            # the rows themselves are the same with and without
    assert [ln for ln in plain.splitlines() if reading.match(ln)] == [ln for ln in lines if reading.match(ln)]


def test_allow_list_and_subtract_flags(tmp_path):
    x = tmp_path / "o.xml"
    run_cli("--mfma", "--xml-file", str(x))
    _, rows = parse_xml(x)
    tags = [t for _, t, _, _ in rows]
    assert tags[0] == "mfma_fp16" and "smfmac_int8" in tags and "mfma_int8" in tags     # Mfma gates dense and sparse, fp and int
    assert not any(t.startswith(("single", "rocblas", "global", "wmma")) for t in tags)
    run_cli("--no-mfma", "--no-int-compute", "--xml-file", str(x))
    _, rows = parse_xml(x)
    tags = [t for _, t, _, _ in rows]
    assert not any("mfma" in t for t in tags) and "integer_compute" not in tags and "rocblas-int" not in tags
    assert "rocblas-fp" in tags and "global_memory_bandwidth" in tags
    run_cli("--bandwidth", "--xml-file", str(x))
    _, rows = parse_xml(x)
    assert {c for c, _, _, _ in rows} == {"bandwidth"}


def test_no_device_is_a_note_and_status_zero():
    r = run_cli(env={"CLPEAK_FAKE_DEVICES": "0"})
    assert r.returncode == 0 and "ROCm: no devices found" in r.stdout and "Backend:" not in r.stdout


def test_list_devices():
    r = run_cli("--list-devices", env={"CLPEAK_FAKE_DEVICES": "2"})
    assert r.returncode == 0 and "=== ROCm backend ===" in r.stdout
    assert "ROCm Device 0: Fake MI355X [GPU]" in r.stdout and "ROCm Device 1: Fake MI355X [GPU]" in r.stdout
    assert "no devices found" in run_cli("--list-devices", env={"CLPEAK_FAKE_DEVICES": "0"}).stdout


def test_device_selection(tmp_path):
    x = tmp_path / "o.xml"
    r = run_cli("--rocm-device", "1", "--kernel-launch-latency", "--xml-file", str(x), env={"CLPEAK_FAKE_DEVICES": "3"})
    assert r.stdout.count("Device 1:") == 1 and "Device 0:" not in r.stdout and "Device 2:" not in r.stdout
    r = run_cli("--rocm-device", "99", "--kernel-launch-latency")
    assert r.returncode == 0 and "Device" not in r.stdout
    assert run_cli("--rocm-device", "x").returncode == 1
    assert run_cli("--no-such-flag").returncode == 1


@pytest.mark.parametrize("entry,tag,metric", [("mfma_dense", "mfma_bf16", "mfma_bf16"), ("gemm_bf16", "rocblas-fp", "bf16"),
                                              ("gemm_f16", "rocblas-fp", "fp16"), ("fill_i8", "rocblas-int", "int8"),
                                              ("gemm_fp8_e5m2", "hipblaslt-fp8", "fp8_e5m2"), ("gemm_mxfp4", "hipblaslt-fp8", "mxf4_e2m1"),
                                              ("local_bandwidth", "local_memory_bandwidth", "float2"),
                                              ("host_alloc", "transfer_bandwidth", "h2d_pinned"),
                                              ("copy_async", "transfer_bandwidth", "d2h_pinned"),
                                              ("global_bandwidth", "global_memory_bandwidth", "float4"),
                                              ("alloc", "single_precision_compute", "float"),
                                              ("launch_roundtrip", "kernel_launch_latency", "roundtrip")])
def test_failures_degrade_to_error_rows(tmp_path, entry, tag, metric):
    """Any failing device call becomes an `error` row for the readings it affects; the run goes on."""
    x = tmp_path / "o.xml"
    r = run_cli("--xml-file", str(x), env={"CLPEAK_FAKE_FAIL": entry})
    assert r.returncode == 0
    _, rows = parse_xml(x)
    assert [t for _, t, _, _ in rows] == [t for t, _, _ in EXPECTED_ROWS]      # same test set, same order
    status = {(t, m[0]): m[1] for _, t, _, ms in rows for m in ms}
    assert status[(tag, metric)] == "error"
    assert status[("kernel_launch_latency", "dispatch")] == "unsupported"


def test_dump_formats_round_trip(tmp_path):
    x, j, c = tmp_path / "a.xml", tmp_path / "a.json", tmp_path / "a.csv"
    r = run_cli("--xml-file", str(x), "--json-file", str(j), "--csv-file", str(c), env={"CLPEAK_FAKE_FAIL": "smfmac"})
    assert r.returncode == 0
    # JSON: one entry object per line, reference field names
    import json
    doc = json.loads(j.read_text())
    assert doc["format_version"] == 2 and doc["devices"][0]["props"][0] == {"k": "Arch", "v": "gfx950:sramecc+:xnack-"}
    _, rows = parse_xml(x)
    n_metrics = sum(len(ms) for _, _, _, ms in rows)
    assert len(doc["entries"]) == n_metrics
    ok = [e for e in doc["entries"] if "value" in e]
    bad = [e for e in doc["entries"] if "status" in e]
    assert len(ok) + len(bad) == n_metrics and all("reason" in e for e in bad) and all("status" not in e for e in ok)
    assert {e["status"] for e in bad} == {"unsupported", "error"}
    assert set(ok[0]) >= {"backend", "platform", "device", "driver", "category", "test", "metric", "unit", "display", "value"}
    # CSV: header + one row per metric, format_version first, 15 columns
    lines = c.read_text().strip().split("\n")
    assert lines[0].startswith("format_version,backend,platform,device,driver,category,test,metric,unit,status,value,reason")
    assert len(lines) == n_metrics + 1 and all(l.startswith("2,ROCm,ROCm,Fake MI355X,") for l in lines[1:])
    # --compare against its own dump prints a zero delta on every measured row (loader round trip)
    for f in (x, j, c):
        r2 = run_cli("--compare", str(f), "--single-precision-compute")
        assert r2.stdout.count("(was 83.89, ") == 3 and r2.stdout.count("0.0%)") == 3, f


def test_reference_result_files_load(tmp_path):
    """A result file in the reference's own XML grammar (written out here by hand from its
    documented tree) loads through --compare and matches on the row key."""
    ref = tmp_path / "ref.xml"
    ref.write_text('<?xml version="1.0" encoding="utf-8"?>\n<clpeak format_version="2" clpeak_version="2.0.16" os="Linux x64">\n'
                   '  <run backend="ROCm" platform="ROCm" device="Fake MI355X" driver="6.0.0">\n    <prop name="CUs" value="256"/>\n'
                   '    <category name="fp_compute">\n      <test name="single_precision_compute" display="Single-precision compute" unit="gflops">\n'
                   '        <metric name="float" info="x &amp; y">41.9431</metric>\n        <metric name="float2" status="unsupported" reason="n/a"/>\n'
                   '      </test>\n    </category>\n  </run>\n</clpeak>\n')
    r = run_cli("--compare", str(ref), "--single-precision-compute")
    assert r.stdout.count("(was 41.94, +100.0%)") == 1 and r.stdout.count("(was ") == 1
    old = tmp_path / "v1.xml"
    old.write_text('<clpeak format_version="1">\n<run backend="ROCm" platform="ROCm" device="Fake MI355X" driver="1">\n</run></clpeak>\n')
    assert "(was" not in run_cli("--compare", str(old), "--single-precision-compute").stdout


# ---- pieces reached through the host library --------------------------------------------------------
@pytest.fixture(scope="module")
def host():
    L = C.CDLL(HOSTLIB)
    L.clpeak_host_pick_iters.argtypes = [C.c_double, C.c_uint, C.c_uint, C.c_uint]; L.clpeak_host_pick_iters.restype = C.c_uint
    L.clpeak_host_target_global_threads.argtypes = [C.c_uint]; L.clpeak_host_target_global_threads.restype = C.c_ulonglong
    L.clpeak_host_seeded_operand.argtypes = [C.c_int, C.c_double, C.c_ulonglong, C.c_uint, C.c_ulonglong, C.c_void_p, C.c_size_t]
    L.clpeak_host_seeded_operand.restype = C.c_size_t
    L.clpeak_host_seeded_bytes.argtypes = [C.c_int, C.c_ulonglong, C.c_uint, C.c_ulonglong, C.c_void_p]
    L.clpeak_host_seeded_bytes.restype = C.c_size_t
    return L


def test_pick_iters_and_launch_width(host):
    """Calibration rules of the reference (src/common/common.cpp:35-45, include/common/common.h:142-147)."""
    p = host.clpeak_host_pick_iters
    assert p(100.0, 500000, 0, 10000) == 5000
    assert p(0.01, 500000, 0, 10000) == 10000            # sub-microsecond probes count as 1 us, then the cap
    assert p(1e9, 500000, 0, 10000) == 1                 # one launch already over budget
    assert p(100.0, 500000, 7, 10000) == 7               # --iters wins
    assert p(1000.0, 0, 0, 10000) == 5000                # 0 = the legacy 5 s budget
    assert p(1.0, 2000000, 0, 100000000) == 2000000      # the CPU harness' larger cap
    assert host.clpeak_host_target_global_threads(256) == 256 * 2048 * 256
    assert host.clpeak_host_target_global_threads(4) == 32 << 20


@pytest.mark.parametrize("fmt,ofmt,sigma", [(0, orc.FMT_F16, 0.01), (1, orc.FMT_BF16, 0.01), (2, orc.FMT_E4M3, 1.0),
                                            (3, orc.FMT_E5M2, 1.0), (4, orc.FMT_E2M3, 1.0), (5, orc.FMT_E3M2, 1.0),
                                            (6, orc.FMT_E2M1, 1.0), (2, orc.FMT_E4M3, 300.0), (0, orc.FMT_F16, 3e4)])
def test_host_operand_generator_matches_oracle(host, fmt, ofmt, sigma):
    """The backend's own host-side generator and the oracle's produce the same operand bytes."""
    n, seed, stream = 8192, wl.DEFAULT_SEED, wl.STREAM_MFMA_A
    bits = {0: 16, 1: 16, 2: 8, 3: 8, 4: 6, 5: 6, 6: 4}[fmt]
    buf = np.zeros(n * bits // 8, dtype=np.uint8)
    assert host.clpeak_host_seeded_operand(fmt, sigma, seed, stream, n, buf.ctypes.data, buf.size) == buf.size
    codes = orc.fill_normal_codes(ofmt, sigma, seed, stream, n)
    ref = codes.view(np.uint8) if bits in (8, 16) else orc.pack_bits(codes, bits)
    assert np.array_equal(buf, ref)


def test_host_int8_scales_and_sparse_metadata_match_oracle(host):
    n, seed = 4096, wl.DEFAULT_SEED
    buf = np.zeros(n, dtype=np.uint8)
    host.clpeak_host_seeded_operand(7, 0.0, seed, wl.STREAM_MFMA_B, n, buf.ctypes.data, n)
    assert np.array_equal(buf.view(np.int8), orc.fill_int8(seed, wl.STREAM_MFMA_B, n))
    host.clpeak_host_seeded_bytes(0, seed, wl.STREAM_SCALE_A, n, buf.ctypes.data)
    assert np.array_equal(buf, orc.fill_e8m0(seed, wl.STREAM_SCALE_A, n))
    host.clpeak_host_seeded_bytes(1, seed, wl.STREAM_SPARSE, n, buf.ctypes.data)
    assert np.array_equal(buf, orc.fill_sparse_meta(seed, wl.STREAM_SPARSE, n))


def test_backend_workloads_equal_oracle_workloads():
    """clpeak_amd.workloads (what bench.py hands the kernels) and oracle.workloads (what the parity tests
    hand the kernels and the oracle) describe the same kinds and build the same bytes."""
    from clpeak_amd import workloads as pw
    assert sorted(pw.DENSE) == sorted(wl.DENSE) and sorted(pw.SPARSE) == sorted(wl.SPARSE)
    for kind in pw.DENSE:
        for key in ("name", "shape", "M", "N", "K", "scaled"):
            assert pw.DENSE[kind][key] == wl.DENSE[kind][key]
        for got, ref in zip(pw.dense_inputs(kind, 8), wl.dense_inputs(kind, 8)):
            assert (got is None and ref is None) or np.array_equal(got, ref.view(np.uint8))
        assert pw.dense_flops(kind, 2048, 4096) == wl.dense_flops(kind, 2048, 4096)
    for kind in pw.SPARSE:
        assert pw.SPARSE[kind]["name"] == wl.SPARSE[kind]["name"] and pw.SPARSE[kind]["K"] == wl.SPARSE[kind]["K"]
        for got, ref in zip(pw.sparse_inputs(kind, 8), wl.sparse_inputs(kind, 8)):
            assert np.array_equal(got, ref.view(np.uint8))
        assert pw.sparse_flops(kind, 2048, 4096) == wl.sparse_flops(kind, 2048, 4096)
    assert [getattr(pw, n) for n in dir(pw) if n.startswith("STREAM_")] == [getattr(wl, n) for n in dir(pw) if n.startswith("STREAM_")]


def test_reference_operands(host, tmp_path):
    """--reference-operands: the host generator's constants are the codes listed for the reference's kernels,
    in the packing of the seeded operands, and the flag leaves the row set as it is."""
    from clpeak_amd import workloads as pw
    for fmt, code in pw.REFERENCE_CODE.items():
        n = 256
        assert np.array_equal(pw.reference_operand(fmt, n), pw.constant_operand(fmt, code, n)), fmt
    # decoded through the oracle's format tables: the values the closed forms of the GPU tests use
    for fmt, ofmt in ((pw.F16, orc.FMT_F16), (pw.BF16, orc.FMT_BF16), (pw.E4M3, orc.FMT_E4M3), (pw.E5M2, orc.FMT_E5M2),
                      (pw.E2M3, orc.FMT_E2M3), (pw.E3M2, orc.FMT_E3M2), (pw.E2M1, orc.FMT_E2M1)):
        dt = np.uint16 if ofmt in (orc.FMT_F16, orc.FMT_BF16) else np.uint8
        assert orc.decode(ofmt, np.array([pw.REFERENCE_CODE[fmt]], dtype=dt))[0] == pw.REFERENCE_VALUE[fmt], fmt
    a, b = tmp_path / "seeded.xml", tmp_path / "reference.xml"
    assert run_cli("--xml-file", str(a)).returncode == 0
    assert run_cli("--reference-operands", "--xml-file", str(b)).returncode == 0
    rows = lambda p: [(c, t, u, [(m, s) for m, s, _ in ms]) for c, t, u, ms in parse_xml(p)[1]]
    assert rows(a) == rows(b)
    assert "--reference-operands" in subprocess.run([CLI, "--help"], capture_output=True, text=True).stdout


# ---- the reference's own result files (tests/golden/reference_results_*.xml, copied as data from its results/) ----
GOLDEN = os.path.join(ROOT, "tests", "golden")


@pytest.mark.parametrize("name,rows", [("reference_results_amd_threadripper.xml", 192),
                                       ("reference_results_nvidia_rtx5060.xml", 217),
                                       ("reference_results_apple_m1pro.xml", 212)])
def test_reference_result_files_survive_load_and_save_byte_for_byte(host, tmp_path, name, rows):
    """The three result files the reference ships were written by its own result store.  Loading one here
    and saving it again must give the same bytes, line for line, but for the root element (which names
    the writing program's version and OS): that pins the loader (every attribute, status, reason, prop,
    entity) and the writer (order, indentation, escaping, number format) to the reference's at once.
    The same rows then go through this backend's JSON and come back unchanged."""
    host.clpeak_host_resave.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    src = os.path.join(GOLDEN, name)
    out = tmp_path / "again.xml"
    assert host.clpeak_host_resave(src.encode(), str(out).encode(), 0) == rows
    want, got = open(src, encoding="utf-8").read().split("\n"), out.read_text(encoding="utf-8").split("\n")
    assert len(want) == len(got)
    assert want[1].startswith("<clpeak format_version=\"2\"") and got[1].startswith("<clpeak format_version=\"2\"")
    assert want[:1] + want[2:] == got[:1] + got[2:]
    # XML -> JSON -> XML
    js, back = tmp_path / "again.json", tmp_path / "back.xml"
    assert host.clpeak_host_resave(src.encode(), str(js).encode(), 1) == rows
    assert host.clpeak_host_resave(str(js).encode(), str(back).encode(), 0) == rows
    assert back.read_text(encoding="utf-8") == out.read_text(encoding="utf-8")
    doc = json.loads(js.read_text(encoding="utf-8"))
    assert doc["format_version"] == 2
    # CSV keeps every row (it has no device properties)
    assert host.clpeak_host_resave(src.encode(), str(tmp_path / "again.csv").encode(), 2) == rows
    assert host.clpeak_host_resave(str(tmp_path / "again.csv").encode(), str(tmp_path / "c.xml").encode(), 0) == rows


def test_shipped_mi355x_result_file_has_the_row_contract():
    """results/AMD/Instinct_MI355X.xml is a dump of a full run of this backend on an MI355X (the reference keeps
    such files under results/<vendor>/): same tests, units and metrics, in the same order, as the stand-in run."""
    path = os.path.join(ROOT, "results", "AMD", "Instinct_MI355X.xml")
    root, rows = parse_xml(path)
    assert root.get("format_version") == "2"
    run = root.find("run")
    assert run.get("backend") == "ROCm" and [p.get("name") for p in run.findall("prop")] == ["Arch", "HIP", "CUs", "Wave", "VRAM"]
    assert [(t, u, [m[0] for m in ms]) for _, t, u, ms in rows] == EXPECTED_ROWS
    measured = {(t, m[0]): float(m[2]) for _, t, _, ms in rows for m in ms if m[1] is None}
    assert measured[("global_memory_bandwidth", "float4")] > 6800.0          # 85 % of 8 TB/s
    assert measured[("mfma_bf16", "mfma_bf16")] > 2125.0 and measured[("mfma_int8", "mfma_int8")] > 4250.0


# Rows with a line in the MI355X datasheet: (test, metric) -> (peak in the row's unit).  Dense matrix peaks; the
# 2:4 sparse ones are twice those.
DATASHEET = {("single_precision_compute", "float"): 157300.0, ("single_precision_compute", "float4"): 157300.0,
             ("double_precision_compute", "double2"): 78600.0,
             ("mfma_fp16", "mfma_fp16"): 2500.0, ("mfma_bf16_32x32x16", "mfma_bf16_32x32x16"): 2500.0,
             ("mfma_fp8", "mfma_fp8"): 5000.0, ("mfma_bf8", "mfma_bf8"): 5000.0, ("mfma_int8", "mfma_int8"): 5000.0,
             ("mfma_mxfp6_e2m3", "mfma_mxfp6_e2m3"): 10100.0, ("mfma_mxfp4", "mfma_mxfp4"): 10100.0,
             ("smfmac_fp16", "smfmac_fp16"): 5000.0, ("smfmac_bf8", "smfmac_bf8"): 10000.0, ("smfmac_int8", "smfmac_int8"): 10000.0,
             ("rocblas-fp", "fp32"): 157.3, ("rocblas-fp", "fp64"): 78.6, ("rocblas-fp", "bf16"): 2500.0,
             ("hipblaslt-fp8", "fp8_e4m3"): 5000.0, ("hipblaslt-fp8", "mxf4_e2m1"): 10100.0, ("rocblas-int", "int8"): 5000.0,
             ("global_memory_bandwidth", "float"): 8000.0, ("global_memory_bandwidth", "float4"): 8000.0}


def _infos(path):
    out = {}
    for run in ET.parse(path).getroot().findall("run"):
        for test in run.iter("test"):
            for m in test.findall("metric"):
                out[(test.get("name"), m.get("name"))] = (m.get("status"), m.text, m.get("info") or "")
    return out


def _check_percent_notes(infos):
    for key, peak in DATASHEET.items():
        status, text, info = infos[key]
        assert status is None, key
        m = re.search(r"(\d+\.\d) % of the MI355X datasheet peak \(([\d.]+) ", info)
        assert m, (key, info)
        assert float(m.group(2)) == peak, (key, info)
        assert abs(float(m.group(1)) - 100.0 * float(text) / peak) <= 0.051, (key, info, text)
    # rows without a datasheet line carry no percentage
    for key in (("half_precision_compute", "half2"), ("integer_compute", "int4"), ("local_memory_bandwidth", "float4"),
                ("transfer_bandwidth", "h2d_pinned"), ("kernel_launch_latency", "roundtrip")):
        assert "datasheet" not in infos[key][2], key
    # every family explains its own widths: no accumulators on the rows that load or pass data
    for test in ("global_memory_bandwidth", "local_memory_bandwidth"):
        for metric in ("float", "float2", "float4"):
            info = infos[(test, metric)][2]
            assert "accumulator" not in info and "bytes) per lane" in info, (test, metric, info)
    assert "per lane and load instruction" in infos[("global_memory_bandwidth", "float4")][2]
    assert "LDS store and load" in infos[("local_memory_bandwidth", "float2")][2]
    assert "4 operations per instruction" in infos[("bfloat16_compute", "bf16")][2]


def test_measured_rows_carry_their_fraction_of_the_datasheet_peak(tmp_path):
    """Each reading with a datasheet line says what fraction of it was reached, in the one free-text field of a reading
    (EmitOptions::description, include/common/logger.h:121-128, rendered by src/common/logger_text.cpp:238-243);
    tags, metrics and units stay the reference's."""
    x = tmp_path / "pct.xml"
    assert run_cli("--xml-file", str(x)).returncode == 0
    _check_percent_notes(_infos(x))
    shown = run_cli("--describe", "--global-memory-bandwidth").stdout
    assert "% of the MI355X datasheet" in " ".join(shown.split())


def test_shipped_mi355x_result_file_carries_percentages_and_clocks():
    infos = _infos(os.path.join(ROOT, "results", "AMD", "Instinct_MI355X.xml"))
    _check_percent_notes(infos)
    for key in (("mfma_fp16", "mfma_fp16"), ("smfmac_int8", "smfmac_int8"), ("mfma_mxfp4", "mfma_mxfp4")):
        m = re.search(r"shader clock held: (\d+) MHz", infos[key][2])
        assert m and 1000 <= int(m.group(1)) <= 2500, (key, infos[key][2])


def test_the_product_holds_no_pretend_device(tmp_path):
    """The program and the library that ship know one device table, the entry points of libclpeak_mi355.so:
    no symbol or string of the tests' pretend device, no flag and no environment switch that selects one."""
    shipped_cli = os.path.join(ROOT, "clpeak_amd", "clpeak-mi355")
    for binary in (shipped_cli, HOSTLIB, os.path.join(ROOT, "clpeak_amd", "libclpeak_mi355.so")):
        syms = subprocess.run(["nm", "-D", "--defined-only", binary], capture_output=True, text=True).stdout
        assert "fake" not in syms.lower(), binary
        blob = open(binary, "rb").read().lower()
        assert b"fake" not in blob and b"clpeak_fake" not in blob, binary
    r = subprocess.run([shipped_cli, "--fake-device"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "--fake-device" in r.stderr
    # and the environment cannot conjure a device: on a machine without a GPU the shipped program lists none
    e = dict(os.environ, CLPEAK_FAKE_DEVICES="2")
    r = subprocess.run([shipped_cli, "--list-devices"], capture_output=True, text=True, env=e, timeout=60)
    assert "Fake" not in r.stdout
