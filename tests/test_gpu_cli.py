"""The CLI on a real MI355X: every row the backend measures comes back as a number, the rest
as the documented skips, and the XML loads."""
import os
import subprocess
import xml.etree.ElementTree as ET

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "clpeak_amd", "clpeak-mi355")


def test_cli_small_shapes_all_rows(tmp_path):
    x = tmp_path / "gpu.xml"
    r = subprocess.run([CLI, "--small-shapes", "--max-time", "20", "--xml-file", str(x)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    root = ET.parse(x).getroot()
    run = root.find("run")
    assert run.get("backend") == "ROCm"
    props = {p.get("name"): p.get("value") for p in run.findall("prop")}
    assert props["Arch"].startswith("gfx950") and int(props["CUs"]) >= 64 and props["Wave"] == "64"
    measured, skipped = {}, {}
    for test in run.iter("test"):
        for m in test.findall("metric"):
            (skipped if m.get("status") else measured)[(test.get("name"), m.get("name"))] = m.get("status") or float(m.text)
    assert not [k for k, v in skipped.items() if v == "error"], skipped
    for key in [("single_precision_compute", "float4"), ("half_precision_compute", "half2"), ("double_precision_compute", "double"),
                ("mixed_precision_compute", "mp"), ("bfloat16_compute", "bf16"), ("integer_compute", "int4"),
                ("integer_compute_int8_dp", "int8_dp8"), ("mfma_fp16", "mfma_fp16"), ("mfma_bf16_32x32x16", "mfma_bf16_32x32x16"),
                ("mfma_int8", "mfma_int8"), ("mfma_fp8", "mfma_fp8"), ("mfma_mxfp6_e2m3", "mfma_mxfp6_e2m3"),
                ("mfma_mxfp4", "mfma_mxfp4"), ("smfmac_fp16", "smfmac_fp16"), ("smfmac_int8", "smfmac_int8"),
                ("rocblas-fp", "bf16"), ("hipblaslt-fp8", "fp8_e4m3"), ("global_memory_bandwidth", "float4"),
                ("kernel_launch_latency", "roundtrip")]:
        assert measured.get(key, 0) > 0, key
    assert skipped[("kernel_launch_latency", "dispatch")] == "unsupported"


def test_cli_reference_operands(tmp_path):
    """The matrix rows on the constants the reference's kernels run on: all measured, none an error."""
    x = tmp_path / "ref.xml"
    r = subprocess.run([CLI, "--small-shapes", "--reference-operands", "--max-time", "20", "--no-bandwidth", "--no-latency",
                        "--xml-file", str(x)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    run = ET.parse(x).getroot().find("run")
    got = {(t.get("name"), m.get("name")): (m.get("status"), m.text) for t in run.iter("test") for m in t.findall("metric")}
    assert not [k for k, (status, _) in got.items() if status == "error"], got
    for key in [("mfma_bf16", "mfma_bf16"), ("mfma_mxfp4", "mfma_mxfp4"), ("smfmac_fp8", "smfmac_fp8"), ("smfmac_int8", "smfmac_int8"),
                ("rocblas-fp", "fp64"), ("rocblas-fp", "bf16"), ("hipblaslt-fp8", "mxf4_e2m1"), ("rocblas-int", "int8")]:
        assert got[key][0] is None and float(got[key][1]) > 0, key


def test_cli_list_devices():
    r = subprocess.run([CLI, "--list-devices"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "=== ROCm backend ===" in r.stdout and "ROCm Device 0:" in r.stdout and "[GPU]" in r.stdout
