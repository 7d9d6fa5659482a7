"""The C-ABI library loads and exports every symbol include/clpeak_mi355.h declares.
No compute calls: this runs without a GPU."""
import os
import re

import pytest

from clpeak_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "clpeak_mi355.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_agree():
    assert declared_symbols() == sorted(capi.SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = capi.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_host_library_exports_every_declared_symbol():
    """libclpeak_host.so: the embedding ABI (clpeak_ffi.h) and the auxiliary one (clpeak_host.h)."""
    import ctypes as C
    lib = C.CDLL(os.path.join(ROOT, "clpeak_amd", "libclpeak_host.so"))
    exported = set()
    for header, prefix, count in (("clpeak_ffi.h", "clpeak_", 6), ("clpeak_host.h", "clpeak_host_", 10)):
        text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", header)).read(), flags=re.S)
        names = sorted(set(re.findall(r"\b(%s[a-z0-9_]+)\s*\(" % prefix, text)))
        assert len(names) == count, (header, names)
        for name in names:
            assert hasattr(lib, name), name
        exported |= set(names)
    # and nothing with the library's prefix is exported without being declared
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", lib._name], capture_output=True, text=True).stdout
    for sym in re.findall(r" T (clpeak_[a-z0-9_]+)", out):
        assert sym in exported, sym


def test_every_entry_point_cites_the_reference():
    """Each declaration is preceded by a comment naming the reference code it replaces
    (or saying that it has no counterpart)."""
    text = open(HEADER).read()
    for name in ("mi355_open", "mi355_global_bandwidth", "mi355_compute_mad", "mi355_launch_roundtrip",
                 "mi355_mfma_dense", "mi355_smfmac", "mi355_gemm_bf16", "mi355_timer_start", "mi355_fill_f32"):
        head = text[:text.index(name + "(")]
        section = head[head.rindex("/* ----"):]  # the section this declaration sits in
        assert re.search(r"src/(rocm|common)/[a-z_0-9/]+\.(cpp|hip):\d+", section), name


def test_constants_match_header():
    text = open(HEADER).read()
    defs = dict(re.findall(r"#define\s+(MI355_[A-Za-z0-9_]+)\s+\(?(-?\d+)\)?", text))
    assert int(defs["MI355_MFMA_KIND_COUNT"]) == 10 and int(defs["MI355_SMFMAC_KIND_COUNT"]) == 5
    for py, c in [("MAD_F32", "MI355_MAD_F32"), ("MAD_I8DP", "MI355_MAD_I8DP"), ("MFMA_MXFP4_E2M1", "MI355_MFMA_MXFP4_E2M1"),
                  ("MFMA_I8_16x16x64", "MI355_MFMA_I8_16x16x64"), ("SMFMAC_I8_16x16x128", "MI355_SMFMAC_I8_16x16x128"),
                  ("ERR_ARCH", "MI355_ERR_ARCH"), ("DIST_UPM1", "MI355_DIST_UPM1")]:
        assert getattr(capi, py) == int(defs[c]), (py, c)


def test_stream_ids_match_device_header():
    from oracle import workloads
    text = open(os.path.join(ROOT, "clpeak_amd", "csrc", "seeded_rng.h")).read()
    ids = dict(re.findall(r"(MI355_STREAM_[A-Z_]+)\s*=\s*(\d+)", text))
    for name, val in ids.items():
        short = name.replace("MI355_", "")
        assert getattr(capi, short) == int(val)
        assert getattr(workloads, short) == int(val)


def test_open_without_gpu_reports_no_device():
    """On a GPU-less host the library says so instead of crashing."""
    import ctypes as C
    lib = capi.load_library()
    n = C.c_int(-1)
    rc = lib.mi355_device_count(C.byref(n))
    if rc == capi.OK and n.value == 0:
        h = C.c_void_p()
        assert lib.mi355_open(0, C.byref(h)) == capi.ERR_NODEV
        assert b"no HIP device" in lib.mi355_last_error(None)
    else:
        pytest.skip("a GPU (or a failing runtime) is present; covered by the gpu tests")
