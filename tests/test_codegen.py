"""Properties of the generated gfx950 code that the hand-scheduled kernels rely on.

The GEMM loop issues its LDS reads as inline assembly whose results arrive asynchronously; a
register spill of such a result would be stored before the data has landed.  The kernel is therefore
only correct when it fits the register file, which the compiler reports in the code object
metadata.  hipcc cross-compiles without a GPU, so this runs on the CPU.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "clpeak_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-S", "--cuda-device-only", "-Wno-unused-command-line-argument"]


def device_asm(tmp_path, source):
    out = tmp_path / (source + ".s")
    subprocess.run([HIPCC, *FLAGS, os.path.join(CSRC, source), "-o", str(out)], check=True,
                   capture_output=True, timeout=600)
    return out.read_text()


def kernel_metadata(asm):
    """{kernel name: {field: int}} from the amdhsa.kernels metadata block."""
    meta, cur = {}, None
    for line in asm.splitlines():
        m = re.match(r"\s+\.name:\s+(\S+)", line)
        if m and "kernel" in m.group(1):
            cur = meta.setdefault(m.group(1), {})
        m = re.match(r"\s+\.(vgpr_count|vgpr_spill_count|sgpr_spill_count|agpr_count|"
                     r"private_segment_fixed_size|group_segment_fixed_size):\s+(\d+)", line)
        if m and cur is not None:
            cur[m.group(1)] = int(m.group(2))
    return meta


def kernel_body(asm, name):
    start = asm.index("\n" + name + ":") + 1
    return asm[start:asm.index(".Lfunc_end", start)]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_kernels_fit_the_register_file(tmp_path):
    asm = device_asm(tmp_path, "gemm.hip")
    meta = kernel_metadata(asm)
    # (kernel template, instantiation tag in the mangled name) -> the matrix instruction of its loop and how
    # many of them two instances of the step (steady state and tail) hold
    expect = {("gemm_bf16_kernel", "ILi0E"): ("v_mfma_f32_16x16x32_bf16", 128),
              ("gemm_bf16_kernel", "ILi1E"): ("v_mfma_f32_16x16x32_f16", 128),
              ("gemm_bf16_kernel", "ILi2E"): ("v_mfma_i32_16x16x64_i8", 128),
              ("gemm_fp8_kernel", "ILb0E"): ("v_mfma_f32_16x16x128_f8f6f4", 64),
              ("gemm_fp8_kernel", "ILb1E"): ("v_mfma_f32_16x16x128_f8f6f4", 64)}
    for (kernel, tag), (insn, count) in expect.items():
        name = next(k for k in meta if kernel + tag in k)
        m = meta[name]
        assert m["vgpr_spill_count"] == 0, (name, m)
        assert m["private_segment_fixed_size"] == 0, (name, m)
        # 8 waves per workgroup, 2 per SIMD: at most 256 registers each
        assert m["vgpr_count"] <= 256, (name, m)
        # the whole LDS of a CU is requested at launch (dynamic), none statically
        assert m.get("group_segment_fixed_size", 0) == 0, (name, m)
        body = kernel_body(asm, name)
        assert body.count(insn) == count, (name, body.count(insn))
        if tag == "ILb1E":
            assert body.count("blgp:1") == count      # the e5m2 operand is the second source
        # the direct-to-LDS loads: 20 in the prologue (five ring slots) + 8 per steady-state step
        assert body.count("global_load_lds_dwordx4") >= 20 + 8, name
        # no LDS stores at all on this path
        assert "ds_write" not in body, name


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("source", ["mfma_dense.hip", "smfmac.hip"])
def test_peak_loops_do_not_spill(tmp_path, source):
    meta = kernel_metadata(device_asm(tmp_path, source))
    assert meta, "no kernels found"
    for name, m in meta.items():
        assert m.get("vgpr_spill_count", 0) == 0, (name, m)
        assert m.get("private_segment_fixed_size", 0) == 0, (name, m)
