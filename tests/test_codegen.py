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
    """{kernel name: {field: int}} from the amdhsa.kernels metadata block (one YAML list item per kernel)."""
    meta, item = {}, None
    fields = r"(vgpr_count|vgpr_spill_count|sgpr_spill_count|agpr_count|private_segment_fixed_size|group_segment_fixed_size)"
    for line in asm.splitlines():
        if re.match(r"  - \.\w+:", line):               # "  - .key: value" at list depth opens the next kernel's item
            item = {}
        if item is None:
            continue
        m = re.match(r"\s+(?:-\s+)?\." + fields + r":\s+(\d+)", line)
        if m:
            item[m.group(1)] = int(m.group(2))
        m = re.match(r"\s+(?:-\s+)?\.name:\s+(\S+)", line)
        if m and "kernel" in m.group(1):
            meta[m.group(1)] = item
    return meta


def kernel_body(asm, name):
    start = asm.index("\n" + name + ":") + 1
    return asm[start:asm.index(".Lfunc_end", start)]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_kernels_fit_the_register_file(tmp_path):
    asm = device_asm(tmp_path, "gemm.hip")
    meta = kernel_metadata(asm)
    # (kernel template, instantiation tag in the mangled name) -> the matrix instruction of its loop and how
    # many of them the one instance of the step holds: 32 slots, one fp8 instruction or a pair per slot
    expect = {("gemm_ring_kernel", "ILi0E"): ("v_mfma_f32_16x16x128_f8f6f4", 32),
              ("gemm_ring_kernel", "ILi1E"): ("v_mfma_f32_16x16x128_f8f6f4", 32),
              ("gemm_ring_kernel", "ILi2E"): ("v_mfma_f32_16x16x32_bf16", 64),
              ("gemm_ring_kernel", "ILi3E"): ("v_mfma_f32_16x16x32_f16", 64),
              ("gemm_ring_kernel", "ILi4E"): ("v_mfma_i32_16x16x64_i8", 64)}
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
        if tag == "ILi1E":
            assert body.count("blgp:1") == count      # the e5m2 operand is the second source
        if count == 64:   # a pair is issued back to back on one accumulator: same destination twice in a row
            dst = re.findall(insn + r" (v\[\d+:\d+\]),", body)
            assert len(dst) == 64 and all(dst[2 * k] == dst[2 * k + 1] for k in range(32)), name
        # the direct-to-LDS loads: 20 in the prologue (five ring slots) + 8 per steady-state step
        assert body.count("global_load_lds_dwordx4") >= 20 + 8, name
        # no LDS stores at all on this path
        assert "ds_write" not in body, name
        # the accumulators leave through the packed conversions, two values per instruction
        if tag != "ILi4E":
            cvt = "v_cvt_pk_f16_f32" if tag == "ILi3E" else "v_cvt_pk_bf16_f32"
            assert body.count(cvt) == 64, (name, body.count(cvt))   # 32 tiles x 4 values per lane


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("source", ["mfma_dense.hip", "smfmac.hip"])
def test_peak_loops_do_not_spill(tmp_path, source):
    meta = kernel_metadata(device_asm(tmp_path, source))
    assert meta, "no kernels found"
    for name, m in meta.items():
        assert m.get("vgpr_spill_count", 0) == 0, (name, m)
        assert m.get("private_segment_fixed_size", 0) == 0, (name, m)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_mxfp4_instantiation_of_the_ring_kernel(tmp_path):
    """The block-scaled kind adds 12 scale registers (this step's and the next step's, written asynchronously by
    loads) to the 128 accumulators and 96 fragment registers: it must still fit 256 without a spill."""
    asm = device_asm(tmp_path, "gemm.hip")
    meta = kernel_metadata(asm)
    name = next(k for k in meta if "gemm_ring_kernelILi5E" in k)
    m = meta[name]
    assert m["vgpr_spill_count"] == 0 and m["private_segment_fixed_size"] == 0 and m["vgpr_count"] <= 256, m
    body = kernel_body(asm, name)
    insn = "v_mfma_scale_f32_16x16x128_f8f6f4"
    assert body.count(insn) == 64 and body.count("cbsz:4 blgp:4") == 64
    # a slot is its two K halves back to back on one accumulator, scale byte picked by op_sel
    ops = re.findall(insn + r" (v\[\d+:\d+\]), .* op_sel:\[(\d),(\d),0\]", body)
    assert len(ops) == 64
    assert all(ops[2 * k][0] == ops[2 * k + 1][0] and ops[2 * k][1:] == ("0", "0") and ops[2 * k + 1][1:] == ("1", "1") for k in range(32))
    # per step: one 16-byte load of A scales and one 8-byte load of B scales (+ the same two before the loop)
    assert len(re.findall(r"global_load_dwordx4 v\[", body)) == 2 and len(re.findall(r"global_load_dwordx2 v\[", body)) == 2
    assert body.count("v_cvt_pk_bf16_f32") == 64 and "ds_write" not in body
    # the pre-pass and the entry point live in gemm_mxfp4.hip
    meta = kernel_metadata(device_asm(tmp_path, "gemm_mxfp4.hip"))
    assert any("mx_scale_layout_kernel" in k for k in meta)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_fp32_and_fp64_kernels(tmp_path):
    """fp32: the ring kernel with four 16x16x4 instructions per 16-byte fragment read, 256 per step.
    fp64: 64 instructions per step in two halves around the barrier, two 32 KiB buffers (64 KiB static LDS, two
    workgroups per CU)."""
    asm = device_asm(tmp_path, "gemm.hip")
    meta = kernel_metadata(asm)
    name = next(k for k in meta if "gemm_f32_kernel" in k)
    assert meta[name]["vgpr_spill_count"] == 0 and meta[name]["private_segment_fixed_size"] == 0 and meta[name]["vgpr_count"] <= 256
    body = kernel_body(asm, name)
    assert body.count("v_mfma_f32_16x16x4_f32") == 256 and "ds_write" not in body
    asm = device_asm(tmp_path, "gemm_f64.hip")
    meta = kernel_metadata(asm)
    name = next(k for k in meta if "gemm_f64_kernel" in k)
    assert meta[name]["vgpr_spill_count"] == 0 and meta[name]["private_segment_fixed_size"] == 0 and meta[name]["vgpr_count"] <= 256
    assert meta[name]["group_segment_fixed_size"] == 65536
    body = kernel_body(asm, name)
    assert body.count("v_mfma_f64_16x16x4_f64") == 64 and "ds_write" not in body
    # the order of a step: the 8 reads of the second K half, a counted wait, the 32 instructions of the first
    # half ahead of the wait for everything and the barrier; then the next slab's loads and first-half reads
    # under the 32 instructions of the second half
    marks = []
    for line in body.split("\n"):
        t = line.strip()
        marks.append("M" if t.startswith("v_mfma_f64") else "B" if t.startswith("s_barrier") else "r" if t.startswith("ds_read_b128")
                     else "w" if t.startswith("s_waitcnt") else "L" if t.startswith("global_load_lds") else "")
    order = "".join(marks)
    assert "r" * 8 + "w" + "M" * 32 + "wB" in order, order
    assert order.count("M" * 32) == 2 and order.count("B") == 2


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_mixed_precision_mad_loops_run_on_the_mixed_instructions(tmp_path):
    """The `mp` row's loop is v_fma_mix_f32 (half sources widened by the instruction, fp32 result) and the `bf16`
    row's loop is v_dot2_f32_bf16; no plain fp32 multiply-add does the work of either, the block round trips are
    there (one conversion per accumulator per block), and nothing spills."""
    asm = device_asm(tmp_path, "compute_mad.hip")
    meta = kernel_metadata(asm)
    mp = next(n for n in meta if "mad_mp_kernel" in n)
    bf = next(n for n in meta if "mad_bf16_kernel" in n)
    for name in (mp, bf):
        assert meta[name].get("vgpr_spill_count", 0) == 0 and meta[name].get("private_segment_fixed_size", 0) == 0, meta[name]
    body = kernel_body(asm, mp)
    # 16 accumulators x (16 steps of a block, entered from fp32 or from the half of the last round trip, + the tail loop)
    assert body.count("v_fma_mix_f32") == 16 * 16 + 16 + 16, body.count("v_fma_mix_f32")
    assert body.count("op_sel_hi:[1,1,1]") == 16          # the first step of a block reads the chain value as half
    assert body.count("v_cvt_f16_f32") >= 16
    assert not re.search(r"\bv_(fma|fmac|fmamk|fmaak|mad|mac)_f32\b", body)
    body = kernel_body(asm, bf)
    assert body.count("v_dot2_f32_bf16") == 16 * 16 + 16, body.count("v_dot2_f32_bf16")
    assert not re.search(r"\bv_(fma|fmac|fmamk|fmaak|mad|mac)_f32\b", body)
