"""Properties of the generated gfx950 code that the hand-scheduled kernels rely on.

The GEMM loops issue their LDS reads as inline assembly whose results arrive asynchronously; a
register spill (or copy) of such a result would be taken before the data has landed.  The kernels are
therefore only correct when they fit the register file, which the compiler reports in the code object
metadata, and the four-wave kernel names its accumulation registers itself, which the instruction text shows.  hipcc cross-compiles without a GPU, so this runs on the CPU.
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


QUAD_KINDS = {  # instantiation tag in the mangled name -> (matrix instruction of the loop, how many per step and parity)
    "ILi0E": ("v_mfma_f32_16x16x128_f8f6f4", 64),
    "ILi1E": ("v_mfma_f32_16x16x128_f8f6f4", 64),
    "ILi2E": ("v_mfma_f32_16x16x32_bf16", 128),
    "ILi3E": ("v_mfma_f32_16x16x32_f16", 128),
    "ILi4E": ("v_mfma_i32_16x16x64_i8", 128),
    "ILi5E": ("v_mfma_scale_f32_16x16x128_f8f6f4", 128),
}


def _acc_range(text):
    lo, hi = (int(x, 0) for x in text.split(":"))
    return lo, hi


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_quad_kernels(tmp_path):
    """The four-wave kernel: the loop is written once per parity of the step, every matrix instruction accumulates in
    the accumulation registers the source names (all 256 of them, tile T in a[4T:4T+3]), nothing spills, and the
    compiler neither copies a fragment register nor touches an accumulation register of its own accord."""
    asm = device_asm(tmp_path, "gemm_quad.hip")
    meta = kernel_metadata(asm)
    for tag, (insn, per_step) in QUAD_KINDS.items():
        name = next(k for k in meta if "gemm_quad_kernel" + tag in k)
        m = meta[name]
        assert m["vgpr_spill_count"] == 0 and m.get("sgpr_spill_count", 0) == 0 and m["private_segment_fixed_size"] == 0, (name, m)
        # one wave per SIMD: up to 512 registers, 256 of them the accumulators
        assert m["agpr_count"] == 256 and m["vgpr_count"] <= 512, (name, m)
        assert m.get("group_segment_fixed_size", 0) == 0, (name, m)   # the whole LDS of a CU is requested at launch
        body = kernel_body(asm, name)
        acc = [_acc_range(x) for x in re.findall(insn + r" a\[([0-9a-fx]+:[0-9a-fx]+)\]", body)]
        assert len(acc) == 2 * per_step, (name, len(acc))
        for half in (acc[:per_step], acc[per_step:]):   # the step of parity 0, then of parity 1
            per_tile = per_step // 64
            assert [r for r in half[::per_tile]] == [(4 * t, 4 * t + 3) for t in range(64)], name
            if per_tile == 2:   # a pair is issued back to back on one accumulator
                assert half[0::2] == half[1::2], name
        # destination and addend are the same registers in every instruction
        assert len(re.findall(insn + r" a\[([0-9a-fx:]+)\], v\[\d+:\d+\], v\[\d+:\d+\], a\[\1\]", body)) == 2 * per_step, name
        if tag == "ILi1E":
            assert body.count("blgp:1") == 2 * per_step      # the e5m2 operand is the second source
        if tag == "ILi5E":
            assert body.count("cbsz:4 blgp:4") == 2 * per_step
            ops = re.findall(insn + r" .* op_sel:\[(\d),(\d),0\]", body)
            assert ops[0::2] == [("0", "0")] * per_step and ops[1::2] == [("1", "1")] * per_step, name
            # per step one 16-byte load of scale bytes per operand (+ the same two before the loop)
            assert len(re.findall(r"global_load_dwordx4 v\[", body)) == 2 * 3, name
        # direct-to-LDS loads: 32 before the loop (two slabs), 16 per step
        assert body.count("global_load_lds_dwordx4") == 32 + 2 * 16, (name, body.count("global_load_lds_dwordx4"))
        assert "ds_write" not in body and "scratch_" not in body, name
        # LDS reads: 16 + 2 * 2 before the loop, 32 per step
        assert body.count("ds_read_b128") == 16 + 4 + 2 * 32, (name, body.count("ds_read_b128"))
        # accumulation registers are read and cleared by the epilogue (one copy behind the step of either parity) and
        # cleared once at the start, nowhere else
        assert body.count("v_accvgpr_read_b32") == 2 * 256 and body.count("v_accvgpr_write_b32") == 3 * 256, name
        assert "v_accvgpr_mov" not in body, name
        # two barriers per step (+ two before the loop)
        assert len(re.findall(r"^\s*s_barrier", body, re.M)) == 2 + 2 * 2, name
        if tag != "ILi4E":
            cvt = "v_cvt_pk_f16_f32" if tag == "ILi3E" else "v_cvt_pk_bf16_f32"
            assert body.count(cvt) == 2 * 128, (name, body.count(cvt))   # 64 tiles x 4 values per lane, two per instruction


def _reg_range(text):
    """'v[10:13]' -> range(10, 14); 'v7' -> range(7, 8)"""
    m = re.match(r"v\[(\d+):(\d+)\]$", text)
    if m:
        return range(int(m.group(1)), int(m.group(2)) + 1)
    return range(int(text[1:]), int(text[1:]) + 1)


def _steps_of(body, insn):
    """The two copies of the step (parity 0, parity 1) as lists of instruction lines: a step runs from behind the last
    matrix instruction of what precedes it to its own last one (on the last accumulator tile, a[252:255])."""
    lines = [l.strip() for l in body.splitlines()]
    lines = [l for l in lines if l and not l.startswith(";")]
    last = [i for i, l in enumerate(lines) if l.startswith(insn) and re.search(r"a\[(0xfc|252):(0xff|255)\]", l)]
    first = [i for i, l in enumerate(lines) if l.startswith(insn) and re.search(r" a\[0:3\]", l)]
    ends = [i for k, i in enumerate(last) if k + 1 == len(last) or last[k + 1] != i + 1]     # last of a run on that tile
    assert len(ends) == 2, ends
    starts = [first[0], next(i for i in first if i > ends[0])]
    steps = []
    for k in range(2):
        begin = starts[k]
        while not (lines[begin - 1].startswith(insn) or lines[begin - 1].startswith("s_barrier") or re.match(r"\.LBB", lines[begin - 1])
                   or lines[begin - 1].startswith("s_cbranch") or lines[begin - 1].startswith("s_branch")):
            begin -= 1          # the reads and address arithmetic in front of the step's first matrix instruction
        steps.append(lines[begin:ends[k] + 1])
    return steps


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("tag", ["ILi2E", "ILi0E", "ILi5E"])
def test_gemm_quad_schedule_waits_for_what_it_uses(tmp_path, tag):
    """A replay of the step as the compiler emitted it, with the two in-order queues the hardware keeps: LDS reads
    (lgkmcnt) and vector-memory loads (vmcnt).  No matrix instruction may name a register that a read or load still in
    flight will write; at barrier X exactly the loads the step itself has issued may be in flight; and the registers the
    burst of one step fills are the B operands of the other step."""
    asm = device_asm(tmp_path, "gemm_quad.hip")
    meta = kernel_metadata(asm)
    insn, per_step = QUAD_KINDS[tag]
    name = next(k for k in meta if "gemm_quad_kernel" + tag in k)
    steps = _steps_of(kernel_body(asm, name), insn)
    b_sources, burst_dests = [], []
    for step in steps:
        lgkm, vm = [], []          # destinations (register ranges) of the operations in flight, oldest first
        mfma_seen = loads_before_x = x_seen = 0
        b_src, dests_after_x = set(), set()
        for line in step:
            op = line.split()[0]
            if op == "ds_read_b128":
                dest = _reg_range(line.split()[1].rstrip(","))
                lgkm.append(dest)
                if x_seen:
                    dests_after_x.update(dest)
            elif op.startswith("global_load_lds"):
                vm.append(range(0))
                loads_before_x += not x_seen
            elif op.startswith("global_load_dword"):
                vm.append(_reg_range(line.split()[1].rstrip(",")))
                loads_before_x += not x_seen
            elif op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", line)
                if m:
                    lgkm = lgkm[max(0, len(lgkm) - int(m.group(1))):]
                m = re.search(r"vmcnt\((\d+)\)", line)
                if m:
                    keep = int(m.group(1))
                    if mfma_seen:      # the wait of barrier X (the block-scaled kind's wait at the top comes before any)
                        assert keep == loads_before_x, (name, keep, loads_before_x)
                        x_seen = 1
                    vm = vm[max(0, len(vm) - keep):]
            elif op == insn:
                mfma_seen += 1
                srcs = re.findall(r"v\[\d+:\d+\]|\bv\d+\b", line)
                in_flight = {r for d in lgkm + vm for r in d}
                for src in srcs:
                    assert not in_flight & set(_reg_range(src)), (name, mfma_seen, line)
                b_src.update(_reg_range(srcs[0]))
        assert mfma_seen == per_step and x_seen, (name, mfma_seen, x_seen)
        assert not lgkm, (name, "reads still in flight at the end of the step", len(lgkm))
        b_sources.append(b_src)
        burst_dests.append(dests_after_x)
    # behind X a step reads the other step's B fragments (16 x 4 registers) and rows 0, 1 of its A fragments (16 more)
    for k in range(2):
        assert len(b_sources[k]) == 64 and b_sources[k] <= burst_dests[1 - k] and len(burst_dests[1 - k]) == 64 + 16, name


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_mxfp4_prepass(tmp_path):
    meta = kernel_metadata(device_asm(tmp_path, "gemm_mxfp4.hip"))
    name = next(k for k in meta if "mx_scale_layout_kernel" in k)
    assert meta[name]["vgpr_spill_count"] == 0 and meta[name]["private_segment_fixed_size"] == 0


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("source", ["mfma_dense.hip", "smfmac.hip"])
def test_peak_loops_do_not_spill(tmp_path, source):
    meta = kernel_metadata(device_asm(tmp_path, source))
    assert meta, "no kernels found"
    for name, m in meta.items():
        assert m.get("vgpr_spill_count", 0) == 0, (name, m)
        assert m.get("private_segment_fixed_size", 0) == 0, (name, m)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_fp32_and_fp64_kernels(tmp_path):
    """fp32: the ring kernel with four 16x16x4 instructions per 16-byte fragment read, 256 per step.
    fp64: 64 instructions per step in two halves around the barrier, on the accumulation registers, the fragment reads
    riding on them; two 32 KiB buffers (64 KiB static LDS, two workgroups per CU)."""
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
    assert meta[name]["agpr_count"] == 128 and "ds_write" not in body
    mfmas = re.findall(r"v_mfma_f64_16x16x4_f64 (\S+), \S+, \S+, (\S+)", body)
    # 32 per K half; the compiler keeps a second copy of (part of) the second half, without reads, for the last step
    assert len(mfmas) in (64, 80, 96) and all(d == c and d.startswith("a[") for d, c in mfmas), mfmas[:4]
    # the order of a step: the fragments of the first K half have arrived; its 32 instructions with the 8 reads of
    # the second half behind every second of the first 16; the wait for everything and the barrier; the next slab's
    # 8 loads; the 32 instructions of the second half with the next slab's first-half reads riding the same way
    marks = []
    for line in body.split("\n"):
        t = line.strip()
        marks.append("M" if t.startswith("v_mfma_f64") else "B" if t.startswith("s_barrier") else "r" if t.startswith("ds_read_b128")
                     else "w" if t.startswith("s_waitcnt") else "L" if t.startswith("global_load_lds") else "")
    order = "".join(marks)
    half = "MrM" * 8 + "M" * 16
    assert "w" + half + "wB" in order, order
    assert "B" + "L" * 8 + "MrM" * 7 + "Mr" in order, order   # (its last 17 instructions are shared with the copy without reads)
    assert order.count("B") == 2


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


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_scalar_half_row_runs_on_the_scalar_half_fma(tmp_path):
    """The `half` row is the reference's scalar __hfma chain (src/rocm/rocm_kernels/compute_hp.hip:12-30): its loop is
    one v_fma_f16 per step and accumulator and holds no packed multiply-add; the `half2` row is the packed form."""
    asm = device_asm(tmp_path, "compute_mad.hip")
    meta = kernel_metadata(asm)
    scalar = next(n for n in meta if "mad_f16_kernelILi1E" in n)
    packed = next(n for n in meta if "mad_f16_kernelILi2E" in n)
    for name in (scalar, packed):
        assert meta[name].get("vgpr_spill_count", 0) == 0 and meta[name].get("private_segment_fixed_size", 0) == 0, meta[name]
    body = kernel_body(asm, scalar)
    assert body.count("v_fma_f16") == 16 * 8 + 16 and "v_pk_fma_f16" not in body, body.count("v_fma_f16")
    body = kernel_body(asm, packed)
    assert "v_pk_fma_f16" in body and not re.search(r"\bv_fma_f16\b", body)


def _registers(operand):
    """Vector registers an operand text names: v7 -> {7}, v[4:7] -> {4..7}."""
    out = set()
    for lo, hi in re.findall(r"\bv\[(\d+):(\d+)\]", operand):
        out |= set(range(int(lo), int(hi) + 1))
    out |= {int(x) for x in re.findall(r"\bv(\d+)\b", operand)}
    return out


def registers_touched_while_a_read_is_in_flight(body):
    """Instructions that name a destination register of an LDS read between the read and the next wait for all LDS
    reads, and branches or labels in that stretch (where paths join, register copies appear).  Instruction text in
    program order; the body must wait with lgkmcnt(0), as the 128x128 GEMM kernel does."""
    pending, found = set(), []
    for line in body.splitlines():
        text = line.split(";")[0].strip()
        if not text or text.startswith("."):
            if pending and re.match(r"\.LBB\d+_\d+:", text):
                found.append(("label", text))
            continue
        op, _, rest = text.partition(" ")
        if op == "s_waitcnt" and "lgkmcnt(0)" in rest:
            pending = set()
        elif op.startswith("ds_read"):
            dst = rest.split(",")[0]
            if _registers(rest) & pending:
                found.append(("reuse", text))
            pending |= _registers(dst)
        elif pending and (op.startswith("s_cbranch") or op == "s_branch"):
            found.append(("branch", text))
        elif pending and _registers(rest) & pending:
            found.append(("touch", text))
    if pending:
        found.append(("end", sorted(pending)[:4]))
    return found


def test_the_checker_of_reads_in_flight_sees_what_it_is_for():
    good = "ds_read_b128 v[4:7], v1 offset:0\n v_mfma_f32_16x16x32_bf16 v[8:11], v[12:15], v[16:19], v[8:11]\n s_waitcnt lgkmcnt(0)\n v_add_u32 v4, v4, v5\n"
    assert registers_touched_while_a_read_is_in_flight(good) == []
    early = "ds_read_b128 v[4:7], v1 offset:0\n v_lshlrev_b32_e32 v5, 2, v9\n s_waitcnt lgkmcnt(0)\n"
    assert [k for k, _ in registers_touched_while_a_read_is_in_flight(early)] == ["touch"]
    copy = "ds_read_b128 v[4:7], v1 offset:0\n v_mov_b64_e32 v[20:21], v[6:7]\n s_waitcnt lgkmcnt(0)\n"
    assert [k for k, _ in registers_touched_while_a_read_is_in_flight(copy)] == ["touch"]
    join = "ds_read_b128 v[4:7], v1 offset:0\n s_cbranch_scc1 .LBB0_3\n.LBB0_3:\n s_waitcnt lgkmcnt(0)\n"
    assert [k for k, _ in registers_touched_while_a_read_is_in_flight(join)] == ["branch", "label"]
    never = "ds_read_b128 v[4:7], v1 offset:0\n s_endpgm\n"
    assert [k for k, _ in registers_touched_while_a_read_is_in_flight(never)] == ["end"]


SMALL_KINDS = {"ILi0E": ("v_mfma_f32_16x16x128_f8f6f4", 16), "ILi1E": ("v_mfma_f32_16x16x128_f8f6f4", 16),
               "ILi2E": ("v_mfma_f32_16x16x32_bf16", 32), "ILi3E": ("v_mfma_f32_16x16x32_f16", 32), "ILi4E": ("v_mfma_i32_16x16x64_i8", 32)}


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_gemm_small_kernels(tmp_path):
    """The kernel on 128x128 tiles.  Nothing spills.  No register that an LDS read is still writing is named before
    the wait for it, and no branch lies in between (a last step that read fragments nobody takes once had their
    registers reused for the addresses of the stores).  The accumulators are the 64 accumulation registers the source
    names, touched by nothing but its matrix instructions, its zeroing and, behind the wait states that follow the last
    matrix instruction, its reads (held as values of the compiler's they were once copied, where two paths joined,
    right behind the matrix instructions that wrote them).  The loop holds two steps, the code behind it one more with
    reads and loads and two without (an even and an odd count of steps)."""
    asm = device_asm(tmp_path, "gemm_small.hip")
    meta = kernel_metadata(asm)
    for tag, (insn, per_step) in SMALL_KINDS.items():
        name = next(k for k in meta if "gemm_small_kernel" + tag in k)
        m = meta[name]
        assert m["vgpr_spill_count"] == 0 and m.get("sgpr_spill_count", 0) == 0 and m["private_segment_fixed_size"] == 0, (name, m)
        assert m["agpr_count"] == 64 and m["vgpr_count"] <= 256 and m.get("group_segment_fixed_size", 0) == 0, (name, m)
        body = kernel_body(asm, name)
        assert registers_touched_while_a_read_is_in_flight(body) == [], name
        lines = [l.split(";")[0].strip() for l in body.splitlines()]
        lines = [l for l in lines if l and not l.startswith(".")]
        on_acc = [(n, l) for n, l in enumerate(lines) if re.search(r"\ba\[?\d+", l)]
        mfma = [n for n, l in on_acc if l.startswith(insn + " ")]
        zero = [n for n, l in on_acc if re.fullmatch(r"v_accvgpr_write_b32 a\[?\d+\]?, 0", l)]
        take = [n for n, l in on_acc if re.fullmatch(r"v_accvgpr_read_b32 v\d+, a\[?\d+\]?", l)]
        assert len(mfma) + len(zero) + len(take) == len(on_acc), [l for _, l in on_acc if not l.startswith(insn)][:3]
        assert len(mfma) == 5 * per_step and len(zero) == 64 and len(take) == 64, (name, len(mfma), len(zero), len(take))
        assert max(zero) < min(mfma), name
        assert all(re.search(r"a\[(\d+):(\d+)\], v\[\d+:\d+\], v\[\d+:\d+\], a\[\1:\2\]", lines[n]) for n in mfma), name
        # the reads of the accumulators: one stretch of straight-line code that begins with the wait states and holds
        # no matrix instruction (the compiler is free to place that block anywhere in the text)
        waits = [n for n, l in enumerate(lines) if l == "s_nop 15"]
        assert len(waits) == 2 and waits[1] == waits[0] + 1 and waits[1] < min(take), (name, waits)
        stretch = [l.split(";")[0].strip() for l in body.splitlines()]
        stretch = [l for l in stretch if l]
        begin, end = stretch.index("s_nop 15"), max(n for n, l in enumerate(stretch) if l.startswith("v_accvgpr_read_b32"))
        assert not any(l.startswith((insn, ".LBB", "s_cbranch", "s_branch")) for l in stretch[begin:end]), name
        assert sum(l.startswith("ds_read_b128 ") for l in lines) == 16 * 4, name          # prologue, two steps, one tail step
        assert sum(l.startswith("global_load_lds_dwordx4 ") for l in lines) == 8 * (4 + 3), name
        assert sum(l == "s_barrier" for l in lines) == 4, name
