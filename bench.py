#!/usr/bin/env python3
"""Benchmark driver of the MI355X clpeak backend.

    python bench.py --gpus 1 --steps K --warmup W

The LAST line of stdout is one compact JSON record (under 2000 bytes); the full record with every row
goes to the rows file (--rows-file) and the rows are listed on stderr.  A "step" is one launch of the headline kernel: the float4
streaming read-reduce over a 4 GiB fp32 buffer resident in HBM (the HBM configuration
of the workload list).  `value` is its throughput in GB/s.  The same line carries

  roofline      the headline kernel against the 8 TB/s HBM3E peak, from HIP events on
                the stream the kernel runs on;
  cpu_baseline  the reference's own DRAM read kernel (where its build exists) and the CPU oracle's kernels,
                timed on this host with the reference's CPU discipline (bounded samples);
  fracs         one fraction of datasheet peak per target kernel (taken from the rows below);
  rows (file)   every other kernel of the backend (float/float2 reads, MAD chains, launch
                latency, dense MFMA, 2:4 SMFMAC, GEMM, LDS, PCIe transfers) with its absolute figure, the
                MI355X datasheet peak it is compared with and the fraction reached; and, measured first by a
                child process on the same board, the vendor library's bf16 / fp8 / block-scaled FP4 GEMM of the same shape (what the
                reference's GEMM rows call; skipped without torch or with --no-vendor).

One GPU only: the path has no exchange step, every unit of work is independent, so more
GPUs would simply run the same kernels side by side.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# MI355X dense peaks (TFLOP/s or TOP/s); 2:4 sparse peaks are twice the dense ones.
PEAK = {"f16": 2500.0, "bf16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "fp6": 10100.0, "fp4": 10100.0,
        "fp32_vec": 157.3, "fp64_vec": 78.6, "fp32_mat": 157.3, "fp64_mat": 78.6}
SEED = 0x5EEDC1BEA4D355


def timed(dev, launch, min_us=300e3, warm_us=300e3, max_iters=10000, board=None):
    """Reference discipline (warm-up, probe, batch sized to a time budget), with the warm-up
    long enough for the clocks to settle under this kernel's load.  Returns us per launch.
    board: a dict that receives the board's mean power during the timed batch, where the machine lets an ordinary user read it."""
    launch(); dev.sync()
    probe = max(dev.time_launches(launch, 1), 1.0)
    dev.time_launches(launch, int(min(max(warm_us / probe, 2), max_iters)))
    n = int(min(max(min_us / probe, 1), max_iters))
    if board is None:
        return dev.time_launches(launch, n) / n, n
    # (The driver's throttler residencies are not read here: its accumulators trail the load by some tenths of a second, so
    # over a batch this short they tell of the row before.  --power-table reads them over seconds.)
    tel = _board_telemetry()
    tel.start()                                  # the power reading: sampled during the timed batch, behind the warm-up
    us = dev.time_launches(launch, n) / n
    stats = tel.stop(skip_s=0.0)
    if stats.get("watts_mean") is not None:
        board["watts"] = stats["watts_mean"]
    return us, n


_TELEMETRY = []


def _board_telemetry():
    if not _TELEMETRY:
        _TELEMETRY.append(_Telemetry())
    return _TELEMETRY[0]


def bench_rows(dev, quick, only):
    from clpeak_amd import capi
    from clpeak_amd import workloads as wl
    rows = []
    budget = dict(min_us=100e3, warm_us=100e3) if quick else {}

    def add(test, metric, value, unit, us, peak=None, **extra):
        r = {"test": test, "metric": metric, "value": round(value, 2), "unit": unit, "us_per_launch": round(us, 2)}
        if peak:
            r["peak"] = peak
            r["frac"] = round(value / peak, 4)
        r.update(extra)
        rows.append(r)

    progress("rows: " + ",".join(sorted(only)))
    if "mad" in only:
        _mad_rows(dev, capi, add, budget)
    if "latency" in only:
        us = dev.launch_roundtrip(2, 10000)
        add("kernel_launch_latency", "roundtrip", us, "us", us)
    if "mfma" in only or "smfmac" in only:
        progress("mfma rows")
        _matrix_rows(dev, wl, add, budget, only, zero=False, one_set=True)
    if "matrix_distinct" in only:
        progress("matrix_distinct rows")
        _matrix_rows(dev, wl, add, budget, ("mfma", "smfmac"), zero=False, one_set=False)
    if "matrix_zero" in only:
        progress("matrix_zero rows")
        _matrix_rows(dev, wl, add, budget, ("mfma", "smfmac"), zero=True, one_set=True)
    if "matrix_ref" in only:
        progress("matrix_ref rows")
        _matrix_rows(dev, wl, add, budget, ("mfma", "smfmac"), zero=False, one_set=True, reference=True)
    if "gemm" in only:
        progress("gemm rows")
        _gemm_rows(dev, capi, wl, add, budget, constant=False)
    if "vendor" in only:
        _vendor_rows(dev, capi, wl, add, budget)
    if "gemm_small" in only:
        progress("gemm_small rows")
        _gemm_small_rows(dev, capi, wl, add, budget)
    if "gemm_const" in only:
        progress("gemm_const rows")
        _gemm_rows(dev, capi, wl, add, budget, constant=True)
    if "lds" in only:
        progress("lds rows")
        _lds_rows(dev, add, budget)
    if "transfer" in only:
        _transfer_rows(dev, capi, add, budget)
    return rows


def _lds_rows(dev, add, budget):
    # --- LDS ping-pong: the reference's grid (max(32 Mi, CUs x 2048 x 256) threads), 64 repetitions -----
    bs, reps = 256, 64
    threads = max(32 << 20, dev.props.num_cus * 2048 * 256)
    blocks = threads // bs
    out = dev.alloc(blocks * bs * 4)
    # 128 bytes per clock and CU at the 2.4 GHz boost clock
    peak = 128 * dev.props.num_cus * 2.4
    for width, metric in ((1, "float"), (2, "float2"), (4, "float4")):
        us, _ = timed(dev, lambda: dev.local_bandwidth(width, out, blocks, bs, reps), **budget)
        add("local_memory_bandwidth", metric, reps * 2 * width * 4 * blocks * bs / us / 1e3, "gbps", us, peak)
    out.free()


def _transfer_rows(dev, capi, add, budget):
    # --- pinned host <-> device copies of 512 MiB ----------------------------------------------------
    nbytes = 1 << 29
    _, hp = dev.host_alloc(nbytes)
    dbuf = dev.alloc(nbytes)
    for metric, direction, d, s in (("h2d_pinned", capi.H2D, dbuf.ptr, hp), ("d2h_pinned", capi.D2H, hp, dbuf.ptr)):
        us, _ = timed(dev, lambda: dev.copy_async(d, s, nbytes, direction), **budget)
        add("transfer_bandwidth", metric, nbytes / us / 1e3, "gbps", us)
    dbuf.free()
    dev.host_free(hp)


def _mad_rows(dev, capi, add, budget):
    # --- vector MAD chains: 2^20 work-items x 16 accumulators x 4096 steps -------------
    n_items, steps = 1 << 20, 4096
    out = dev.alloc(n_items * 8)
    mad = [("single_precision_compute", capi.MAD_F32, [(1, "float"), (2, "float2"), (4, "float4")], 2, "gflops", PEAK["fp32_vec"] * 1e3),
           ("half_precision_compute", capi.MAD_F16, [(1, "half"), (2, "half2")], 2, "gflops", None),
           ("double_precision_compute", capi.MAD_F64, [(1, "double"), (2, "double2"), (4, "double4")], 2, "gflops", PEAK["fp64_vec"] * 1e3),
           ("mixed_precision_compute", capi.MAD_MP, [(1, "mp")], 2, "gflops", None),
           ("bfloat16_compute", capi.MAD_BF16, [(1, "bf16")], 4, "gflops", None),   # two products and two additions per step
           ("integer_compute", capi.MAD_I32, [(1, "int"), (2, "int2"), (4, "int4")], 2, "gops", None)]
    for test, kind, variants, ops, unit, peak in mad:
        for width, metric in variants:
            us, _ = timed(dev, lambda: dev.compute_mad(kind, width, SEED, n_items, steps, out), **budget)
            add(test, metric, n_items * 16 * steps * ops / us / 1e3, unit, us, peak)
    for chains, metric in ((1, "int8_dp"), (2, "int8_dp2"), (4, "int8_dp4"), (8, "int8_dp8")):
        us, _ = timed(dev, lambda: dev.compute_mad(capi.MAD_I8DP, chains, SEED, n_items, steps, out), **budget)
        add("integer_compute_int8_dp", metric, n_items * chains * steps * 8 / us / 1e3, "gops", us)
    out.free()


def _matrix_rows(dev, wl, add, budget, only, zero, one_set, reference=False):
    # --- dense MFMA / SMFMAC: 2048 waves x 4 chains x 4096 iterations ------------------------
    # one_set: the four accumulator chains of a wave share one A and one B fragment, held in the same
    # registers, as the reference's kernels do (src/rocm/rocm_kernels/mfma_bf16.hip:16-30); that is the
    # workload's "per wave: A/B fragments ... 4 independent accumulator chains" and what the rows report.
    # Not one_set ("distinct operands per chain"): every chain has fragments of its own, in registers of
    # its own; same arithmetic, more register reads, a lower clock.
    # zero: the same launches on all-zero operands.  Nothing toggles in the multipliers, the part holds
    # its boost clock, and the row shows the issue rate of the loop itself (the seeded rows show what the
    # part sustains under the power that random operands draw).
    # reference: the same launches on the constants the reference's own kernels multiply (1.0, byte 0x38,
    # byte 0x01, nibble 4 under scales of 0x3f, sparsity index 0): like for like with what it measures.
    waves, iters = 2048, 4096
    tail = " zero operands" if zero else " reference operands" if reference else ("" if one_set else " distinct operands per chain")
    clk = dev.alloc(16)
    peaks = {0: "f16", 1: "bf16", 2: "f16", 3: "bf16", 4: "int8", 5: "fp8", 6: "fp8", 7: "fp6", 8: "fp6", 9: "fp4"}
    for kind in sorted(wl.DENSE) if "mfma" in only else []:
        s = wl.DENSE[kind]
        A, B, sA, sB = wl.reference_dense_inputs(kind, waves) if reference else wl.dense_inputs(kind, waves, SEED)
        if zero:
            A, B = np.zeros_like(A), np.zeros_like(B)
        bufs = [dev.from_host(A), dev.from_host(B), dev.from_host(sA) if sA is not None else None,
                dev.from_host(sB) if sB is not None else None]
        o = dev.alloc(waves * 4 * s["M"] * s["N"] * 4)
        board = {}
        us, _ = timed(dev, lambda: dev.mfma_dense(kind, bufs[0], bufs[1], bufs[2], bufs[3], o, waves, iters, clk, one_set=one_set), board=board, **budget)
        c = clk.download(np.uint64, 2)
        unit = "tops" if s["fmt"] == wl.I8 else "tflops"
        add(s["name"], s["name"] + tail, wl.dense_flops(kind, waves, iters) / us / 1e6, unit, us, PEAK[peaks[kind]],
            shape=s["shape"], sclk_mhz=round(float(c[0]) / max(float(c[1]), 1.0) * 100.0, 0), **board)
        for b in bufs + [o]:
            if b is not None:
                b.free()
    speaks = {0: "f16", 1: "bf16", 2: "fp8", 3: "fp8", 4: "int8"}
    for kind in sorted(wl.SPARSE) if "smfmac" in only else []:
        s = wl.SPARSE[kind]
        Ac, meta, B = wl.reference_sparse_inputs(kind, waves) if reference else wl.sparse_inputs(kind, waves, SEED)
        if zero:
            Ac, B = np.zeros_like(Ac), np.zeros_like(B)
        bufs = [dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)]
        o = dev.alloc(waves * 4 * 256 * 4)
        board = {}
        us, _ = timed(dev, lambda: dev.smfmac(kind, bufs[0], bufs[1], bufs[2], o, waves, iters, clk, one_set=one_set), board=board, **budget)
        c = clk.download(np.uint64, 2)
        unit = "tops" if s["fmt"] == wl.I8 else "tflops"
        add(s["name"], s["name"] + tail, wl.sparse_flops(kind, waves, iters) / us / 1e6, unit, us, 2 * PEAK[speaks[kind]],
            shape=s["shape"], sclk_mhz=round(float(c[0]) / max(float(c[1]), 1.0) * 100.0, 0), **board)
        for b in bufs + [o]:
            b.free()
    clk.free()


def _gemm_rows(dev, capi, wl, add, budget, constant):
    # --- GEMM 8192^3: (test, metric, bytes per element, bytes per output, peak key, unit, constant fill byte) ----
    M = N = K = 8192
    s43, s52 = 448.0, 57344.0
    kinds = [("rocblas-fp", "fp32", 4, 4, "fp32_mat", "tflops", 0x3f),
             ("rocblas-fp", "fp64", 8, 8, "fp64_mat", "tflops", 0x3f),
             ("rocblas-fp", "fp16", 2, 2, "f16", "tflops", 0x3f),
             ("rocblas-fp", "bf16", 2, 2, "bf16", "tflops", 0x3f),
             ("hipblaslt-fp8", "fp8_e4m3", 1, 2, "fp8", "tflops", 0x38),
             ("hipblaslt-fp8", "fp8_e5m2", 1, 2, "fp8", "tflops", 0x38),
             ("hipblaslt-fp8", "mxf4_e2m1", 0.5, 2, "fp4", "tflops", 0x38),
             ("rocblas-int", "int8", 1, 4, "int8", "tops", 0x3f)]
    for test, metric, eb, ob, peak, unit, const_byte in kinds:
        dA, dB, dC = dev.alloc(int(M * K * eb)), dev.alloc(int(N * K * eb)), dev.alloc(M * N * ob)
        extra = []
        if metric == "mxf4_e2m1":
            dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
            extra = [dSA, dSB]
            dev.fill_bytes(dA, M * K // 2, SEED, wl.STREAM_GEMM_A, 0, 256); dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
            dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9); dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
            if constant:
                dev.memset(dSA, 0x7f); dev.memset(dSB, 0x7f)
            # the scales stay what they are over the timed launches (as in the reference's loop, one set of scale
            # pointers for every product): laid out for the kernel once; the one-call form is a row of its own below
            dPrep = dev.alloc((M + N) * K // 32)
            extra.append(dPrep)
            dev.gemm_mxfp4_prepare_scales(dSA, dSB, M, N, K, dPrep)
            fn = lambda: dev.gemm_mxfp4_prepared(dA, dB, dPrep, dC, M, N, K)
        elif metric == "fp32":
            dev.fill_f32(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f32(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_f32(dA, dB, dC, M, N, K)
        elif metric == "fp64":
            dev.fill_f64(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f64(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_f64(dA, dB, dC, M, N, K)
        elif metric == "fp16":
            dev.fill_f16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_f16(dA, dB, dC, M, N, K)
        elif metric == "bf16":
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_bf16(dA, dB, dC, M, N, K)
        elif metric == "fp8_e4m3":
            dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, s43)
            dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, s43)
            fn = lambda: dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1 / s43, 1 / s43)
        elif metric == "fp8_e5m2":
            dev.fill_fp8_e5m2(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, s52)
            dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, s43)
            fn = lambda: dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1 / s52, 1 / s43)
        else:
            dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
            fn = lambda: dev.gemm_i8(dA, dB, dC, M, N, K)
        if constant:
            # the same launch on constant buffers, as the reference fills them (every byte 0x3f in its rocBLAS
            # test, src/rocm/rocblas.cpp:211-212, every byte 0x38 under block scales of 0x7f in its hipBLASLt
            # test, src/rocm/hipblaslt_gemm.cpp:272-273 and 417-418): constant operands draw less power and the
            # part holds a higher clock
            dev.memset(dA, const_byte); dev.memset(dB, const_byte)
            metric += " constant operands"
        board = {}
        us, _ = timed(dev, fn, board=board, **budget)
        add(test, metric, 2.0 * M * N * K / us / 1e6, unit, us, PEAK[peak], shape="8192x8192x8192", **board)
        if metric.startswith("mxf4_e2m1"):
            us, _ = timed(dev, lambda: dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K), **budget)
            add(test, metric + ", scale layout on every call", 2.0 * M * N * K / us / 1e6, unit, us, PEAK[peak], shape="8192x8192x8192")
        for b in [dA, dB, dC] + extra:
            b.free()


def _gemm_small_rows(dev, capi, wl, add, budget):
    """2048 cubed, 64 tiles of 256 x 256 on a part of 256 CUs: the 8- and 16-bit kinds on the tiling the library picks
    there (128 x 128, one tile per CU) and on the 256 x 256 tiles it would otherwise run on.  Seeded operands."""
    M = N = K = 2048
    s43, s52 = 448.0, 57344.0
    for test, metric, eb, ob, peak, unit in (("rocblas-fp", "fp16", 2, 2, "f16", "tflops"), ("rocblas-fp", "bf16", 2, 2, "bf16", "tflops"),
                                             ("hipblaslt-fp8", "fp8_e4m3", 1, 2, "fp8", "tflops"), ("hipblaslt-fp8", "fp8_e5m2", 1, 2, "fp8", "tflops"),
                                             ("rocblas-int", "int8", 1, 4, "int8", "tops")):
        dA, dB, dC = dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * ob)
        if metric == "fp16":
            dev.fill_f16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_f16(dA, dB, dC, M, N, K)
        elif metric == "bf16":
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            fn = lambda: dev.gemm_bf16(dA, dB, dC, M, N, K)
        elif metric == "fp8_e4m3":
            dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, s43); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, s43)
            fn = lambda: dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1 / s43, 1 / s43)
        elif metric == "fp8_e5m2":
            dev.fill_fp8_e5m2(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, s52); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, s43)
            fn = lambda: dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1 / s52, 1 / s43)
        else:
            dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
            fn = lambda: dev.gemm_i8(dA, dB, dC, M, N, K)
        for tiling, name in ((capi.GEMM_TILING_128, "128x128 tiles"), (capi.GEMM_TILING_256, "256x256 tiles")):
            dev.gemm_tiling(tiling)
            us, _ = timed(dev, fn, **budget)
            dev.gemm_tiling(capi.GEMM_TILING_AUTO)
            add(test, f"{metric} on {name}", 2.0 * M * N * K / us / 1e6, unit, us, PEAK[peak], shape="2048x2048x2048")
        for b in (dA, dB, dC):
            b.free()


def _vendor_rows(dev, capi, wl, add, budget):
    """The vendor library the reference's GEMM rows call (rocBLAS / hipBLASLt, reached here through torch.matmul,
    torch._scaled_mm and torch._int_mm), timed in this process on this board right beside this library's kernel of the
    same row, on operands of the same distribution (uniform [-1,1) rounded to the type; int8 uniform in [-8,7]) and on
    the reference's constant fill.  Not part of the default rows: it needs torch, whose first import takes a minute."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(SEED & 0x7fffffff)
    # 8192 cubed: the rows' own shape.  2048 cubed: 64 tiles of 256 x 256 on a part of 256 CUs, the shape this library
    # gives to its kernel on 128 x 128 tiles (timed on the 256 x 256 tiles as well).
    for D in (8192, 2048):
        _vendor_rows_of(dev, capi, wl, add, budget, torch, g, D)


def _vendor_rows_of(dev, capi, wl, add, budget, torch, g, D):
    import time
    M = N = K = D
    flops = 2.0 * M * N * K
    shape = f"{D}x{D}x{D}"

    def t_torch(fn):
        torch.cuda.synchronize()
        t0 = time.time()
        while time.time() - t0 < budget.get("warm_us", 300e3) / 1e6:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        reps = max(10, int(budget.get("min_us", 300e3) / (600.0 * (D / 8192.0) ** 3 + 10.0)))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    one = torch.ones((), device="cuda")
    cases = [("rocblas-fp", "bf16", torch.bfloat16, "bf16", "tflops", 0x3f), ("rocblas-fp", "fp16", torch.float16, "f16", "tflops", 0x3f),
             ("hipblaslt-fp8", "fp8_e4m3", torch.float8_e4m3fn, "fp8", "tflops", 0x38), ("rocblas-int", "int8", torch.int8, "int8", "tops", 0x3f)]
    for test, metric, dt, peak, unit, const_byte in cases:
        if dt == torch.int8:
            A = torch.randint(-8, 8, (M, K), device="cuda", dtype=dt, generator=g); B = torch.randint(-8, 8, (N, K), device="cuda", dtype=dt, generator=g)
            fn = lambda: torch._int_mm(A, B.t())
        elif dt == torch.float8_e4m3fn:
            A = ((torch.rand(M, K, device="cuda", generator=g) * 2 - 1) * 448).to(dt); B = ((torch.rand(N, K, device="cuda", generator=g) * 2 - 1) * 448).to(dt)
            fn = lambda: torch._scaled_mm(A, B.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        else:
            A = (torch.rand(M, K, device="cuda", generator=g) * 2 - 1).to(dt); B = (torch.rand(N, K, device="cuda", generator=g) * 2 - 1).to(dt)
            fn = lambda: torch.matmul(A, B.t())
        for what in ("uniform random operands", "constant operands"):
            if what.startswith("constant"):
                A.view(torch.uint8).fill_(const_byte); B.view(torch.uint8).fill_(const_byte)
            us = t_torch(fn)
            add(test, f"{metric} vendor library, {what}", flops / us / 1e6, unit, us, PEAK[peak], shape=shape)
        del A, B
        torch.cuda.empty_cache()
        # this library's kernel of the same row, right behind it on the same board
        eb, ob = (2, 2) if dt in (torch.bfloat16, torch.float16) else (1, 4 if dt == torch.int8 else 2)
        dA, dB, dC = dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * ob)
        if metric == "bf16":
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            mine = lambda: dev.gemm_bf16(dA, dB, dC, M, N, K)
        elif metric == "fp16":
            dev.fill_f16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            mine = lambda: dev.gemm_f16(dA, dB, dC, M, N, K)
        elif metric == "fp8_e4m3":
            dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, 448.0); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, 448.0)
            mine = lambda: dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0, 1.0)
        else:
            dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
            mine = lambda: dev.gemm_i8(dA, dB, dC, M, N, K)
        small = 2 * (M // 256) * (N // 256) <= dev.props.num_cus     # the library's own choice of tiling at this shape
        for what in ("seeded operands", "constant operands"):
            if what.startswith("constant"):
                dev.memset(dA, const_byte); dev.memset(dB, const_byte)
            us, _ = timed(dev, mine, **budget)
            add(test, f"{metric} this library, {what}", flops / us / 1e6, unit, us, PEAK[peak], shape=shape)
            if small:
                dev.gemm_tiling(capi.GEMM_TILING_256)
                us, _ = timed(dev, mine, **budget)
                dev.gemm_tiling(capi.GEMM_TILING_AUTO)
                add(test, f"{metric} this library on 256x256 tiles, {what}", flops / us / 1e6, unit, us, PEAK[peak], shape=shape)
        for b in (dA, dB, dC):
            b.free()


class _Telemetry:
    """Samples the board's power (hwmon power1_input / power1_average, microwatts) and shader clock (the
    starred line of pp_dpm_sclk) from sysfs on a thread of its own, every `period` seconds."""

    def __init__(self, period=0.01):
        import glob
        self.period = period
        self.power = next((f for pat in ("power1_input", "power1_average")
                           for f in sorted(glob.glob(f"/sys/class/drm/card*/device/hwmon/hwmon*/{pat}"))), None)
        self.sclk = next(iter(sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))), None)
        cap = next(iter(sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"))), None)
        self.cap_w = self._read_uw(cap)
        self.metrics = next(iter(sorted(glob.glob("/sys/class/drm/card*/device/gpu_metrics"))), None)
        self.samples = []
        self._run = False

    # The driver's metrics table (sysfs gpu_metrics), format 1, content revision 8: the layout of the fields read here was
    # checked on the box against the names `rocm-smi --showmetrics` gives the same numbers.  All little-endian.
    #   @24 u64 energy_accumulator (units of 15.259 uJ)      @40 u32 accumulation_counter (one per millisecond)
    #   @44.. u32 x5 accumulated throttler residencies: prochot, ppt (package power), socket thermal, vr thermal, hbm thermal
    #   @288 u64 firmware_timestamp (10 ns)                   @296 u16 x8 current_gfxclk per XCD (MHz)
    THROTTLERS = ("prochot", "ppt", "socket_thm", "vr_thm", "hbm_thm")

    def snapshot(self):
        """{"energy_j", "acc", residencies..., "gfxclk": [8], "fw_s"} or None when the table is absent or of another revision."""
        import struct
        try:
            b = open(self.metrics, "rb").read()
            size, fmt, rev = struct.unpack_from("<HBB", b, 0)
            if (fmt, rev) != (1, 8) or len(b) < 312:
                return None
            out = {"energy_j": struct.unpack_from("<Q", b, 24)[0] * 15.259e-6, "acc": struct.unpack_from("<I", b, 40)[0],
                   "fw_s": struct.unpack_from("<Q", b, 288)[0] * 1e-8, "gfxclk": list(struct.unpack_from("<8H", b, 296))}
            out.update(zip(self.THROTTLERS, struct.unpack_from("<5I", b, 44)))
            return out
        except (OSError, TypeError, struct.error):
            return None

    @classmethod
    def between(cls, a, b):
        """What the table says happened between two snapshots: mean power from the energy counter, and for each throttler
        the share of the firmware's accumulation cycles in which it was active (its residency)."""
        if a is None or b is None:
            return {}
        cycles = (b["acc"] - a["acc"]) & 0xffffffff
        dt = b["fw_s"] - a["fw_s"]
        out = {"watts_energy_counter": round((b["energy_j"] - a["energy_j"]) / dt, 1) if dt > 0 else None,
               "gfxclk_mhz_per_xcd": b["gfxclk"]}
        for k in cls.THROTTLERS:
            out[k + "_residency"] = round(((b[k] - a[k]) & 0xffffffff) / cycles, 4) if cycles else None
        return out

    @staticmethod
    def _read_uw(path):
        try:
            return int(open(path).read().strip()) / 1e6
        except (OSError, ValueError, TypeError):
            return None

    def _read_mhz(self):
        try:
            for ln in open(self.sclk).read().splitlines():
                if ln.rstrip().endswith("*"):
                    return float(ln.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        except (OSError, ValueError, TypeError, IndexError):
            pass
        return None

    def start(self):
        import threading
        self.samples, self._run = [], True

        def loop():
            while self._run:
                self.samples.append((time.perf_counter(), self._read_uw(self.power), self._read_mhz()))
                time.sleep(self.period)
        self._thread = threading.Thread(target=loop, daemon=True)
        self._thread.start()

    def stop(self, skip_s=0.5):
        """Mean and maximum over the samples taken after the first `skip_s` seconds."""
        self._run = False
        self._thread.join()
        t0 = self.samples[0][0] if self.samples else 0.0
        w = [p for t, p, _ in self.samples if p is not None and t - t0 >= skip_s]
        m = [c for t, _, c in self.samples if c is not None and t - t0 >= skip_s]
        return {"samples": len(w), "watts_mean": round(sum(w) / len(w), 1) if w else None, "watts_max": round(max(w), 1) if w else None,
                "sclk_mhz_mean": round(sum(m) / len(m), 0) if m else None, "sclk_mhz_min": min(m) if m else None}


def _vendor_child():
    """Child-process leg: the vendor library's bf16, fp8 and block-scaled FP4 GEMM at 8192^3 on uniform random operands
    (FP4: uniform codes under scales 2^-4 .. 2^4, as this library's row), through torch.matmul / torch._scaled_mm
    (hipBLASLt), one JSON line {"bf16": us, "fp8_e4m3": us, "mxf4_e2m1": us}.  A process of its own
    because torch brings a HIP runtime that has to be the one to initialise the device in its process."""
    import torch
    M = N = K = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(SEED & 0x7fffffff)
    one = torch.ones((), device="cuda")
    out = {}

    def t_torch(fn, warm_s=0.3, run_s=0.3):
        torch.cuda.synchronize()
        t0 = time.time()
        while time.time() - t0 < warm_s:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        reps = max(10, int(run_s * 1e6 / 600.0))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    A = (torch.rand(M, K, device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    B = (torch.rand(N, K, device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    out["bf16"] = t_torch(lambda: torch.matmul(A, B.t()))
    del A, B
    try:
        A = ((torch.rand(M, K, device="cuda", generator=g) * 2 - 1) * 448).to(torch.float8_e4m3fn)
        B = ((torch.rand(N, K, device="cuda", generator=g) * 2 - 1) * 448).to(torch.float8_e4m3fn)
        out["fp8_e4m3"] = t_torch(lambda: torch._scaled_mm(A, B.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
    except Exception as e:   # an older torch without the fp8 product: the bf16 figure stands alone
        sys.stderr.write(f"bench.py: vendor fp8 product not available: {e!r}\n")
    try:
        del A, B
        A = torch.randint(0, 256, (M, K // 2), device="cuda", dtype=torch.uint8, generator=g).view(torch.float4_e2m1fn_x2)
        B = torch.randint(0, 256, (N, K // 2), device="cuda", dtype=torch.uint8, generator=g).view(torch.float4_e2m1fn_x2)
        sa = torch.randint(123, 132, (M, K // 32), device="cuda", dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
        sb = torch.randint(123, 132, (N, K // 32), device="cuda", dtype=torch.uint8, generator=g).view(torch.float8_e8m0fnu)
        out["mxf4_e2m1"] = t_torch(lambda: torch._scaled_mm(A, B.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16))
    except Exception as e:
        sys.stderr.write(f"bench.py: vendor block-scaled FP4 product not available: {e!r}\n")
    print(json.dumps(out), flush=True)


def vendor_beside(timeout_s=150):
    """Rows of the vendor library's GEMM (what the reference's rocblas-fp / hipblaslt-fp8 rows call) measured on this
    board by a child process, or [] when torch is missing, slow to load or fails: a comparison, never a dependency.
    Runs before this process touches the GPU."""
    import subprocess
    try:
        r = subprocess.run([sys.executable, os.path.abspath(__file__), "--vendor-child"], capture_output=True, text=True, timeout=timeout_s)
        got = json.loads(r.stdout.strip().splitlines()[-1]) if r.returncode == 0 and r.stdout.strip() else {}
        if not got:
            sys.stderr.write(f"bench.py: vendor library leg gave nothing (exit status {r.returncode}): {r.stderr.strip()[-300:]}\n")
    except (subprocess.TimeoutExpired, OSError, ValueError) as e:
        sys.stderr.write(f"bench.py: vendor library leg skipped: {e!r}\n")
        return []
    rows, flops = [], 2.0 * 8192 ** 3
    for key, test, peak in (("bf16", "rocblas-fp", "bf16"), ("fp8_e4m3", "hipblaslt-fp8", "fp8"), ("mxf4_e2m1", "hipblaslt-fp8", "fp4")):
        if key in got:
            us = float(got[key])
            rows.append({"test": test, "metric": f"{key} vendor library, uniform random operands", "value": round(flops / us / 1e6, 2),
                         "unit": "tflops", "us_per_launch": round(us, 2), "peak": PEAK[peak], "frac": round(flops / us / 1e6 / PEAK[peak], 4),
                         "shape": "8192x8192x8192"})
    return rows


def progress(what):
    """A line on stderr per phase: a reader that takes a silent run for a hung one sees this one move."""
    sys.stderr.write(f"bench.py [{time.strftime('%H:%M:%S')}] {what}\n")
    sys.stderr.flush()


def power_table(dev, seconds):
    """Board power and shader clock while each matrix workload runs for `seconds`: the seeded launches beside
    the same launches on constant and on zero operands.  One JSON line per workload."""
    from clpeak_amd import capi
    from clpeak_amd import workloads as wl
    tel = _Telemetry()
    out = []

    idle_w = [None]

    def run(label, fn, work, unit, clock_buf=None):
        """work: operations (or bytes) per launch; clock_buf: where the kernel leaves its two loop counters."""
        fn(); dev.sync()
        tel.start()
        t0 = time.perf_counter()
        n = 0
        snap0 = None
        while time.perf_counter() - t0 < seconds:
            if snap0 is None and time.perf_counter() - t0 >= 0.5:
                snap0 = tel.snapshot()            # the driver's table from 0.5 s into the load ...
            us = dev.time_launches(fn, 50)      # HIP events around 50 launches; returns synchronised
            n += 50
            last_us = us / 50
        snap1 = tel.snapshot()                    # ... to its end
        stats = tel.stop()
        stats.update(tel.between(snap0, snap1))
        row = {"workload": label, "us_per_launch": round(last_us, 2), "value": round(work / last_us / 1e6, 1), "unit": unit, **stats}
        if clock_buf is not None:
            c = clock_buf.download(np.uint64, 2)
            row["clock_in_kernel_mhz"] = round(float(c[0]) / max(float(c[1]), 1.0) * 100.0, 0)
        if idle_w[0] and stats.get("watts_mean"):
            # energy per operation (or byte) above the idle board, and the rate the package power cap would allow at that
            # energy: value x (cap - idle) / (W - idle), in the unit of value
            per_s = row["value"] * (1e12 if unit in ("tflops", "tops") else 1e9)
            row["pj_per_op_above_idle"] = round((stats["watts_mean"] - idle_w[0]) / per_s * 1e12, 4)
            if tel.cap_w:
                row["rate_at_power_cap"] = round(row["value"] * (tel.cap_w - idle_w[0]) / (stats["watts_mean"] - idle_w[0]), 1)
                row["of_rate_at_power_cap"] = round(row["value"] / row["rate_at_power_cap"], 4)
        out.append(row)
        print(json.dumps(row), flush=True)

    t0 = time.perf_counter()
    snap0 = tel.snapshot()
    tel.start(); time.sleep(min(seconds, 2.0)); idle = tel.stop(skip_s=0.0)
    idle.update(tel.between(snap0, tel.snapshot()))
    idle_w[0] = idle.get("watts_mean")
    print(json.dumps({"workload": "idle", "power_cap_w": tel.cap_w, **idle}), flush=True)
    M = N = K = 8192
    dA, dB, dC = dev.alloc(M * K * 2), dev.alloc(N * K * 2), dev.alloc(M * N * 2)
    flops = 2.0 * M * N * K
    dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
    run("gemm bf16 8192^3, seeded operands", lambda: dev.gemm_bf16(dA, dB, dC, M, N, K), flops, "tflops")
    dev.memset(dA, 0x3f); dev.memset(dB, 0x3f)
    run("gemm bf16 8192^3, constant operands (every byte 0x3f)", lambda: dev.gemm_bf16(dA, dB, dC, M, N, K), flops, "tflops")
    dev.memset(dA, 0); dev.memset(dB, 0)
    run("gemm bf16 8192^3, zero operands", lambda: dev.gemm_bf16(dA, dB, dC, M, N, K), flops, "tflops")
    for b in (dA, dB, dC):
        b.free()
    # the 8-bit and 4-bit kinds of the same kernel, seeded
    dA, dB, dC = dev.alloc(M * K), dev.alloc(N * K), dev.alloc(M * N * 4)
    dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, 448.0); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, 448.0)
    run("gemm fp8 e4m3 8192^3, seeded operands", lambda: dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1 / 448.0, 1 / 448.0), flops, "tflops")
    dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
    run("gemm int8 8192^3, seeded operands", lambda: dev.gemm_i8(dA, dB, dC, M, N, K), flops, "tops")
    dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
    dev.fill_bytes(dA, M * K // 2, SEED, wl.STREAM_GEMM_A, 0, 256); dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
    dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9); dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
    run("gemm block-scaled fp4 8192^3, seeded operands", lambda: dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K), flops, "tflops")
    for b in (dA, dB, dC, dSA, dSB):
        b.free()
    waves, iters = 2048, 4096
    clk = dev.alloc(16)
    # the register-resident rows as they are reported (one operand set per wave), every kind on seeded operands and four
    # of them on zero operands as well
    with_zero = (capi.MFMA_BF16_16x16x32, capi.MFMA_F16_32x32x16, capi.MFMA_MXFP6_E3M2)
    for kind in sorted(wl.DENSE):
        sh = wl.DENSE[kind]
        for zero in (False, True) if kind in with_zero else (False,):
            A, B, sA, sB = wl.dense_inputs(kind, waves, SEED)
            if zero:
                A, B = np.zeros_like(A), np.zeros_like(B)
            bufs = [dev.from_host(A), dev.from_host(B), dev.from_host(sA) if sA is not None else None, dev.from_host(sB) if sB is not None else None]
            o = dev.alloc(waves * 4 * sh["M"] * sh["N"] * 4)
            run(f"{sh['name']} {sh['shape']}, {'zero' if zero else 'seeded'} operands",
                lambda: dev.mfma_dense(kind, bufs[0], bufs[1], bufs[2], bufs[3], o, waves, iters, clk, one_set=True), wl.dense_flops(kind, waves, iters),
                "tops" if sh["fmt"] == wl.I8 else "tflops", clock_buf=clk)
            for b in bufs + [o]:
                if b is not None:
                    b.free()
    for kind in sorted(wl.SPARSE):
        sh = wl.SPARSE[kind]
        for zero in (False, True) if kind == capi.SMFMAC_F16_16x16x64 else (False,):
            Ac, meta, B = wl.sparse_inputs(kind, waves, SEED)
            if zero:
                Ac, B = np.zeros_like(Ac), np.zeros_like(B)
            bufs = [dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)]
            o = dev.alloc(waves * 4 * 256 * 4)
            run(f"{sh['name']} {sh['shape']}, {'zero' if zero else 'seeded'} operands",
                lambda: dev.smfmac(kind, bufs[0], bufs[1], bufs[2], o, waves, iters, clk, one_set=True), wl.sparse_flops(kind, waves, iters),
                "tops" if sh["fmt"] == wl.I8 else "tflops", clock_buf=clk)
            for b in bufs + [o]:
                b.free()
    # Where the limit acts: the same seeded launch with only part of the chip taking part (the other workgroups return at
    # once).  A limit on the package would let four busy XCDs, at half the power, run faster than eight.
    subsets = (("XCDs 0-3 only", dict(on_xcds=(0, 1, 2, 3)), 0.5), ("XCDs 0-1 only", dict(on_xcds=(0, 1)), 0.25), ("XCD 0 only", dict(on_xcds=(0,)), 0.125),
               ("XCDs 0 and 4 only", dict(on_xcds=(0, 4)), 0.25), ("half the CUs of every XCD", dict(half_cus=True), 0.5))
    for sparse, kind in ((True, capi.SMFMAC_F16_16x16x64), (False, capi.MFMA_F16_32x32x16), (False, capi.MFMA_BF16_16x16x32)):
        sh = (wl.SPARSE if sparse else wl.DENSE)[kind]
        if sparse:
            Ac, meta, B = wl.sparse_inputs(kind, waves, SEED)
            bufs = [dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)]
            work = wl.sparse_flops(kind, waves, iters)
            o = dev.alloc(waves * 4 * 256 * 4)
            fn = lambda **kw: dev.smfmac(kind, bufs[0], bufs[1], bufs[2], o, waves, iters, clk, one_set=True, **kw)
        else:
            A, B, _, _ = wl.dense_inputs(kind, waves, SEED)
            bufs = [dev.from_host(A), dev.from_host(B)]
            work = wl.dense_flops(kind, waves, iters)
            o = dev.alloc(waves * 4 * sh["M"] * sh["N"] * 4)
            fn = lambda **kw: dev.mfma_dense(kind, bufs[0], bufs[1], None, None, o, waves, iters, clk, one_set=True, **kw)
        for label, kw, share in subsets:
            run(f"{sh['name']} {sh['shape']}, seeded operands, {label}", lambda: fn(**kw), work * share, "tflops", clock_buf=clk)
        for b in bufs + [o]:
            b.free()
    # How fast the limit acts: isolated launches of increasing length (the board idle for 4 ms before each), with the
    # clock read inside the kernel (shader cycles over a constant-rate counter, by wave 0).  A limit on average power
    # would let a short launch from an idle board run at the boost clock.
    for kind in (capi.MFMA_F16_32x32x16,):
        sh = wl.DENSE[kind]
        for zero in (False, True):
            A, B, _, _ = wl.dense_inputs(kind, waves, SEED)
            if zero:
                A, B = np.zeros_like(A), np.zeros_like(B)
            bufs = [dev.from_host(A), dev.from_host(B)]
            o = dev.alloc(waves * 4 * sh["M"] * sh["N"] * 4)
            for n_it in (32, 128, 512, 2048, 4096):
                us, mhz = [], []
                for _ in range(12):
                    time.sleep(0.004)
                    us.append(dev.time_launches(lambda: dev.mfma_dense(kind, bufs[0], bufs[1], None, None, o, waves, n_it, clk), 1))
                    c = clk.download(np.uint64, 2)
                    mhz.append(float(c[0]) / max(float(c[1]), 1.0) * 100.0)
                us.sort(); mhz.sort()
                row = {"workload": f"{sh['name']} {sh['shape']}, {'zero' if zero else 'seeded'} operands, isolated launch of {n_it} iterations",
                       "us_per_launch": round(us[len(us) // 2], 1), "clock_in_kernel_mhz": round(mhz[len(mhz) // 2], 0)}
                out.append(row)
                print(json.dumps(row), flush=True)
            for b in bufs + [o]:
                b.free()
    clk.free()
    n_items, steps = 1 << 20, 4096
    o = dev.alloc(n_items * 8)
    run("mad fp32 float4 (vector FMA chains)", lambda: dev.compute_mad(capi.MAD_F32, 4, SEED, n_items, steps, o), n_items * 16 * steps * 2 * 1.0, "tflops")
    o.free()
    n = 1 << 30
    src, o = dev.alloc(n * 4), dev.alloc(dev.props.num_cus * 256 * 4)
    dev.fill_f32(src, n, SEED, wl.STREAM_BW, capi.DIST_U01)
    run("hbm float4 read over 4 GiB", lambda: dev.global_bandwidth(4, src, n, o, dev.props.num_cus, 256), n * 4 * 1e3, "gbps")
    src.free(); o.free()
    return out


def _llc_bytes():
    """Total last-level cache of the machine: the sum of the distinct L3 caches sysfs lists."""
    seen, total = set(), 0
    base = "/sys/devices/system/cpu"
    try:
        cpus = [d for d in os.listdir(base) if d.startswith("cpu") and d[3:].isdigit()]
    except OSError:
        return 0
    for c in cpus:
        d = os.path.join(base, c, "cache", "index3")
        try:
            shared = open(os.path.join(d, "shared_cpu_list")).read().strip()
            size = open(os.path.join(d, "size")).read().strip()
        except OSError:
            continue
        if shared in seen:
            continue
        seen.add(shared)
        mult = {"K": 1 << 10, "M": 1 << 20, "G": 1 << 30}.get(size[-1].upper(), 1)
        total += int(size[:-1] if size[-1].isalpha() else size) * mult
    return total


def _stream_floats(threads):
    """Array length of the DRAM test, the reference's rule (src/cpu/bandwidth.cpp:250-265): four times the
    last-level cache, at least 64 MiB, at most 512 MiB unless that is less than twice the cache."""
    llc = _llc_bytes()
    array_bytes = max(4 * llc, 64 << 20)
    try:
        total_mem = os.sysconf("SC_PAGE_SIZE") * os.sysconf("SC_PHYS_PAGES")
    except (ValueError, OSError):
        total_mem = 0
    cap = min(512 << 20, total_mem // 16) if total_mem else 512 << 20
    if cap < 2 * llc:
        cap = 2 * llc
    # A virtual machine can under-report its caches (one 32 MiB L3 for 16 vCPUs that really sit on several
    # chiplets), which would leave every thread's chunk cache-resident: never go below 2 GiB.
    n = max(min(array_bytes, cap), 2 << 30) // 4
    return max(n // threads * threads, threads), llc


def _port_families(orc, pool, target_us):
    """The CPU oracle's kernel of every GPU row family, timed at one thread and at all of them on a bounded sample
    of the same seeded workload.  Returns {row: figures}; "_headline" is the raw result of the float4 read."""
    from oracle import workloads as owl
    port = {}
    small = 60_000        # budget of a timed batch of the emulated families, in microseconds

    def entry(q, unit, what):
        return {"ST": round(q.giga_st, 3), "MT": round(q.giga_mt, 3), "unit": unit, "threads": q.threads_mt,
                "iters_ST": q.iters_st, "iters_MT": q.iters_mt, "sample": what}

    def ptr(a):
        return a.ctypes.data if a is not None else None

    # --- read-reduce over the 256 MiB buffer of the CPU configuration, 2^20 partial sums, every width
    n, T = 1 << 26, 1 << 20
    buf = orc.fill_f32(n, SEED, owl.STREAM_BW, 0)
    for width, metric in ((4, "float4"), (2, "float2"), (1, "float")):
        op = orc.CpuhOp(op=orc.OP_READ, width=width, p0=ptr(buf), n_floats=n, T=T)
        q = pool.measure_op(op, n * 4.0, n * 4.0 / pool.max_threads, target_us=target_us if width == 4 else small, keep=(buf,))
        port[f"global_memory_bandwidth {metric}"] = entry(q, "GB/s", f"{metric} read-reduce over a 256 MiB (2^26 float) seeded buffer, "
                                                          "2^20 partial sums, one pass per iteration")
        if width == 4:
            port["_headline"] = q
    del buf
    # --- vector multiply-add chains: 8 work-items x 16 accumulators (or `chains`) x 4096 steps per iteration
    for row, kind, width, chains, ops, unit in (
            ("single_precision_compute float4", 0, 4, 16, 2, "gflops"), ("half_precision_compute half2", 1, 2, 16, 2, "gflops"),
            ("double_precision_compute double", 2, 1, 16, 2, "gflops"), ("mixed_precision_compute mp", 3, 1, 16, 2, "gflops"),
            ("bfloat16_compute bf16", 4, 1, 16, 4, "gflops"), ("integer_compute int", 5, 1, 16, 2, "gops"),
            ("integer_compute_int8_dp int8_dp8", 6, 8, 8, 8, "gops")):
        op = orc.CpuhOp(op=orc.OP_MAD, kind=kind, width=width, seed=SEED)
        q = pool.measure_op(op, orc.OP_MAD_ITEMS * chains * 4096.0 * ops, warmup=1, target_us=target_us if kind == 0 else small)
        port[row] = entry(q, unit, f"{orc.OP_MAD_ITEMS} work-items x {chains} chains x 4096 steps per iteration")
    # --- emulated matrix instructions: the 4 chains of one wave, one instruction each, per iteration
    for kind, sh in sorted(owl.DENSE.items()):
        A, B, sA, sB = owl.dense_inputs(kind, 1, SEED)
        op = orc.CpuhOp(op=orc.OP_MFMA, kind=kind, p0=ptr(A), p1=ptr(B), p2=ptr(sA), p3=ptr(sB))
        q = pool.measure_op(op, 4 * 2.0 * sh["M"] * sh["N"] * sh["K"], warmup=1, target_us=small, keep=(A, B, sA, sB))
        port[sh["name"]] = entry(q, "gops" if sh["fmt"] is None else "gflops", f"4 emulated {sh['shape']} products per iteration (one wave of 2048)")
    for kind, sh in sorted(owl.SPARSE.items()):
        Ac, meta, B = owl.sparse_inputs(kind, 1, SEED)
        op = orc.CpuhOp(op=orc.OP_SMFMAC, kind=kind, p0=ptr(Ac), p1=ptr(meta), p2=ptr(B))
        q = pool.measure_op(op, 4 * 2.0 * 16 * 16 * sh["K"], warmup=1, target_us=small, keep=(Ac, meta, B))
        port[sh["name"]] = entry(q, "gops" if sh["fmt"] is None else "gflops",
                                 f"4 emulated 2:4 sparse {sh['shape']} products per iteration, dense-equivalent operations")
    # --- GEMM: one 32x32 tile of the K = 8192 product per iteration (of 65536 such tiles)
    K, t = 8192, 32
    for row, fa, fb, unit in (("rocblas-fp bf16", orc.FMT_BF16, orc.FMT_BF16, "gflops"), ("rocblas-fp fp16", orc.FMT_F16, orc.FMT_F16, "gflops"),
                              ("rocblas-fp fp32", orc.FMT_F32, orc.FMT_F32, "gflops"), ("rocblas-fp fp64", orc.FMT_F64, orc.FMT_F64, "gflops"),
                              ("hipblaslt-fp8 fp8_e4m3", orc.FMT_E4M3, orc.FMT_E4M3, "gflops"),
                              ("hipblaslt-fp8 fp8_e5m2", orc.FMT_E5M2, orc.FMT_E4M3, "gflops"), ("rocblas-int int8", orc.FMT_I8, orc.FMT_I8, "gops")):
        def operand(fmt, stream):
            if fmt == orc.FMT_I8:
                return orc.fill_int8(SEED, stream, t * K)
            if fmt == orc.FMT_F32:
                return orc.fill_f32(t * K, SEED, stream, 1)
            if fmt == orc.FMT_F64:
                return orc.fill_f32(t * K, SEED, stream, 1).astype(np.float64)
            return orc.fill_fmt(fmt, t * K, SEED, stream, 1, 448.0 if fmt == orc.FMT_E4M3 else 57344.0 if fmt == orc.FMT_E5M2 else 1.0)
        A, B = operand(fa, owl.STREAM_GEMM_A), operand(fb, owl.STREAM_GEMM_B)
        op = orc.CpuhOp(op=orc.OP_GEMM, kind=fa, width=fb, p0=ptr(A), p1=ptr(B), K=K, tile=t, scale=1.0)
        q = pool.measure_op(op, 2.0 * t * t * K, warmup=1, target_us=small, keep=(A, B))
        port[row] = entry(q, unit, f"one {t}x{t} tile of the K={K} product per iteration")
    A, B = orc.fill_bytes(t * K // 2, SEED, owl.STREAM_GEMM_A, 0, 256), orc.fill_bytes(t * K // 2, SEED, owl.STREAM_GEMM_B, 0, 256)
    SA, SB = orc.fill_bytes(t * K // 32, SEED, owl.STREAM_SCALE_A, 123, 9), orc.fill_bytes(t * K // 32, SEED, owl.STREAM_SCALE_B, 123, 9)
    op = orc.CpuhOp(op=orc.OP_GEMM_MX, p0=ptr(A), p1=ptr(B), p2=ptr(SA), p3=ptr(SB), K=K, tile=t)
    q = pool.measure_op(op, 2.0 * t * t * K, warmup=1, target_us=small, keep=(A, B, SA, SB))
    port["hipblaslt-fp8 mxf4_e2m1"] = entry(q, "gflops", f"one {t}x{t} tile of the K={K} block-scaled product per iteration")
    return port


def cpu_baseline(target_us=1_500_000, extra_target_us=600_000):
    """CPU figures beside the GPU ones, all timed with the reference's CPU discipline (pinned persistent
    pool, warm-ups, settle phase before the all-core run, adaptive probe, one timed batch sized to the
    budget), at one thread (ST) and at every logical core (MT).

    Where the build of the reference's own CPU kernels exists (oracle/_ref, made from the reference's
    sources on the machine that has them) the headline value is the reference's DRAM read kernel and its
    fp32 chain is listed too (kind "reference"); the oracle's kernels on the seeded workloads (kind
    "port") are always listed under "port"."""
    from oracle import pyoracle as orc
    cores = len(os.sched_getaffinity(0))
    t0 = time.perf_counter()
    ref = orc.reference_kernels()
    with orc.CpuPool(cores) as pool:
        port = _port_families(orc, pool, extra_target_us)
        r = port.pop("_headline")
        # the other two rows of the reference's DRAM test, restated (all workers only, as it times them)
        n_stream, llc = _stream_floats(cores)
        for name, kind, what in (("global_memory_bandwidth copy", 0, "memcpy of one array into another, 2 x 4 bytes per element"),
                                 ("global_memory_bandwidth triad", 1, "a[i] = b[i] + 1.5 c[i], 3 x 4 bytes per element")):
            q, _ = pool.measure_stream(pool.own_populate_ptr(), n_stream, kind, 1, extra_target_us)
            port[name] = {"MT": round(q.giga_mt, 2), "unit": "GB/s", "threads": q.threads_mt, "iters_MT": q.iters_mt,
                          "sample": f"{what}; three arrays of {n_stream * 4 >> 20} MiB, per-thread contiguous chunks"}
        reference = None
        if ref is not None:
            rd = pool.measure_read_fn(ref["read_fn"], ref["populate_fn"], n_stream, 2, target_us)
            ch = pool.measure_chain_fn(ref["fp32_fn"], ref["fp32_ops"], 2, extra_target_us)
            reference = {"isa": ref["isa"],
                         "global_memory_bandwidth read": {"ST": round(rd.giga_st, 2), "MT": round(rd.giga_mt, 2), "unit": "GB/s",
                                                          "iters_ST": rd.iters_st, "iters_MT": rd.iters_mt},
                         "single_precision_compute float": {"ST": round(ch.giga_st, 2), "MT": round(ch.giga_mt, 2),
                                                            "unit": "gflops", "iters_ST": ch.iters_st, "iters_MT": ch.iters_mt}}
    dt = time.perf_counter() - t0
    if reference is not None:
        value, kind = reference["global_memory_bandwidth read"]["MT"], "reference"
        sample = (f"the reference's DRAM read kernel (readBufferChecksum, {ref['isa']} build of its own source) over a "
                  f"{n_stream * 4 >> 20} MiB array (its sizing rule but at least 2 GiB; reported last-level cache {llc >> 20} MiB) filled by its populate(), "
                  f"per-thread contiguous chunks: {rd.iters_st} passes on 1 thread, "
                  f"{rd.iters_mt} passes on {rd.threads_mt} threads; whole CPU leg {dt:.1f} s")
    else:
        value, kind = port["global_memory_bandwidth float4"]["MT"], "port"
        sample = (f"float4 read-reduce over a 256 MiB (2^26 float) seeded buffer, 2^20 partial sums, C oracle (no fast-math): "
                  f"{r.iters_st} passes on 1 thread, {r.iters_mt} passes on {r.threads_mt} threads; whole CPU leg {dt:.1f} s")
    return {"value": value, "unit": "GB/s", "cores": r.threads_mt, "kind": kind, "pinned_workers": r.pinned,
            "sample": sample, "reference": reference, "port": port}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-rows", action="store_true", help="headline kernel only")
    ap.add_argument("--quick", action="store_true", help="shorter time budget per extra row")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--rows-file", default=os.path.join(ROOT, "gpurun_out", "bench_rows.json"),
                    help="where the full record (every row, every CPU figure) is written; '' to skip")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only the plain copy kernel over 1 GiB (20 launches): under rocprofv3 --pmc this "
                         "gives what FETCH_SIZE / WRITE_SIZE read for a transfer of known size")
    ap.add_argument("--power-table", type=float, default=0.0, metavar="SECONDS",
                    help="run only the power / clock telemetry: each matrix workload for SECONDS while board power and "
                         "shader clock are sampled from sysfs every 10 ms; one JSON line per workload")
    ap.add_argument("--only", default="mad,latency,mfma,smfmac,matrix_distinct,matrix_zero,matrix_ref,gemm,gemm_const,lds,transfer",
                    help="comma list of extra row groups to run: mad,latency,mfma,smfmac,matrix_distinct,matrix_zero,matrix_ref,gemm,gemm_const,lds,transfer; "
                         "and, not among the defaults, vendor: the vendor library's GEMM beside this library's (needs torch); "
                         "gemm_small: 2048 cubed on the 128x128 and on the 256x256 tiles")
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor library's bf16 / fp8 / FP4 GEMM beside this library's (a child process that imports torch)")
    ap.add_argument("--vendor-child", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.vendor_child:
        _vendor_child()
        return
    if "vendor" in args.only.split(","):
        # torch brings a HIP runtime of its own: it has to be the one that initialises the device in this process
        import torch
        torch.cuda.init()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; the hot path has no multi-GPU step "
                 "(every kernel is independent per device), run with --gpus 1")

    vendor = []
    # (not under a profiler, which would follow the child and report its kernels among this library's)
    profiled = any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ)
    if not (args.no_rows or args.no_vendor or profiled or args.power_table or args.calibrate_copy or "gemm" not in args.only.split(",")):
        progress("vendor library's bf16 / fp8 / block-scaled FP4 GEMM in a child process (torch)")
        vendor = vendor_beside()
    from clpeak_amd import capi
    from clpeak_amd import workloads as wl
    dev = capi.Device(0)

    if args.power_table:
        power_table(dev, args.power_table)
        dev.close()
        return

    if args.calibrate_copy:
        nbytes = 1 << 30
        a, b = dev.alloc(nbytes), dev.alloc(nbytes)
        dev.fill_f32(a, nbytes // 4, SEED, wl.STREAM_BW, capi.DIST_U01)
        for _ in range(20):
            dev.copy(b, a, nbytes)
        dev.sync()
        print(json.dumps({"calibrate_copy_bytes": nbytes, "launches": 20}))
        return

    n = 1 << 30                                   # 4 GiB of fp32, far past the 256 MB Infinity Cache
    src = dev.alloc(n * 4)
    dev.fill_f32(src, n, SEED, wl.STREAM_BW, capi.DIST_U01)
    blocks, bs = dev.props.num_cus * HEADLINE_BLOCKS_PER_CU, 256
    out = dev.alloc(blocks * bs * 4)
    step = lambda: dev.global_bandwidth(4, src, n, out, blocks, bs)

    for _ in range(args.warmup):
        step()
    dev.sync()
    t0 = time.perf_counter()
    ev_us = dev.time_launches(step, args.steps)   # HIP events on the kernel's stream; ends synchronised
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_us = ev_us / args.steps
    gbps = n * 4 / (wall / args.steps) / 1e9

    rows = []
    # the other two widths of the same test, same discipline
    for width, metric in ((1, "float"), (2, "float2")):
        fn = lambda: dev.global_bandwidth(width, src, n, out, blocks, bs)
        for _ in range(max(args.warmup // 4, 2)):
            fn()
        us = dev.time_launches(fn, max(args.steps // 4, 1)) / max(args.steps // 4, 1)
        rows.append({"test": "global_memory_bandwidth", "metric": metric, "value": round(n * 4 / us / 1e3, 2), "unit": "gbps",
                     "us_per_launch": round(us, 2), "peak": HBM_PEAK_GBPS, "frac": round(n * 4 / us / 1e3 / HBM_PEAK_GBPS, 4)})
    src.free(); out.free()
    if not args.no_rows:
        rows += bench_rows(dev, args.quick, set(args.only.split(",")))
    rows += vendor
    dev.close()
    if not args.no_cpu:
        progress("CPU baseline leg")

    achieved = n * 4 / kernel_us / 1e3
    full = {
        "metric": "MFMA TFLOPS/TOPS per dtype (dense, 2:4) + HBM GB/s, as % of MI355X peak",
        "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "HBM streaming read: float4 grid-stride read-reduce over a 4 GiB fp32 buffer "
                               "(uniform[0,1) seeded on device), one fp32 partial sum per thread",
                   "buffer_bytes": n * 4, "threads": blocks * bs, "pct_of_peak": round(100 * gbps / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel_us": round(kernel_us, 2), "algorithmic_bytes": n * 4},
        "cpu_baseline": None if args.no_cpu else cpu_baseline(),
        "rows": rows,
        "rows_file": os.path.relpath(args.rows_file, ROOT) if args.rows_file else None,
    }
    emit(full, args.rows_file)


def emit(full, rows_file):
    """Write the whole record (every row, every CPU figure) to `rows_file`, list the rows on stderr, and
    print the compact record as the LAST line of stdout."""
    if rows_file:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(rows_file)), exist_ok=True)
            with open(rows_file, "w") as f:
                json.dump(full, f, indent=1)
        except OSError as e:
            sys.stderr.write(f"bench.py: could not write {rows_file}: {e}\n")
    for r in full["rows"]:
        frac = f"  {100 * r['frac']:5.1f} % of {r['peak']:g}" if "frac" in r else ""
        clk = f"  {r['sclk_mhz']:.0f} MHz" if "sclk_mhz" in r else ""
        sys.stderr.write(f"{r['test']:28s} {r['metric']:44s} {r['value']:12.2f} {r['unit']:6s} {r['us_per_launch']:10.2f} us{frac}{clk}\n")
    sys.stderr.flush()
    print(json.dumps(compact_line(full), separators=(",", ":")), flush=True)


# One number per target of the workload list: (key in "fracs", test, metric).
FRAC_KEYS = [("hbm_float", "global_memory_bandwidth", "float"), ("hbm_float2", "global_memory_bandwidth", "float2"),
             ("mad_fp32", "single_precision_compute", "float4"), ("mad_fp64", "double_precision_compute", "double"),
             ("mfma_fp16", "mfma_fp16", "mfma_fp16"), ("mfma_bf16", "mfma_bf16", "mfma_bf16"),
             ("mfma_fp16_32x32x16", "mfma_fp16_32x32x16", "mfma_fp16_32x32x16"),
             ("mfma_bf16_32x32x16", "mfma_bf16_32x32x16", "mfma_bf16_32x32x16"),
             ("mfma_int8", "mfma_int8", "mfma_int8"), ("mfma_fp8", "mfma_fp8", "mfma_fp8"), ("mfma_bf8", "mfma_bf8", "mfma_bf8"),
             ("mfma_mxfp6_e2m3", "mfma_mxfp6_e2m3", "mfma_mxfp6_e2m3"), ("mfma_mxfp6_e3m2", "mfma_mxfp6_e3m2", "mfma_mxfp6_e3m2"),
             ("mfma_mxfp4", "mfma_mxfp4", "mfma_mxfp4"),
             ("smfmac_fp16", "smfmac_fp16", "smfmac_fp16"), ("smfmac_bf16", "smfmac_bf16", "smfmac_bf16"),
             ("smfmac_fp8", "smfmac_fp8", "smfmac_fp8"), ("smfmac_bf8", "smfmac_bf8", "smfmac_bf8"),
             ("smfmac_int8", "smfmac_int8", "smfmac_int8"),
             ("gemm_bf16_seeded", "rocblas-fp", "bf16"), ("gemm_fp16_seeded", "rocblas-fp", "fp16"),
             ("gemm_fp32", "rocblas-fp", "fp32"), ("gemm_fp64", "rocblas-fp", "fp64"),
             ("gemm_fp8_e4m3_seeded", "hipblaslt-fp8", "fp8_e4m3"), ("gemm_fp8_e5m2_seeded", "hipblaslt-fp8", "fp8_e5m2"),
             ("gemm_mxfp4_seeded", "hipblaslt-fp8", "mxf4_e2m1"), ("gemm_int8_seeded", "rocblas-int", "int8"),
             ("gemm_bf16_const", "rocblas-fp", "bf16 constant operands"),
             ("gemm_bf16_vendor", "rocblas-fp", "bf16 vendor library, uniform random operands"),
             ("gemm_fp8_vendor", "hipblaslt-fp8", "fp8_e4m3 vendor library, uniform random operands"),
             ("gemm_mxfp4_vendor", "hipblaslt-fp8", "mxf4_e2m1 vendor library, uniform random operands"),
             ("lds_float4", "local_memory_bandwidth", "float4")]


# What the workload list asks of each family, as a fraction of the datasheet peak.
TARGET_FRAC = {"mfma": 0.85, "smfmac": 0.80, "hbm": 0.85, "gemm": 0.70}


def compact_line(full):
    """The record the driver reads: the contract's keys, the roofline of the headline kernel, the CPU
    baseline's headline figures and one fraction of peak per target; kept under 2000 bytes (the full
    record with every row is in the rows file)."""
    line = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                                 "scaling", "vs_baseline", "dtype", "data")}
    line["config"] = {"workload": "HBM streaming read: float4 grid-stride read-reduce over a 4 GiB seeded fp32 buffer",
                      "buffer_bytes": full["config"]["buffer_bytes"], "threads": full["config"]["threads"]}
    line["roofline"] = full["roofline"]
    cb = full.get("cpu_baseline")
    if cb is not None:
        c = {k: cb[k] for k in ("value", "unit", "cores", "kind")}
        head = (cb.get("reference") or {}).get("global_memory_bandwidth read") or cb["port"]["global_memory_bandwidth float4"]
        c["ST"], c["MT"] = head.get("ST"), head.get("MT")
        c["sample"] = cb["sample"][:120]
        line["cpu_baseline"] = c
    else:
        line["cpu_baseline"] = None
    by_key = {(r["test"], r["metric"]): r for r in full["rows"]}
    fracs = {}
    for key, test, metric in FRAC_KEYS:
        r = by_key.get((test, metric))
        if r is not None and "frac" in r:
            fracs[key] = round(r["frac"], 3)
    line["fracs"] = fracs
    # which launch the matrix fractions are: the four accumulator chains of a wave share one A and one B
    # fragment (the rows "distinct operands per chain" in the rows file are the other launch)
    line["mfma_operands"] = "one set per wave"
    # for each matrix or bf16 GEMM row below its target: [clock held (MHz, read inside the kernel; null for the GEMM, which does
    # not read it), board power during the timed batch (W)]
    held = {}
    for key, test, metric in FRAC_KEYS:
        r = by_key.get((test, metric))
        target = TARGET_FRAC.get(key.split("_")[0]) if key.startswith(("mfma", "smfmac")) or key == "gemm_bf16_seeded" else None
        if r is not None and target and r.get("frac", 1.0) < target and ("sclk_mhz" in r or "watts" in r):
            held[key] = [int(r["sclk_mhz"]) if "sclk_mhz" in r else None, int(round(r["watts"])) if "watts" in r else None]
    line["below_target_mhz_w"] = held
    lat = by_key.get(("kernel_launch_latency", "roundtrip"))
    if lat is not None:
        line["launch_roundtrip_us"] = lat["value"]
    line["rows_file"] = full.get("rows_file")
    # the record must fit a reader that keeps a 2000-byte tail of stdout: the free text gives way first (it is whole in the rows file)
    while len(json.dumps(line, separators=(",", ":")).encode()) > 1950 and line["cpu_baseline"] and line["cpu_baseline"]["sample"]:
        line["cpu_baseline"]["sample"] = line["cpu_baseline"]["sample"][:-20]
    return line


# Workgroups per CU of the headline launch (256 threads each); one per CU measured best (a
# small grid keeps the strided loads of one unrolled group inside a few 2 MiB pages).
HEADLINE_BLOCKS_PER_CU = 1
# HBM bytes per launch of the headline kernel from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE in
# KiB per dispatch), each scaled by what the counter reads for the plain copy kernel of known size
# (FETCH_SIZE x 2.0000, WRITE_SIZE x 1.0000 to four decimals): profiles/hbm_float4_read_4GiB_traffic.md.
TRAFFIC_BYTES_PER_LAUNCH = 4295171094

if __name__ == "__main__":
    main()
