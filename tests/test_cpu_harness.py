"""CPU baseline harness: pool, timing discipline, ST/MT accounting.

The harness restates src/cpu/thread_pool.cpp:23-102 (pool), src/cpu/cpu_peak.cpp:46-128
(run_workload), src/common/common.cpp:35-45 (pick_iters) and src/cpu/compute_common.h:21-60 (ST/MT
values) of the reference.  These tests pin it against what those sources fix: the clamp rules of
pick_iters at their documented corners, a body of known duration, the dispatch contract of the pool
(exactly workers 0..n-1 run, each once), and the giga-unit formula.
"""
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from oracle import workloads as wl


@pytest.fixture(scope="module")
def pool():
    p = orc.CpuPool(min(4, len(os.sched_getaffinity(0))))
    yield p
    p.close()


@pytest.mark.parametrize("per_iter, target, forced, cap, want", [
    (10.0, 1000, 0, 10000, 100),          # target / per-iteration time
    (0.01, 1000, 0, 10000, 1000),         # per-iteration time floors at 1 us
    (1.0, 0, 0, 100000000, 5000000),      # target 0 means the 5 s legacy default
    (1.0, 10**9, 0, 10000, 10000),        # clamp to the cap
    (5000.0, 1000, 0, 10000, 1),          # never below one iteration
    (123.0, 1000, 77, 10000, 77),         # forced wins over everything
    (3.0, 1000, 0, 10000, 333),           # truncation, not rounding
])
def test_pick_iters_corners(per_iter, target, forced, cap, want):
    assert orc.pick_iters(per_iter, target, forced, cap) == want


def test_pool_runs_exactly_the_first_n_workers(pool):
    for n in range(1, pool.max_threads + 1):
        counts = pool.count(n, 7)
        want = np.array([(t + 1) * 7 if t < n else 0 for t in range(pool.max_threads)], dtype=np.uint64)
        assert (counts == want).all(), (n, counts)
    # n outside [1, max] is clamped, as the reference's run() does
    assert pool.count(0, 1)[0] == 1
    assert (pool.count(pool.max_threads + 5, 1) > 0).all()


def test_workers_are_pinned_to_their_own_cpu(pool):
    pool.count(pool.max_threads, 1)  # every worker has started once this returns
    allowed = os.sched_getaffinity(0)
    for t in range(pool.max_threads):
        got = pool.pinned_cpu(t)
        if t in allowed:
            assert got == t
        else:
            assert got in (t, -1)   # pinning outside the allowed set may be refused: best effort


def test_run_workload_recovers_a_known_iteration_time(pool):
    # a body that sleeps 500 us per iteration: the probe must grow past one iteration (2 ms rule), the
    # batch must be sized for the 100 ms budget, and the mean must come back near 500 us (sleep overshoots)
    for n in (1, pool.max_threads):
        us, iters = pool.time_sleep_body(n, 500, 100_000)
        assert 500.0 <= us < 5000.0, us          # sleep overshoots, much more so on a busy machine
        assert 100_000 / 5000.0 <= iters <= 100_000 / 500.0 + 1, iters


def test_ranged_read_reduce_is_the_same_sum():
    n, T = 1 << 18, 1 << 10
    data = orc.fill_f32(n, wl.DEFAULT_SEED, wl.STREAM_BW, 0)
    for width in (1, 2, 4):
        whole = orc.global_bandwidth(width, data, T)
        parts = np.zeros(T, dtype=np.float32)
        for t0, t1 in ((0, 100), (100, 101), (101, 777), (777, T)):
            orc.global_bandwidth_range(width, data, T, t0, t1, parts)
        assert (parts.view(np.uint32) == whole.view(np.uint32)).all()
    # ragged tail: the last stride is only partly filled
    data = data[: n - 4 * 300]
    whole = orc.global_bandwidth(4, data, T)
    parts = np.zeros(T, dtype=np.float32)
    orc.global_bandwidth_range(4, data, T, 0, 512, parts)
    orc.global_bandwidth_range(4, data, T, 512, T, parts)
    assert (parts.view(np.uint32) == whole.view(np.uint32)).all()


def test_measure_reports_st_and_mt_in_giga_units(pool):
    r = pool.measure(orc.CPUH_MAD_F32, wl.DEFAULT_SEED, warmup=1, target_us=50_000)
    assert r.threads_mt == pool.max_threads
    assert r.iters_st >= 1 and r.iters_mt >= 1
    # one iteration = 8 items x 16 accumulators x 4096 fma x 2 flops
    assert r.units_per_iter_st == 8 * 16 * 4096 * 2
    assert r.giga_st == pytest.approx(r.units_per_iter_st / (r.us_st * 1e3))
    assert r.giga_mt == pytest.approx(r.units_per_iter_mt * r.threads_mt / (r.us_mt * 1e3))
    assert 0.05 < r.giga_st < 1000.0          # a scalar fma chain on any x86 core of this decade
    with pytest.raises(RuntimeError):
        pool.measure(99, 1)


def test_chain_given_as_function_pointer_is_priced_per_thread(pool):
    import ctypes as C
    import time
    calls = []

    @C.CFUNCTYPE(C.c_double, C.c_uint64)
    def chain(outer):           # 200 us per outer iteration, whatever thread runs it
        calls.append(outer)
        time.sleep(200e-6 * outer)
        return 1.0

    r = pool.measure_chain_fn(C.cast(chain, C.c_void_p).value, 1000.0, warmup=1, target_us=40_000)
    assert r.threads_mt == pool.max_threads and r.units_per_iter_st == 1000.0
    assert 200.0 <= r.us_st < 2000.0 and 200.0 <= r.us_mt < 2000.0   # sleep overshoots on a busy machine
    # 1000 units per 200+ us on one thread: < 5 giga-units / 1000; MT counts every thread's units
    assert r.giga_st == pytest.approx(1000.0 / (r.us_st * 1e3))
    assert r.giga_mt == pytest.approx(1000.0 * r.threads_mt / (r.us_mt * 1e3))
    # the timed batch is ONE dispatch whose body loops itself: the batch sizes were passed as `outer`
    assert r.iters_st in calls and calls.count(r.iters_mt) >= pool.max_threads


def test_reference_kernels_run_under_the_harness(pool):
    ref = orc.reference_kernels()
    if ref is None:
        pytest.skip("reference build (oracle/_ref) not present")
    # ops per outer iteration = INNER * NACC * LANES * 2 of the ISA's table entry (src/cpu/cpu_kernels_impl.h:54)
    assert ref["fp32_ops"] in (4096 * 12 * 8 * 2.0, 4096 * 24 * 16 * 2.0)
    ch = pool.measure_chain_fn(ref["fp32_fn"], ref["fp32_ops"], warmup=1, target_us=50_000)
    # a SIMD FMA chain that scales with threads (other work on the machine may take some of them away)
    assert 5.0 < ch.giga_st < 500.0 and ch.giga_mt > (ch.giga_st if pool.max_threads >= 4 else 0.5 * ch.giga_st)
    rd = pool.measure_read_fn(ref["read_fn"], ref["populate_fn"], 1 << 24, warmup=1, target_us=50_000)
    assert 1.0 < rd.giga_st < 200.0 and rd.giga_mt > 0.4 * rd.giga_st
    assert rd.units_per_iter_st == (1 << 24) // pool.max_threads * pool.max_threads * 4.0


def test_populate_restated_against_the_first_values_and_its_mask():
    """xorshift32 from 0xDEADBEEF (src/common/common.cpp:76-95): the first states computed here by hand in
    Python; the mask clears the sign and sets the lowest exponent bit, so every value is positive and normal
    or, one time in 128, has an all-ones exponent (the reference's comment calls them all finite; they are not)."""
    import ctypes as C
    L = orc.lib()
    n = 1000
    buf = np.zeros(n, dtype=np.float32)
    L.cpuh_populate.argtypes = [C.c_void_p, C.c_ulonglong]; L.cpuh_populate.restype = None
    L.cpuh_populate(buf.ctypes.data, n)
    state, want = 0xDEADBEEF, []
    for _ in range(n):
        state ^= (state << 13) & 0xFFFFFFFF
        state ^= state >> 17
        state ^= (state << 5) & 0xFFFFFFFF
        want.append((state & 0x7F7FFFFF) | 0x00800000)
    assert [int(x) for x in buf.view(np.uint32)] == want
    bits = buf.view(np.uint32)
    assert np.all(bits >> 31 == 0) and np.all((bits >> 23) & 1 == 1)
    assert 0 < np.count_nonzero(~np.isfinite(buf)) < n // 32


@pytest.mark.parametrize("kind", [0, 1])
def test_stream_copy_and_triad_rows(kind):
    """copy: A = C; triad: A = B + 1.5 C (src/cpu/bandwidth.cpp:323-352).  All three arrays hold the same
    populate() sequence per chunk, so after any number of passes A[i] is C[i] or B[i] + 1.5 C[i] = 2.5 C[i];
    bytes per pass are 2 N x 4 and 3 N x 4."""
    n = 1 << 20
    with orc.CpuPool(4) as pool:
        r, probe = pool.measure_stream(pool.own_populate_ptr(), n, kind, 1, 20_000)
    a_mid, b_mid, c_mid = probe[1], probe[3], probe[4]
    assert b_mid.view(np.uint32) == c_mid.view(np.uint32) and np.isfinite(c_mid) and c_mid > 0
    with np.errstate(over="ignore"):
        want = c_mid if kind == 0 else np.float32(np.float32(1.5) * c_mid) + b_mid
    assert a_mid.view(np.uint32) == np.float32(want).view(np.uint32)
    assert r.iters_mt >= 1 and r.us_mt > 0 and r.threads_mt == 4
    assert r.units_per_iter_st == (2 if kind == 0 else 3) * n * 4
    assert abs(r.giga_mt - r.units_per_iter_st / (r.us_mt * 1e3)) <= 1e-6 * r.giga_mt
    assert r.giga_st == -1.0 and r.iters_st == 0          # all workers only, as the reference times these rows


def test_measure_op_times_any_oracle_kernel_on_given_operands():
    """cpuh_measure_op: the harness's discipline around one oracle kernel on operands the caller built.  Unit
    accounting is the caller's: giga = units x threads / (us x 1e3); and a full-size CPU baseline families
    table builds without a GPU."""
    from oracle import workloads as owl
    with orc.CpuPool(2) as pool:
        A, B, _, _ = owl.dense_inputs(4, 1, 3)          # int8 16x16x64, the 4 chains of one wave
        op = orc.CpuhOp(op=orc.OP_MFMA, kind=4, p0=A.ctypes.data, p1=B.ctypes.data)
        units = 4 * 2.0 * 16 * 16 * 64
        r = pool.measure_op(op, units, warmup=1, target_us=20_000, keep=(A, B))
        assert r.iters_st >= 1 and r.iters_mt >= 1 and r.threads_mt == 2
        assert abs(r.giga_st - units / (r.us_st * 1e3)) <= 1e-9 * r.giga_st
        assert abs(r.giga_mt - units * 2 / (r.us_mt * 1e3)) <= 1e-9 * r.giga_mt
        # the read splits one pass over the buffer among the threads
        n, T = 1 << 20, 1 << 12
        buf = orc.fill_f32(n, 3, owl.STREAM_BW, 0)
        op = orc.CpuhOp(op=orc.OP_READ, width=2, p0=buf.ctypes.data, n_floats=n, T=T)
        r = pool.measure_op(op, n * 4.0, n * 4.0 / 2, warmup=1, target_us=20_000, keep=(buf,))
        assert r.units_per_iter_st == n * 4.0 and r.units_per_iter_mt == n * 2.0 and r.giga_mt > 0
        with pytest.raises(RuntimeError):
            pool.measure_op(orc.CpuhOp(op=99), 1.0)


def test_cpu_baseline_covers_every_gpu_row_family():
    """The families table of the benchmark driver's CPU leg names one oracle kernel per GPU row family."""
    import bench
    with orc.CpuPool(2) as pool:
        port = bench._port_families(orc, pool, 30_000)   # tiny budgets: this checks coverage and plumbing, not speed
    port.pop("_headline")
    tests_covered = {k.split(" ")[0] for k in port}
    for test in ("global_memory_bandwidth", "single_precision_compute", "half_precision_compute", "double_precision_compute",
                 "mixed_precision_compute", "bfloat16_compute", "integer_compute", "integer_compute_int8_dp",
                 "mfma_fp16", "mfma_bf16", "mfma_fp16_32x32x16", "mfma_bf16_32x32x16", "mfma_int8", "mfma_fp8", "mfma_bf8",
                 "mfma_mxfp6_e2m3", "mfma_mxfp6_e3m2", "mfma_mxfp4", "smfmac_fp16", "smfmac_bf16", "smfmac_fp8",
                 "smfmac_bf8", "smfmac_int8", "rocblas-fp", "rocblas-int", "hipblaslt-fp8"):
        assert test in tests_covered, test
    assert {"global_memory_bandwidth float", "global_memory_bandwidth float2", "global_memory_bandwidth float4",
            "hipblaslt-fp8 fp8_e4m3", "hipblaslt-fp8 mxf4_e2m1"} <= set(port)
    assert all(v["MT"] > 0 and v["ST"] > 0 for v in port.values())
