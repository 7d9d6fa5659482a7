"""ctypes binding of oracle/liboracle.so -- the CPU oracle (test infrastructure).

Import this only from tests/, from __graft_entry__.smoke() and from the cpu_baseline
leg of bench.py.  The product never does.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")

FMT_F16, FMT_BF16, FMT_E4M3, FMT_E5M2, FMT_E2M3, FMT_E3M2, FMT_E2M1 = range(7)

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} not found: build it with `make -C oracle`")
        L = C.CDLL(LIB_PATH)
        vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
        L.orc_rng_word.argtypes = [u64, u32, u64]; L.orc_rng_word.restype = u64
        L.orc_u01.argtypes = [u64, u32, u64]; L.orc_u01.restype = C.c_float
        L.orc_upm1.argtypes = [u64, u32, u64]; L.orc_upm1.restype = C.c_float
        L.orc_below.argtypes = [u64, u32, u64, u32]; L.orc_below.restype = u32
        L.orc_normal.argtypes = [u64, u32, u64]; L.orc_normal.restype = C.c_double
        L.orc_fill_f32.argtypes = [vp, u64, u64, u32, i32, u64]; L.orc_fill_f32.restype = None
        L.orc_decode.argtypes = [i32, u32]; L.orc_decode.restype = C.c_double
        L.orc_encode.argtypes = [i32, C.c_double]; L.orc_encode.restype = u32
        L.orc_e8m0.argtypes = [u32]; L.orc_e8m0.restype = C.c_double
        L.orc_global_bandwidth.argtypes = [i32, vp, u64, u64, vp]; L.orc_global_bandwidth.restype = None
        L.orc_global_bandwidth_thread.argtypes = [i32, u64, u32, u64, u64, u64]
        L.orc_global_bandwidth_thread.restype = C.c_float
        L.orc_sum_u01.argtypes = [u64, u32, u64]; L.orc_sum_u01.restype = C.c_double
        L.orc_compute_mad.argtypes = [i32, i32, u64, u64, u64, u32, vp]; L.orc_compute_mad.restype = i32
        L.orc_mfma_dense.argtypes = [i32, vp, vp, vp, vp, vp, vp, u32, u32]; L.orc_mfma_dense.restype = i32
        L.orc_smfmac.argtypes = [i32, vp, vp, vp, vp, vp, u32, u32]; L.orc_smfmac.restype = i32
        L.orc_gemm_tile.argtypes = [i32, vp, vp, u32, u32, u32, u32, u32, u32, u32, C.c_double, vp]
        L.orc_gemm_tile.restype = i32
        _lib = L
    return _lib


def rng_word(seed, stream, i):
    return lib().orc_rng_word(seed, stream, i)


def fill_f32(n, seed, stream, dist, first=0):
    out = np.empty(n, dtype=np.float32)
    lib().orc_fill_f32(out.ctypes.data, n, seed, stream, dist, first)
    return out


def normal(n, seed, stream, first=0):
    L = lib()
    return np.array([L.orc_normal(seed, stream, first + i) for i in range(n)], dtype=np.float64)


def decode(fmt, codes):
    L = lib()
    return np.array([L.orc_decode(fmt, int(c)) for c in np.asarray(codes).ravel()], dtype=np.float64).reshape(np.shape(codes))


def encode(fmt, values):
    L = lib()
    return np.array([L.orc_encode(fmt, float(v)) for v in np.asarray(values).ravel()], dtype=np.uint32).reshape(np.shape(values))


def global_bandwidth(width, data, T):
    data = np.ascontiguousarray(data, dtype=np.float32)
    out = np.empty(T, dtype=np.float32)
    lib().orc_global_bandwidth(width, data.ctypes.data, data.size, T, out.ctypes.data)
    return out


def global_bandwidth_thread(width, seed, stream, n_floats, T, t):
    return lib().orc_global_bandwidth_thread(width, seed, stream, n_floats, T, t)


def sum_u01(seed, stream, n):
    return lib().orc_sum_u01(seed, stream, n)


_MAD_OUT = {0: np.float32, 1: np.uint16, 2: np.float64, 3: np.float32, 4: np.float32, 5: np.uint32, 6: np.int32}


def compute_mad(kind, width, seed, first, n, steps):
    out = np.empty(n, dtype=_MAD_OUT[kind])
    rc = lib().orc_compute_mad(kind, width, seed, first, n, steps, out.ctypes.data)
    assert rc == 0, rc
    return out


def mfma_dense(kind, A, B, scaleA, scaleB, waves, iters, out_elems, is_int=False):
    """Returns (out[waves*4*out_elems], abs_scale) -- abs_scale = iters * sum|a*b| per element."""
    out = np.empty(waves * 4 * out_elems, dtype=np.int32 if is_int else np.float32)
    ab = np.empty(waves * 4 * out_elems, dtype=np.float64)
    A = np.ascontiguousarray(A); B = np.ascontiguousarray(B)
    sa = np.ascontiguousarray(scaleA) if scaleA is not None else None
    sb = np.ascontiguousarray(scaleB) if scaleB is not None else None
    rc = lib().orc_mfma_dense(kind, A.ctypes.data, B.ctypes.data, sa.ctypes.data if sa is not None else None,
                              sb.ctypes.data if sb is not None else None, out.ctypes.data, ab.ctypes.data, waves, iters)
    assert rc == 0, rc
    return out, ab


def smfmac(kind, Ac, meta, B, waves, iters, is_int=False):
    out = np.empty(waves * 4 * 256, dtype=np.int32 if is_int else np.float32)
    ab = np.empty(waves * 4 * 256, dtype=np.float64)
    Ac = np.ascontiguousarray(Ac); meta = np.ascontiguousarray(meta, dtype=np.uint8); B = np.ascontiguousarray(B)
    rc = lib().orc_smfmac(kind, Ac.ctypes.data, meta.ctypes.data, B.ctypes.data, out.ctypes.data, ab.ctypes.data, waves, iters)
    assert rc == 0, rc
    return out, ab


def gemm_tile(fmt, A, B, K, lda, ldb, m0, n0, tm, tn, scale=1.0):
    out = np.empty((tm, tn), dtype=np.float64)
    rc = lib().orc_gemm_tile(fmt, A.ctypes.data, B.ctypes.data, K, lda, ldb, m0, n0, tm, tn, scale, out.ctypes.data)
    assert rc == 0, rc
    return out


def gemm_tile2(fmt_a, fmt_b, A, B, K, lda, ldb, m0, n0, tm, tn, scale=1.0):
    """fmt: FMT_F16 / FMT_BF16 / FMT_E4M3 / FMT_E5M2, FMT_I8, FMT_F32 or FMT_F64; A and B may differ."""
    out = np.empty((tm, tn), dtype=np.float64)
    L = lib()
    L.orc_gemm_tile2.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p] + [C.c_uint32] * 7 + [C.c_double, C.c_void_p]
    L.orc_gemm_tile2.restype = C.c_int
    rc = L.orc_gemm_tile2(fmt_a, fmt_b, A.ctypes.data, B.ctypes.data, K, lda, ldb, m0, n0, tm, tn, scale, out.ctypes.data)
    assert rc == 0, rc
    return out


FMT_I8 = 7
FMT_F32 = 8
FMT_F64 = 9


def gemm_mx_tile(A, B, SA, SB, K, m0, n0, tm, tn):
    out = np.empty((tm, tn), dtype=np.float64)
    L = lib()
    L.orc_gemm_mx_tile.argtypes = [C.c_void_p] * 4 + [C.c_uint32] * 5 + [C.c_void_p]
    L.orc_gemm_mx_tile.restype = C.c_int
    rc = L.orc_gemm_mx_tile(A.ctypes.data, B.ctypes.data, SA.ctypes.data, SB.ctypes.data, K, m0, n0, tm, tn, out.ctypes.data)
    assert rc == 0, rc
    return out


def fill_bytes(n, seed, stream, lo, span, first=0):
    out = np.empty(n, dtype=np.uint8)
    L = lib()
    L.orc_fill_bytes.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64]
    L.orc_fill_bytes.restype = None
    L.orc_fill_bytes(out.ctypes.data, n, seed, stream, lo, span, first)
    return out


def fill_fmt(fmt, n, seed, stream, dist, scale=1.0, first=0):
    out = np.empty(n, dtype=np.uint16 if fmt <= FMT_BF16 else np.uint8)
    L = lib()
    L.orc_fill_fmt.argtypes = [C.c_int, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint32, C.c_int, C.c_float, C.c_uint64]
    L.orc_fill_fmt.restype = None
    L.orc_fill_fmt(fmt, out.ctypes.data, n, seed, stream, dist, scale, first)
    return out


def _bind_builders():
    L = lib()
    if getattr(L, "_builders_bound", False):
        return L
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
    L.orc_fill_normal_codes.argtypes = [i32, C.c_double, u64, u32, u64, u64, vp]; L.orc_fill_normal_codes.restype = None
    L.orc_fill_int8.argtypes = [u64, u32, u64, u64, vp]; L.orc_fill_int8.restype = None
    L.orc_fill_e8m0.argtypes = [u64, u32, u64, u64, vp]; L.orc_fill_e8m0.restype = None
    L.orc_fill_sparse_meta.argtypes = [u64, u32, u64, u64, vp]; L.orc_fill_sparse_meta.restype = None
    L.orc_pack_bits.argtypes = [vp, u64, i32, vp]; L.orc_pack_bits.restype = None
    L.orc_fill_bf16.argtypes = [vp, u64, u64, u32, i32, u64]; L.orc_fill_bf16.restype = None
    L.orc_fill_e4m3.argtypes = [vp, u64, u64, u32, i32, C.c_float, u64]; L.orc_fill_e4m3.restype = None
    L._builders_bound = True
    return L


def fill_normal_codes(fmt, sigma, seed, stream, n, first=0):
    out = np.empty(n, dtype=np.uint16 if fmt <= FMT_BF16 else np.uint8)
    _bind_builders().orc_fill_normal_codes(fmt, sigma, seed, stream, first, n, out.ctypes.data)
    return out


def fill_int8(seed, stream, n, first=0):
    out = np.empty(n, dtype=np.int8)
    _bind_builders().orc_fill_int8(seed, stream, first, n, out.ctypes.data)
    return out


def fill_e8m0(seed, stream, n, first=0):
    out = np.empty(n, dtype=np.uint8)
    _bind_builders().orc_fill_e8m0(seed, stream, first, n, out.ctypes.data)
    return out


def fill_sparse_meta(seed, stream, n, first=0):
    out = np.empty(n, dtype=np.uint8)
    _bind_builders().orc_fill_sparse_meta(seed, stream, first, n, out.ctypes.data)
    return out


def pack_bits(codes, bits):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty((codes.size * bits + 7) // 8, dtype=np.uint8)
    _bind_builders().orc_pack_bits(codes.ctypes.data, codes.size, bits, out.ctypes.data)
    return out


def fill_bf16(n, seed, stream, dist, first=0):
    out = np.empty(n, dtype=np.uint16)
    _bind_builders().orc_fill_bf16(out.ctypes.data, n, seed, stream, dist, first)
    return out


def fill_e4m3(n, seed, stream, dist, scale, first=0):
    out = np.empty(n, dtype=np.uint8)
    _bind_builders().orc_fill_e4m3(out.ctypes.data, n, seed, stream, dist, scale, first)
    return out


def global_bandwidth_range(width, data, T, t0, t1, out=None):
    data = np.ascontiguousarray(data, dtype=np.float32)
    if out is None:
        out = np.zeros(T, dtype=np.float32)
    L = lib()
    L.orc_global_bandwidth_range.argtypes = [C.c_int, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_void_p]
    L.orc_global_bandwidth_range.restype = None
    L.orc_global_bandwidth_range(width, data.ctypes.data, data.size, T, t0, t1, out.ctypes.data)
    return out


def local_bandwidth(width, blocks, block_size, reps):
    out = np.empty(blocks * block_size, dtype=np.float32)
    L = lib()
    L.orc_local_bandwidth.argtypes = [C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]
    L.orc_local_bandwidth.restype = None
    L.orc_local_bandwidth(width, blocks, block_size, reps, out.ctypes.data)
    return out


# --- CPU baseline harness (cpu_harness.c) -----------------------------------------------------------
CPUH_READ_FLOAT4, CPUH_MAD_F32, CPUH_MFMA_BF16, CPUH_MFMA_I8, CPUH_GEMM_BF16 = range(5)


class CpuhResult(C.Structure):
    _fields_ = [("us_st", C.c_double), ("us_mt", C.c_double), ("iters_st", C.c_uint), ("iters_mt", C.c_uint),
                ("threads_mt", C.c_int), ("pinned", C.c_int), ("units_per_iter_st", C.c_double),
                ("units_per_iter_mt", C.c_double), ("giga_st", C.c_double), ("giga_mt", C.c_double)]


class CpuhOp(C.Structure):
    _fields_ = [("op", C.c_int), ("kind", C.c_int), ("width", C.c_int), ("seed", C.c_uint64),
                ("p0", C.c_void_p), ("p1", C.c_void_p), ("p2", C.c_void_p), ("p3", C.c_void_p),
                ("K", C.c_uint32), ("tile", C.c_uint32), ("scale", C.c_double), ("n_floats", C.c_uint64), ("T", C.c_uint64)]


OP_MAD, OP_MFMA, OP_SMFMAC, OP_GEMM, OP_GEMM_MX, OP_READ = range(6)
OP_MAD_ITEMS = 8


def _bind_harness():
    L = lib()
    if getattr(L, "_harness_bound", False):
        return L
    vp, u64, u32, i32, dbl = C.c_void_p, C.c_uint64, C.c_uint, C.c_int, C.c_double
    L.cpuh_pool_create.argtypes = [i32]; L.cpuh_pool_create.restype = vp
    L.cpuh_pool_destroy.argtypes = [vp]; L.cpuh_pool_destroy.restype = None
    L.cpuh_pool_max_threads.argtypes = [vp]; L.cpuh_pool_max_threads.restype = i32
    L.cpuh_pool_pinned_cpu.argtypes = [vp, i32]; L.cpuh_pool_pinned_cpu.restype = i32
    L.cpuh_pool_count.argtypes = [vp, i32, u64, vp]; L.cpuh_pool_count.restype = None
    L.cpuh_pick_iters.argtypes = [dbl, u32, u32, u32]; L.cpuh_pick_iters.restype = u32
    L.cpuh_time_sleep_body.argtypes = [vp, i32, u32, u32, C.POINTER(u32)]; L.cpuh_time_sleep_body.restype = dbl
    L.cpuh_measure.argtypes = [vp, i32, u64, u32, u32, C.POINTER(CpuhResult)]; L.cpuh_measure.restype = i32
    L.cpuh_measure_op.argtypes = [vp, C.POINTER(CpuhOp), dbl, dbl, u32, u32, C.POINTER(CpuhResult)]; L.cpuh_measure_op.restype = i32
    L.cpuh_measure_chain_fn.argtypes = [vp, vp, dbl, u32, u32, C.POINTER(CpuhResult)]; L.cpuh_measure_chain_fn.restype = i32
    L.cpuh_measure_read_fn.argtypes = [vp, vp, vp, u64, u32, u32, C.POINTER(CpuhResult)]; L.cpuh_measure_read_fn.restype = i32
    L.cpuh_measure_stream.argtypes = [vp, vp, u64, i32, u32, u32, C.POINTER(CpuhResult), vp]; L.cpuh_measure_stream.restype = i32
    L._harness_bound = True
    return L


class CpuPool:
    """Persistent pinned worker pool of the CPU baseline harness."""

    def __init__(self, max_threads=None):
        self.L = _bind_harness()
        self.max_threads = max_threads or len(os.sched_getaffinity(0))
        self.h = self.L.cpuh_pool_create(self.max_threads)
        if not self.h:
            raise MemoryError("cpuh_pool_create failed")

    def close(self):
        if self.h:
            self.L.cpuh_pool_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def pinned_cpu(self, tid):
        return self.L.cpuh_pool_pinned_cpu(self.h, tid)

    def count(self, n, iters):
        counts = np.zeros(self.max_threads, dtype=np.uint64)
        self.L.cpuh_pool_count(self.h, n, iters, counts.ctypes.data)
        return counts

    def time_sleep_body(self, n_threads, sleep_us, target_us):
        iters = C.c_uint(0)
        us = self.L.cpuh_time_sleep_body(self.h, n_threads, sleep_us, target_us, C.byref(iters))
        return us, iters.value

    def measure(self, kind, seed, warmup=2, target_us=2_000_000):
        r = CpuhResult()
        rc = self.L.cpuh_measure(self.h, kind, seed, warmup, target_us, C.byref(r))
        if rc != 0:
            raise RuntimeError(f"cpuh_measure({kind}) failed: {rc}")
        return r


    def measure_op(self, op, units_st, units_mt=None, warmup=2, target_us=1_000_000, keep=()):
        """Times one oracle kernel (a CpuhOp descriptor) at 1 thread and at every worker; `keep` holds the numpy
        operands alive for the duration of the call."""
        r = CpuhResult()
        rc = self.L.cpuh_measure_op(self.h, C.byref(op), units_st, units_st if units_mt is None else units_mt, warmup,
                                    target_us, C.byref(r))
        if rc != 0:
            raise RuntimeError(f"cpuh_measure_op({op.op}, {op.kind}) failed: {rc}")
        return r

    def measure_chain_fn(self, fn_ptr, ops_per_iter, warmup=2, target_us=2_000_000):
        """Times a `double fn(uint64_t outer)` chain given as a raw function pointer."""
        r = CpuhResult()
        rc = self.L.cpuh_measure_chain_fn(self.h, fn_ptr, ops_per_iter, warmup, target_us, C.byref(r))
        if rc != 0:
            raise RuntimeError(f"cpuh_measure_chain_fn failed: {rc}")
        return r

    def measure_read_fn(self, read_ptr, populate_ptr, n_floats, warmup=2, target_us=2_000_000):
        """Times a `uint64_t fn(const float*, size_t, uint64_t iters)` streaming read over a shared array."""
        r = CpuhResult()
        rc = self.L.cpuh_measure_read_fn(self.h, read_ptr, populate_ptr, n_floats, warmup, target_us, C.byref(r))
        if rc != 0:
            raise RuntimeError(f"cpuh_measure_read_fn failed: {rc}")
        return r


    def own_populate_ptr(self):
        """Address of the harness's restatement of the reference's populate()."""
        return C.cast(self.L.cpuh_populate, C.c_void_p).value

    def measure_stream(self, populate_ptr, n_floats, kind, warmup=2, target_us=2_000_000):
        """The reference's DRAM `copy` (kind 0) / `triad` (kind 1) rows over three shared arrays, all workers.
        Returns (result, probe) with probe = a[0], a[n/2], a[n-1], b[n/2], c[n/2] after the run."""
        r = CpuhResult()
        probe = np.zeros(5, dtype=np.float32)
        rc = self.L.cpuh_measure_stream(self.h, populate_ptr, n_floats, kind, warmup, target_us, C.byref(r), probe.ctypes.data)
        if rc != 0:
            raise RuntimeError(f"cpuh_measure_stream failed: {rc}")
        return r, probe


REF_LIB_PATH = os.path.join(_HERE, "_ref", "libclpeak_ref.so")


def reference_kernels():
    """The reference's own CPU kernels (built by ref.mk where its checkout is present), for the widest ISA
    this host runs: dict(isa, fp32_fn, fp32_ops, read_fn, populate_fn), or None when the build is absent."""
    if not os.path.exists(REF_LIB_PATH):
        return None
    flags = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    flags = line
                    break
    except OSError:
        return None
    have = set(flags.split())
    if {"avx512f", "avx512bw", "avx512vl", "avx512dq"} <= have:
        isa, name = 1, "AVX-512"
    elif {"avx2", "fma", "f16c"} <= have:
        isa, name = 0, "AVX2+FMA"
    else:
        return None
    R = C.CDLL(REF_LIB_PATH)
    R.ref_fp32_chain_fn.argtypes = [C.c_int]; R.ref_fp32_chain_fn.restype = C.c_void_p
    R.ref_fp32_chain_ops.argtypes = [C.c_int]; R.ref_fp32_chain_ops.restype = C.c_double
    R.ref_readsum_fn.argtypes = [C.c_int]; R.ref_readsum_fn.restype = C.c_void_p
    return {"isa": name, "lib": R, "fp32_fn": R.ref_fp32_chain_fn(isa), "fp32_ops": R.ref_fp32_chain_ops(isa),
            "read_fn": R.ref_readsum_fn(isa), "populate_fn": C.cast(R.ref_populate, C.c_void_p).value}


def pick_iters(per_iter_us, target_us, forced, max_iters):
    return _bind_harness().cpuh_pick_iters(per_iter_us, target_us, forced, max_iters)
