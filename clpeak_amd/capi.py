"""ctypes binding of include/clpeak_mi355.h.

Loads ``clpeak_amd/libclpeak_mi355.so`` (built by ``clpeak_amd/csrc/Makefile``).  There
is no fallback: a missing library or a missing symbol is an ImportError / AttributeError
at load time, and every non-zero status from the library raises :class:`Mi355Error`.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libclpeak_mi355.so")

# Every symbol include/clpeak_mi355.h declares.  tests/test_abi.py checks this list
# against the header text and against the built library.
SYMBOLS = [
    "mi355_device_count", "mi355_open", "mi355_close", "mi355_get_props", "mi355_last_error",
    "mi355_alloc", "mi355_free", "mi355_upload", "mi355_download", "mi355_memset", "mi355_sync",
    "mi355_timer_start", "mi355_timer_stop",
    "mi355_fill_f32", "mi355_fill_bf16", "mi355_fill_fp8_e4m3", "mi355_copy",
    "mi355_global_bandwidth", "mi355_compute_mad", "mi355_launch_roundtrip",
    "mi355_mfma_dense", "mi355_smfmac", "mi355_mfma_raw",
    "mi355_gemm_bf16", "mi355_gemm_fp8_e4m3",
    "mi355_local_bandwidth", "mi355_host_alloc", "mi355_host_free", "mi355_copy_async",
    "mi355_fill_f16", "mi355_fill_fp8_e5m2", "mi355_fill_i8", "mi355_gemm_f16", "mi355_gemm_i8", "mi355_gemm_fp8_e5m2",
    "mi355_gemm_f32", "mi355_gemm_f64", "mi355_fill_f64",
    "mi355_gemm_mxfp4", "mi355_gemm_mxfp4_static", "mi355_fill_bytes",
    "mi355_gemm_mxfp4_prepare_scales", "mi355_gemm_mxfp4_prepared", "mi355_scratch_bytes", "mi355_gemm_tiling",
]

OK, ERR_ARG, ERR_HIP, ERR_NODEV, ERR_ARCH, ERR_OOM = 0, -1, -2, -3, -4, -5
DIST_U01, DIST_UPM1 = 0, 1
H2D, D2H = 0, 1
MAD_F32, MAD_F16, MAD_F64, MAD_MP, MAD_BF16, MAD_I32, MAD_I8DP = range(7)
(MFMA_F16_16x16x32, MFMA_BF16_16x16x32, MFMA_F16_32x32x16, MFMA_BF16_32x32x16, MFMA_I8_16x16x64,
 MFMA_FP8_16x16x128, MFMA_BF8_16x16x128, MFMA_MXFP6_E2M3, MFMA_MXFP6_E3M2, MFMA_MXFP4_E2M1) = range(10)
SMFMAC_F16_16x16x64, SMFMAC_BF16_16x16x64, SMFMAC_FP8_16x16x128, SMFMAC_BF8_16x16x128, SMFMAC_I8_16x16x128 = range(5)
GEMM_TILING_AUTO, GEMM_TILING_256, GEMM_TILING_128 = 0, 1, 2
MATRIX_ON_HALF_THE_CUS = 0x200   # diagnosis: only the workgroups of the first 16 CUs of every XCD take part
MFMA_ONE_OPERAND_SET = 0x100   # OR into an MFMA / SMFMAC kind: every chain of a wave takes chain 0's operands

# Stream ids of the seeded generator (clpeak_amd/csrc/seeded_rng.h).
STREAM_BW, STREAM_MAD, STREAM_MFMA_A, STREAM_MFMA_B, STREAM_SCALE_A, STREAM_SCALE_B, \
    STREAM_SPARSE, STREAM_GEMM_A, STREAM_GEMM_B, STREAM_MAD_Y = range(10)


class Mi355Error(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"mi355 error {code}: {message}")
        self.code = code


class Props(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("driver_version", C.c_char * 32),
                ("runtime_version", C.c_char * 32), ("num_cus", C.c_int32), ("wave_size", C.c_int32),
                ("max_threads_per_block", C.c_int32), ("clock_khz", C.c_int32), ("total_mem", C.c_uint64)]


def load_library(path=LIB_PATH):
    if not os.path.exists(path):
        raise ImportError(f"{path} not found: build it with `make -C clpeak_amd/csrc` "
                          "(or __graft_entry__.build()); there is no CPU fallback")
    lib = C.CDLL(path)
    for name in SYMBOLS:
        getattr(lib, name)  # AttributeError if the library lacks a declared entry point
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
    lib.mi355_device_count.argtypes = [C.POINTER(C.c_int)]
    lib.mi355_open.argtypes = [C.c_int, C.POINTER(vp)]
    lib.mi355_close.argtypes = [vp]
    lib.mi355_get_props.argtypes = [vp, C.POINTER(Props)]
    lib.mi355_last_error.argtypes = [vp]
    lib.mi355_last_error.restype = C.c_char_p
    lib.mi355_alloc.argtypes = [vp, C.c_size_t, C.POINTER(vp)]
    lib.mi355_free.argtypes = [vp, vp]
    lib.mi355_upload.argtypes = [vp, vp, vp, C.c_size_t]
    lib.mi355_download.argtypes = [vp, vp, vp, C.c_size_t]
    lib.mi355_memset.argtypes = [vp, vp, C.c_int, C.c_size_t]
    lib.mi355_sync.argtypes = [vp]
    lib.mi355_timer_start.argtypes = [vp]
    lib.mi355_timer_stop.argtypes = [vp, C.POINTER(C.c_float)]
    lib.mi355_fill_f32.argtypes = [vp, vp, u64, u64, u32, i32]
    lib.mi355_fill_bf16.argtypes = [vp, vp, u64, u64, u32, i32]
    lib.mi355_fill_fp8_e4m3.argtypes = [vp, vp, u64, u64, u32, i32, C.c_float]
    lib.mi355_copy.argtypes = [vp, vp, vp, C.c_size_t]
    lib.mi355_global_bandwidth.argtypes = [vp, i32, vp, u64, vp, u32, u32]
    lib.mi355_compute_mad.argtypes = [vp, i32, i32, u64, u64, u32, vp, u32]
    lib.mi355_launch_roundtrip.argtypes = [vp, u32, u32, C.POINTER(C.c_double)]
    lib.mi355_mfma_dense.argtypes = [vp, i32, vp, vp, vp, vp, vp, u32, u32, vp]
    lib.mi355_smfmac.argtypes = [vp, i32, vp, vp, vp, vp, u32, u32, vp]
    lib.mi355_mfma_raw.argtypes = [vp, i32, i32, vp, vp, vp, vp, vp, i32, i32, vp]
    lib.mi355_gemm_bf16.argtypes = [vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_fp8_e4m3.argtypes = [vp, vp, vp, vp, u32, u32, u32, C.c_float, C.c_float]
    lib.mi355_local_bandwidth.argtypes = [vp, i32, vp, u32, u32, u32]
    lib.mi355_fill_f16.argtypes = [vp, vp, u64, u64, u32, i32]
    lib.mi355_fill_fp8_e5m2.argtypes = [vp, vp, u64, u64, u32, i32, C.c_float]
    lib.mi355_fill_i8.argtypes = [vp, vp, u64, u64, u32]
    lib.mi355_gemm_f16.argtypes = [vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_tiling.argtypes = [vp, C.c_int]
    lib.mi355_gemm_i8.argtypes = [vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_f32.argtypes = [vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_f64.argtypes = [vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_fill_f64.argtypes = [vp, vp, u64, u64, u32, i32]
    lib.mi355_gemm_fp8_e5m2.argtypes = [vp, vp, vp, vp, u32, u32, u32, C.c_float, C.c_float]
    lib.mi355_gemm_mxfp4.argtypes = [vp, vp, vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_mxfp4_static.argtypes = [vp, vp, vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_gemm_mxfp4_prepare_scales.argtypes = [vp, vp, vp, u32, u32, u32, vp]
    lib.mi355_gemm_mxfp4_prepared.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32]
    lib.mi355_scratch_bytes.argtypes = [vp, C.POINTER(C.c_size_t)]
    lib.mi355_fill_bytes.argtypes = [vp, vp, u64, u64, u32, u32, u32]
    lib.mi355_host_alloc.argtypes = [vp, C.c_size_t, C.POINTER(vp)]
    lib.mi355_host_free.argtypes = [vp, vp]
    lib.mi355_copy_async.argtypes = [vp, vp, vp, C.c_size_t, i32]
    for name in SYMBOLS:
        if name != "mi355_last_error":
            getattr(lib, name).restype = C.c_int
    return lib


class DeviceBuffer:
    """A device allocation owned by a :class:`Device`."""

    def __init__(self, dev, nbytes):
        self.dev, self.nbytes = dev, int(nbytes)
        p = C.c_void_p()
        dev._check(dev.lib.mi355_alloc(dev.h, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, array):
        import numpy as np
        a = np.ascontiguousarray(array)
        assert a.nbytes <= self.nbytes, (a.nbytes, self.nbytes)
        self.dev._check(self.dev.lib.mi355_upload(self.dev.h, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count=None, offset_bytes=0):
        import numpy as np
        dt = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset_bytes) // dt.itemsize
        out = np.empty(count, dtype=dt)
        assert offset_bytes + out.nbytes <= self.nbytes
        self.dev._check(self.dev.lib.mi355_download(self.dev.h, out.ctypes.data, self.ptr + offset_bytes, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.dev._check(self.dev.lib.mi355_free(self.dev.h, self.ptr))
            self.ptr = None


class Device:
    """One opened GPU: thin, one-to-one wrappers over the C entry points."""

    def __init__(self, ordinal=0, lib=None):
        self.lib = lib or load_library()
        h = C.c_void_p()
        rc = self.lib.mi355_open(ordinal, C.byref(h))
        if rc != OK:
            raise Mi355Error(rc, (self.lib.mi355_last_error(None) or b"").decode())
        self.h = h
        p = Props()
        self._check(self.lib.mi355_get_props(self.h, C.byref(p)))
        self.props = p

    def _check(self, rc):
        if rc != OK:
            raise Mi355Error(rc, (self.lib.mi355_last_error(self.h) or b"").decode())

    def close(self):
        if self.h:
            self.lib.mi355_close(self.h)
            self.h = None

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def from_host(self, array):
        import numpy as np
        a = np.ascontiguousarray(array)
        return DeviceBuffer(self, max(a.nbytes, 1)).upload(a)

    def memset(self, buf, byte, nbytes=None):
        self._check(self.lib.mi355_memset(self.h, buf.ptr, byte, buf.nbytes if nbytes is None else nbytes))

    def sync(self):
        self._check(self.lib.mi355_sync(self.h))

    def timer_start(self):
        self._check(self.lib.mi355_timer_start(self.h))

    def timer_stop(self):
        us = C.c_float()
        self._check(self.lib.mi355_timer_stop(self.h, C.byref(us)))
        return us.value

    def time_launches(self, launch, n):
        """Elapsed microseconds (HIP events on the handle's stream) of n back-to-back launches."""
        self.timer_start()
        for _ in range(n):
            launch()
        return self.timer_stop()

    # --- one wrapper per kernel entry point -------------------------------------------
    def fill_f32(self, buf, n, seed, stream, dist):
        self._check(self.lib.mi355_fill_f32(self.h, buf.ptr, n, seed, stream, dist))

    def fill_bf16(self, buf, n, seed, stream, dist):
        self._check(self.lib.mi355_fill_bf16(self.h, buf.ptr, n, seed, stream, dist))

    def fill_fp8_e4m3(self, buf, n, seed, stream, dist, scale):
        self._check(self.lib.mi355_fill_fp8_e4m3(self.h, buf.ptr, n, seed, stream, dist, scale))

    def fill_f16(self, buf, n, seed, stream, dist):
        self._check(self.lib.mi355_fill_f16(self.h, buf.ptr, n, seed, stream, dist))

    def fill_fp8_e5m2(self, buf, n, seed, stream, dist, scale):
        self._check(self.lib.mi355_fill_fp8_e5m2(self.h, buf.ptr, n, seed, stream, dist, scale))

    def fill_i8(self, buf, n, seed, stream):
        self._check(self.lib.mi355_fill_i8(self.h, buf.ptr, n, seed, stream))

    def copy(self, dst, src, nbytes):
        self._check(self.lib.mi355_copy(self.h, dst.ptr, src.ptr, nbytes))

    def global_bandwidth(self, width, inbuf, n_floats, outbuf, blocks, block_size=256):
        self._check(self.lib.mi355_global_bandwidth(self.h, width, inbuf.ptr, n_floats, outbuf.ptr, blocks, block_size))

    def compute_mad(self, kind, width, seed, n_items, steps, outbuf, block_size=256):
        self._check(self.lib.mi355_compute_mad(self.h, kind, width, seed, n_items, steps, outbuf.ptr, block_size))

    def local_bandwidth(self, width, outbuf, blocks, block_size=256, reps=64):
        self._check(self.lib.mi355_local_bandwidth(self.h, width, outbuf.ptr, blocks, block_size, reps))

    def host_alloc(self, nbytes):
        """Pinned host buffer as a numpy uint8 array (free it with host_free)."""
        import numpy as np
        p = C.c_void_p()
        self._check(self.lib.mi355_host_alloc(self.h, nbytes, C.byref(p)))
        arr = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(nbytes,))
        return arr, p

    def host_free(self, handle):
        self._check(self.lib.mi355_host_free(self.h, handle))

    def copy_async(self, dst_ptr, src_ptr, nbytes, direction):
        self._check(self.lib.mi355_copy_async(self.h, dst_ptr, src_ptr, nbytes, direction))

    def launch_roundtrip(self, warmup, launches):
        us = C.c_double()
        self._check(self.lib.mi355_launch_roundtrip(self.h, warmup, launches, C.byref(us)))
        return us.value

    @staticmethod
    def _subset(on_xcds, half_cus):
        """The diagnosis bits of a matrix kind: on_xcds = iterable of XCD numbers that take part (None: all)."""
        bits = MATRIX_ON_HALF_THE_CUS if half_cus else 0
        if on_xcds is not None:
            bits |= (sum(1 << x for x in on_xcds) & 0xff) << 16
        return bits

    def mfma_dense(self, kind, A, B, scaleA, scaleB, out, waves, iters, clocks=None, one_set=False, on_xcds=None, half_cus=False):
        kind |= (MFMA_ONE_OPERAND_SET if one_set else 0) | self._subset(on_xcds, half_cus)
        self._check(self.lib.mi355_mfma_dense(self.h, kind, A.ptr, B.ptr, scaleA.ptr if scaleA else None,
                                              scaleB.ptr if scaleB else None, out.ptr, waves, iters,
                                              clocks.ptr if clocks else None))

    def smfmac(self, kind, Ac, meta, B, out, waves, iters, clocks=None, one_set=False, on_xcds=None, half_cus=False):
        kind |= (MFMA_ONE_OPERAND_SET if one_set else 0) | self._subset(on_xcds, half_cus)
        self._check(self.lib.mi355_smfmac(self.h, kind, Ac.ptr, meta.ptr, B.ptr, out.ptr, waves, iters,
                                          clocks.ptr if clocks else None))

    def mfma_raw(self, sparse, kind, a, b, c, aux0, aux1, sel0, sel1, d):
        self._check(self.lib.mi355_mfma_raw(self.h, int(sparse), kind, a.ptr, b.ptr, c.ptr, aux0.ptr, aux1.ptr,
                                            sel0, sel1, d.ptr))

    def gemm_tiling(self, tiling):
        """GEMM_TILING_AUTO / _256 / _128 for the 8- and 16-bit GEMM calls of this handle."""
        self._check(self.lib.mi355_gemm_tiling(self.h, tiling))

    def gemm_bf16(self, A, B, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_bf16(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K))

    def gemm_mxfp4(self, A, B, SA, SB, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_mxfp4(self.h, A.ptr, B.ptr, SA.ptr, SB.ptr, Cbuf.ptr, M, N, K))

    def gemm_mxfp4_static(self, A, B, SA, SB, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_mxfp4_static(self.h, A.ptr, B.ptr, SA.ptr, SB.ptr, Cbuf.ptr, M, N, K))

    def gemm_mxfp4_prepare_scales(self, SA, SB, M, N, K, prepared):
        self._check(self.lib.mi355_gemm_mxfp4_prepare_scales(self.h, SA.ptr, SB.ptr, M, N, K, prepared.ptr))

    def gemm_mxfp4_prepared(self, A, B, prepared, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_mxfp4_prepared(self.h, A.ptr, B.ptr, prepared.ptr, Cbuf.ptr, M, N, K))

    def scratch_bytes(self):
        n = C.c_size_t()
        self._check(self.lib.mi355_scratch_bytes(self.h, C.byref(n)))
        return n.value

    def fill_bytes(self, buf, n, seed, stream, lo, span):
        self._check(self.lib.mi355_fill_bytes(self.h, buf.ptr, n, seed, stream, lo, span))

    def gemm_f16(self, A, B, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_f16(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K))

    def gemm_i8(self, A, B, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_i8(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K))

    def gemm_f32(self, A, B, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_f32(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K))

    def gemm_f64(self, A, B, Cbuf, M, N, K):
        self._check(self.lib.mi355_gemm_f64(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K))

    def fill_f64(self, buf, n, seed, stream, dist):
        self._check(self.lib.mi355_fill_f64(self.h, buf.ptr, n, seed, stream, dist))

    def gemm_fp8_e5m2(self, A, B, Cbuf, M, N, K, scale_a, scale_b):
        self._check(self.lib.mi355_gemm_fp8_e5m2(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K, scale_a, scale_b))

    def gemm_fp8_e4m3(self, A, B, Cbuf, M, N, K, scale_a, scale_b):
        self._check(self.lib.mi355_gemm_fp8_e4m3(self.h, A.ptr, B.ptr, Cbuf.ptr, M, N, K, scale_a, scale_b))
