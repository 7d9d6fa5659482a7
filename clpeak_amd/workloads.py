"""Shapes and seeded operands of the matrix workloads, as the backend itself builds them.

The operand bytes come from the host layer's own generator (``clpeak_amd/host/seeded_inputs.cpp``,
reached through ``libclpeak_host.so``): the same bytes ``Mi355Peak`` uploads before it times an MFMA or
SMFMAC row.  Nothing here computes a result; the kernels are reached through ``clpeak_amd.capi``.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libclpeak_host.so")

# stream ids of the counter generator (clpeak_amd/csrc/seeded_rng.h)
STREAM_BW, STREAM_MAD, STREAM_MFMA_A, STREAM_MFMA_B, STREAM_SCALE_A, STREAM_SCALE_B, \
    STREAM_SPARSE, STREAM_GEMM_A, STREAM_GEMM_B, STREAM_MAD_Y = range(10)

DEFAULT_SEED = 0x5EEDC1BEA4D355

# operand formats of the host generator (enum OperandFormat)
F16, BF16, E4M3, E5M2, E2M3, E3M2, E2M1, I8 = range(8)
_BITS = {F16: 16, BF16: 16, E4M3: 8, E5M2: 8, E2M3: 6, E3M2: 6, E2M1: 4, I8: 8}

# kind id (MI355_MFMA_* / MI355_SMFMAC_* of include/clpeak_mi355.h) -> row tag, tile, operand format, sigma
DENSE = {
    0: dict(name="mfma_fp16", shape="16x16x32", M=16, N=16, K=32, fmt=F16, scaled=False, sigma=0.01),
    1: dict(name="mfma_bf16", shape="16x16x32", M=16, N=16, K=32, fmt=BF16, scaled=False, sigma=0.01),
    2: dict(name="mfma_fp16_32x32x16", shape="32x32x16", M=32, N=32, K=16, fmt=F16, scaled=False, sigma=0.01),
    3: dict(name="mfma_bf16_32x32x16", shape="32x32x16", M=32, N=32, K=16, fmt=BF16, scaled=False, sigma=0.01),
    4: dict(name="mfma_int8", shape="16x16x64", M=16, N=16, K=64, fmt=I8, scaled=False, sigma=0.0),
    5: dict(name="mfma_fp8", shape="16x16x128", M=16, N=16, K=128, fmt=E4M3, scaled=False, sigma=1.0),
    6: dict(name="mfma_bf8", shape="16x16x128", M=16, N=16, K=128, fmt=E5M2, scaled=False, sigma=1.0),
    7: dict(name="mfma_mxfp6_e2m3", shape="16x16x128", M=16, N=16, K=128, fmt=E2M3, scaled=True, sigma=1.0),
    8: dict(name="mfma_mxfp6_e3m2", shape="16x16x128", M=16, N=16, K=128, fmt=E3M2, scaled=True, sigma=1.0),
    9: dict(name="mfma_mxfp4", shape="16x16x128", M=16, N=16, K=128, fmt=E2M1, scaled=True, sigma=1.0),
}
SPARSE = {
    0: dict(name="smfmac_fp16", shape="16x16x64", K=64, fmt=F16, sigma=0.01),
    1: dict(name="smfmac_bf16", shape="16x16x64", K=64, fmt=BF16, sigma=0.01),
    2: dict(name="smfmac_fp8", shape="16x16x128", K=128, fmt=E4M3, sigma=1.0),
    3: dict(name="smfmac_bf8", shape="16x16x128", K=128, fmt=E5M2, sigma=1.0),
    4: dict(name="smfmac_int8", shape="16x16x128", K=128, fmt=I8, sigma=0.0),
}

# The operand codes of the reference's own kernels, which run on constants: 1.0 in the 16-bit kinds
# (src/rocm/rocm_kernels/mfma_fp16.hip:24-25, mfma_bf16.hip:16-17), byte 0x38 in the 8-bit floating kinds
# (mfma_fp8.hip:17-18: 1.0 as e4m3, 0.5 as e5m2), byte 0x01 for int8 (mfma_int8.hip:17-18), nibble 4 (2.0 as
# e2m1) under E8M0 scales of 0x3f for the block-scaled kind (mfma_mxfp4.hip:23-29), sparsity index 0
# (smfmac_fp16.hip:26).  The two fp6 kinds, which the reference does not have, take their code of 1.0.
REFERENCE_CODE = {F16: 0x3C00, BF16: 0x3F80, E4M3: 0x38, E5M2: 0x38, E2M3: 0x08, E3M2: 0x0C, E2M1: 0x4, I8: 0x01}
REFERENCE_VALUE = {F16: 1.0, BF16: 1.0, E4M3: 1.0, E5M2: 0.5, E2M3: 1.0, E3M2: 1.0, E2M1: 2.0, I8: 1}
REFERENCE_SCALE, REFERENCE_META = 0x3F, 0x00

_lib = None


def _host():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError(f"{HOST_LIB_PATH} is not built (python -c 'import __graft_entry__ as g; g.build()')")
        L = C.CDLL(HOST_LIB_PATH)
        L.clpeak_host_seeded_operand.argtypes = [C.c_int, C.c_double, C.c_ulonglong, C.c_uint, C.c_ulonglong,
                                                 C.c_void_p, C.c_size_t]
        L.clpeak_host_seeded_operand.restype = C.c_size_t
        L.clpeak_host_reference_operand.argtypes = [C.c_int, C.c_ulonglong, C.c_void_p, C.c_size_t]
        L.clpeak_host_reference_operand.restype = C.c_size_t
        L.clpeak_host_seeded_bytes.argtypes = [C.c_int, C.c_ulonglong, C.c_uint, C.c_ulonglong, C.c_void_p]
        L.clpeak_host_seeded_bytes.restype = C.c_size_t
        _lib = L
    return _lib


def operand(fmt, sigma, seed, stream, n):
    """n elements of `stream` in `fmt`, packed K-contiguously (uint8 array)."""
    out = np.empty(n * _BITS[fmt] // 8, dtype=np.uint8)
    got = _host().clpeak_host_seeded_operand(fmt, sigma, seed, stream, n, out.ctypes.data, out.size)
    if got != out.size:
        raise RuntimeError(f"host generator wrote {got} of {out.size} bytes")
    return out


def constant_operand(fmt, code, n):
    """n elements, each the bit pattern `code` of `fmt`, packed as `operand` packs them."""
    bits = _BITS[fmt]
    if bits == 16:
        return np.full(n, code, dtype="<u2").view(np.uint8)
    if bits == 8:
        return np.full(n, code, dtype=np.uint8)
    if bits == 4:
        return np.full(n // 2, code | code << 4, dtype=np.uint8)
    word = code | code << 6 | code << 12 | code << 18          # four 6-bit elements in three bytes
    return np.tile(np.array([word & 0xFF, word >> 8 & 0xFF, word >> 16 & 0xFF], dtype=np.uint8), n // 4)


def reference_operand(fmt, n):
    """n elements of the reference's constant for `fmt`, from the host layer's generator (what `Mi355Peak`
    uploads under --reference-operands)."""
    out = np.empty(n * _BITS[fmt] // 8, dtype=np.uint8)
    got = _host().clpeak_host_reference_operand(fmt, n, out.ctypes.data, out.size)
    if got != out.size:
        raise RuntimeError(f"host generator wrote {got} of {out.size} bytes")
    return out


def reference_dense_inputs(kind, waves):
    """The shapes of `dense_inputs`, every element the constant the reference's kernel of the kind holds."""
    s = DENSE[kind]
    units = waves * 4
    A = reference_operand(s["fmt"], units * s["M"] * s["K"])
    B = reference_operand(s["fmt"], units * s["N"] * s["K"])
    sA = sB = None
    if s["scaled"]:
        sA = np.full(units * s["M"] * (s["K"] // 32), REFERENCE_SCALE, dtype=np.uint8)
        sB = np.full(units * s["N"] * (s["K"] // 32), REFERENCE_SCALE, dtype=np.uint8)
    return A, B, sA, sB


def reference_sparse_inputs(kind, waves):
    s = SPARSE[kind]
    units = waves * 4
    Ac = reference_operand(s["fmt"], units * 16 * (s["K"] // 2))
    B = reference_operand(s["fmt"], units * 16 * s["K"])
    return Ac, np.full(units * 16 * (s["K"] // 4), REFERENCE_META, dtype=np.uint8), B


def e8m0_scales(seed, stream, n):
    out = np.empty(n, dtype=np.uint8)
    _host().clpeak_host_seeded_bytes(0, seed, stream, n, out.ctypes.data)
    return out


def sparse_meta(seed, stream, n):
    out = np.empty(n, dtype=np.uint8)
    _host().clpeak_host_seeded_bytes(1, seed, stream, n, out.ctypes.data)
    return out


def dense_inputs(kind, waves, seed=DEFAULT_SEED):
    """A[wave][chain][M][K], B[wave][chain][N][K] (packed bytes), scaleA, scaleB (or None)."""
    s = DENSE[kind]
    units = waves * 4
    A = operand(s["fmt"], s["sigma"], seed, STREAM_MFMA_A, units * s["M"] * s["K"])
    B = operand(s["fmt"], s["sigma"], seed, STREAM_MFMA_B, units * s["N"] * s["K"])
    sA = sB = None
    if s["scaled"]:
        sA = e8m0_scales(seed, STREAM_SCALE_A, units * s["M"] * (s["K"] // 32))
        sB = e8m0_scales(seed, STREAM_SCALE_B, units * s["N"] * (s["K"] // 32))
    return A, B, sA, sB


def sparse_inputs(kind, waves, seed=DEFAULT_SEED):
    """Ac[wave][chain][16][K/2], meta[wave][chain][16][K/4], B[wave][chain][16][K]."""
    s = SPARSE[kind]
    units = waves * 4
    Ac = operand(s["fmt"], s["sigma"], seed, STREAM_MFMA_A, units * 16 * (s["K"] // 2))
    B = operand(s["fmt"], s["sigma"], seed, STREAM_MFMA_B, units * 16 * s["K"])
    meta = sparse_meta(seed, STREAM_SPARSE, units * 16 * (s["K"] // 4))
    return Ac, meta, B


def dense_flops(kind, waves, iters):
    s = DENSE[kind]
    return 2.0 * s["M"] * s["N"] * s["K"] * 4 * waves * iters


def sparse_flops(kind, waves, iters):
    return 2.0 * 16 * 16 * SPARSE[kind]["K"] * 4 * waves * iters
