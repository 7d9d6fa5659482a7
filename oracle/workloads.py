"""Seeded operands of the matrix workloads, built with the CPU oracle's generator.

Test infrastructure (like everything under oracle/): used by tests/, by
__graft_entry__.smoke() and by bench.py to make the inputs that are handed both to the
HIP kernels (through the C ABI) and to the oracle.
"""
import numpy as np

from . import pyoracle as orc

# stream ids (must match clpeak_amd/csrc/seeded_rng.h; tests/test_abi.py checks)
STREAM_BW, STREAM_MAD, STREAM_MFMA_A, STREAM_MFMA_B, STREAM_SCALE_A, STREAM_SCALE_B, \
    STREAM_SPARSE, STREAM_GEMM_A, STREAM_GEMM_B, STREAM_MAD_Y = range(10)

DEFAULT_SEED = 0x5EEDC1BEA4D355  # one fixed seed for every seeded input

# kind id -> (name, M, N, K, oracle fmt (None = int8), bits, scaled, sigma, flops-unit)
DENSE = {
    0: dict(name="mfma_fp16", shape="16x16x32", M=16, N=16, K=32, fmt=orc.FMT_F16, bits=16, scaled=False, sigma=0.01),
    1: dict(name="mfma_bf16", shape="16x16x32", M=16, N=16, K=32, fmt=orc.FMT_BF16, bits=16, scaled=False, sigma=0.01),
    2: dict(name="mfma_fp16_32x32x16", shape="32x32x16", M=32, N=32, K=16, fmt=orc.FMT_F16, bits=16, scaled=False, sigma=0.01),
    3: dict(name="mfma_bf16_32x32x16", shape="32x32x16", M=32, N=32, K=16, fmt=orc.FMT_BF16, bits=16, scaled=False, sigma=0.01),
    4: dict(name="mfma_int8", shape="16x16x64", M=16, N=16, K=64, fmt=None, bits=8, scaled=False, sigma=None),
    5: dict(name="mfma_fp8", shape="16x16x128", M=16, N=16, K=128, fmt=orc.FMT_E4M3, bits=8, scaled=False, sigma=1.0),
    6: dict(name="mfma_bf8", shape="16x16x128", M=16, N=16, K=128, fmt=orc.FMT_E5M2, bits=8, scaled=False, sigma=1.0),
    7: dict(name="mfma_mxfp6_e2m3", shape="16x16x128", M=16, N=16, K=128, fmt=orc.FMT_E2M3, bits=6, scaled=True, sigma=1.0),
    8: dict(name="mfma_mxfp6_e3m2", shape="16x16x128", M=16, N=16, K=128, fmt=orc.FMT_E3M2, bits=6, scaled=True, sigma=1.0),
    9: dict(name="mfma_mxfp4", shape="16x16x128", M=16, N=16, K=128, fmt=orc.FMT_E2M1, bits=4, scaled=True, sigma=1.0),
}
SPARSE = {
    0: dict(name="smfmac_fp16", shape="16x16x64", K=64, fmt=orc.FMT_F16, bits=16, sigma=0.01),
    1: dict(name="smfmac_bf16", shape="16x16x64", K=64, fmt=orc.FMT_BF16, bits=16, sigma=0.01),
    2: dict(name="smfmac_fp8", shape="16x16x128", K=128, fmt=orc.FMT_E4M3, bits=8, sigma=1.0),
    3: dict(name="smfmac_bf8", shape="16x16x128", K=128, fmt=orc.FMT_E5M2, bits=8, sigma=1.0),
    4: dict(name="smfmac_int8", shape="16x16x128", K=128, fmt=None, bits=8, sigma=None),
}


def _codes(spec, seed, stream, n):
    if spec["fmt"] is None:
        return orc.fill_int8(seed, stream, n).view(np.uint8)
    return orc.fill_normal_codes(spec["fmt"], spec["sigma"], seed, stream, n)


def _pack(codes, bits):
    if bits in (8, 16):
        return codes.view(np.uint8)
    return orc.pack_bits(codes, bits)  # rows are multiples of 8 bits, so packing the flat stream keeps rows apart


def dense_inputs(kind, waves, seed=DEFAULT_SEED):
    """A[wave][chain][M][K], B[wave][chain][N][K] (packed bytes), scaleA, scaleB (or None)."""
    s = DENSE[kind]
    units = waves * 4
    A = _pack(_codes(s, seed, STREAM_MFMA_A, units * s["M"] * s["K"]), s["bits"])
    B = _pack(_codes(s, seed, STREAM_MFMA_B, units * s["N"] * s["K"]), s["bits"])
    sA = sB = None
    if s["scaled"]:
        sA = orc.fill_e8m0(seed, STREAM_SCALE_A, units * s["M"] * (s["K"] // 32))
        sB = orc.fill_e8m0(seed, STREAM_SCALE_B, units * s["N"] * (s["K"] // 32))
    return A, B, sA, sB


def sparse_inputs(kind, waves, seed=DEFAULT_SEED):
    """Ac[wave][chain][16][K/2], meta[wave][chain][16][K/4], B[wave][chain][16][K]."""
    s = SPARSE[kind]
    units = waves * 4
    Ac = _codes(s, seed, STREAM_MFMA_A, units * 16 * (s["K"] // 2)).view(np.uint8)
    B = _codes(s, seed, STREAM_MFMA_B, units * 16 * s["K"]).view(np.uint8)
    meta = orc.fill_sparse_meta(seed, STREAM_SPARSE, units * 16 * (s["K"] // 4))
    return Ac, meta, B


def dense_flops(kind, waves, iters):
    s = DENSE[kind]
    return 2.0 * s["M"] * s["N"] * s["K"] * 4 * waves * iters


def sparse_flops(kind, waves, iters):
    return 2.0 * 16 * 16 * SPARSE[kind]["K"] * 4 * waves * iters
