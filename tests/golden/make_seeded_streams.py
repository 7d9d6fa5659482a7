#!/usr/bin/env python3
"""Writes tests/golden/seeded_streams.json: the first 16 elements of every seeded input stream, in every
form the path uses, for the one fixed seed.  Made with the CPU oracle's generator at the time the
generator was pinned (tests/test_oracle_inputs.py); from then on the oracle, the host layer's generator
and the device fills are all held to this file, so that none of them can drift without a test failing.

    python tests/golden/make_seeded_streams.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import pyoracle as orc          # noqa: E402
from oracle import workloads as wl          # noqa: E402

N = 16
SEED = wl.DEFAULT_SEED


def build():
    doc = {"seed": SEED, "count": N, "words": {}, "f32": {}, "operands": {}, "bytes": {}}
    for stream in range(10):
        doc["words"][str(stream)] = [int(orc.rng_word(SEED, stream, i)) for i in range(N)]
    # fp32 draws as bit patterns: uniform [0,1) and uniform [-1,1)
    for stream, dist, key in ((wl.STREAM_BW, 0, "bw_u01"), (wl.STREAM_GEMM_A, 1, "gemm_a_upm1"), (wl.STREAM_GEMM_B, 1, "gemm_b_upm1")):
        doc["f32"][key] = [int(x) for x in orc.fill_f32(N, SEED, stream, dist).view(np.uint32)]
    # matrix operands: N(0,1)*sigma rounded once to the format (codes), as the MFMA / SMFMAC inputs
    for name, fmt, sigma in (("f16", orc.FMT_F16, 0.01), ("bf16", orc.FMT_BF16, 0.01), ("e4m3", orc.FMT_E4M3, 1.0),
                             ("e5m2", orc.FMT_E5M2, 1.0), ("e2m3", orc.FMT_E2M3, 1.0), ("e3m2", orc.FMT_E3M2, 1.0),
                             ("e2m1", orc.FMT_E2M1, 1.0)):
        doc["operands"][name] = [int(x) for x in orc.fill_normal_codes(fmt, sigma, SEED, wl.STREAM_MFMA_A, N)]
    doc["operands"]["int8"] = [int(x) for x in orc.fill_int8(SEED, wl.STREAM_MFMA_B, N)]
    doc["bytes"]["e8m0_scale_a"] = [int(x) for x in orc.fill_e8m0(SEED, wl.STREAM_SCALE_A, N)]
    doc["bytes"]["sparse_meta"] = [int(x) for x in orc.fill_sparse_meta(SEED, wl.STREAM_SPARSE, N)]
    # GEMM operand fills (uniform [-1,1), scaled for the 8-bit formats) and byte fills
    doc["operands"]["gemm_a_bf16"] = [int(x) for x in orc.fill_bf16(N, SEED, wl.STREAM_GEMM_A, 1)]
    doc["operands"]["gemm_a_e4m3_x448"] = [int(x) for x in orc.fill_e4m3(N, SEED, wl.STREAM_GEMM_A, 1, 448.0)]
    doc["bytes"]["gemm_a_fp4_pairs"] = [int(x) for x in orc.fill_bytes(N, SEED, wl.STREAM_GEMM_A, 0, 256)]
    doc["bytes"]["gemm_scale_a_123_9"] = [int(x) for x in orc.fill_bytes(N, SEED, wl.STREAM_SCALE_A, 123, 9)]
    return doc


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "seeded_streams.json")
    with open(path, "w") as f:
        json.dump(build(), f, indent=1)
        f.write("\n")
    print("wrote", path)
