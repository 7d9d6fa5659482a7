"""Pins the operand layouts of every matrix instruction the backend uses: one
instruction, register images built from logical integer-valued matrices, result compared
with the exact integer product (fp32 is exact for these magnitudes, so the comparison
is equality whatever order the hardware sums in).  The 8-bit float kinds do not sum
even small integers exactly (their products are aligned with few bits), so for them A
keeps a single non-zero per row: every output is one product, which is exact."""
import numpy as np
import pytest

from clpeak_amd import capi
from oracle import pyoracle as orc
from oracle import workloads as wl
from mfma_layouts import (c_regs_from_matrix, matrix_from_d_regs, operand_regs, pack_codes, scale_regs,
                          split_k_regs, sparse_index_regs)

pytestmark = pytest.mark.gpu


def _int_codes(fmt, ints):
    if fmt is None:
        return (ints.astype(np.int8)).view(np.uint8).astype(np.uint32)
    return orc.encode(fmt, ints.astype(np.float64))


def _raw(dev, sparse, kind, a, b, c, aux0, aux1, sel0=0, sel1=0):
    bufs = [dev.from_host(np.ascontiguousarray(x, dtype=np.uint32)) for x in (a, b, c, aux0, aux1)]
    d = dev.alloc(64 * 16 * 4)
    dev.mfma_raw(sparse, kind, *bufs, sel0, sel1, d)
    out = d.download(np.uint32, 64 * 16).reshape(64, 16)
    for x in bufs + [d]:
        x.free()
    return out


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
@pytest.mark.parametrize("sel", [(0, 0), (1, 2), (3, 3), (2, 0), (0, 1)])
def test_dense_instruction_layout(dev, kind, sel):
    s = wl.DENSE[kind]
    if not s["scaled"] and s["K"] != 128 and sel != (0, 0):
        pytest.skip("selectors only exist on the scaled instruction")
    M, N, K, bits = s["M"], s["N"], s["K"], s["bits"]
    rng = np.random.default_rng(100 + kind + 17 * sel[0] + 31 * sel[1])
    a = rng.integers(-3, 4, (M, K)); b = rng.integers(-3, 4, (N, K)); c = rng.integers(-50, 50, (M, N))
    if s["fmt"] in (orc.FMT_E4M3, orc.FMT_E5M2):
        keep = np.zeros_like(a)
        cols = rng.integers(0, K, M)
        keep[np.arange(M), cols] = rng.integers(1, 4, M) * rng.choice([-1, 1], M)
        a = keep
        b = np.where(b == 0, 1, b)
        c = np.zeros_like(c)
    dw = 8
    if K == 128 and bits == 8:
        a_regs = split_k_regs(pack_codes(_int_codes(s["fmt"], a), bits))
        b_regs = split_k_regs(pack_codes(_int_codes(s["fmt"], b), bits))
    else:
        a_regs = operand_regs(pack_codes(_int_codes(s["fmt"], a), bits), M, dw)
        b_regs = operand_regs(pack_codes(_int_codes(s["fmt"], b), bits), N, dw)
    is_int = s["fmt"] is None
    c_m = c.astype(np.int32) if is_int else c.astype(np.float32)
    ea = np.zeros((16, 4), dtype=np.int64); eb = np.zeros((16, 4), dtype=np.int64)
    aux0 = np.full(64, 0x7f7f7f7f, dtype=np.uint32); aux1 = aux0.copy()
    if K == 128:   # f8f6f4: exercise the block scales (exponents in [-2,2] keep every sum exact)
        ea = rng.integers(-2, 3, (16, 4)); eb = rng.integers(-2, 3, (16, 4))
        aux0 = scale_regs(127 + ea, sel[0]); aux1 = scale_regs(127 + eb, sel[1])
    d = _raw(dev, False, kind, a_regs, b_regs, c_regs_from_matrix(c_m), aux0, aux1, *sel)
    got = matrix_from_d_regs(d, M, N, np.int32 if is_int else np.float32)
    if K == 128:
        af = a * np.repeat(2.0 ** ea, 32, axis=1); bf = b * np.repeat(2.0 ** eb, 32, axis=1)
        ref = af @ bf.T + c
    else:
        ref = a @ b.T + c
    assert np.array_equal(got.astype(np.float64), ref.astype(np.float64)), s["name"]


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
@pytest.mark.parametrize("abid", [0, 1])
def test_sparse_instruction_layout(dev, kind, abid):
    s = wl.SPARSE[kind]
    K, bits = s["K"], s["bits"]
    if bits == 8 and abid:
        pytest.skip("8-bit kinds use all 32 index bits")
    rng = np.random.default_rng(200 + kind)
    ac = rng.integers(1, 4, (16, K // 2)) * rng.choice([-1, 1], (16, K // 2))   # non-zero kept values
    b = rng.integers(-3, 4, (16, K)); c = rng.integers(-50, 50, (16, 16))
    meta = orc.fill_sparse_meta(7, wl.STREAM_SPARSE, 16 * (K // 4)).reshape(16, K // 4)
    dense = np.zeros((16, K // 4, 4), dtype=np.int64)
    r, g = np.indices(meta.shape)
    dense[r, g, meta & 3] = ac.reshape(16, K // 4, 2)[..., 0]
    dense[r, g, (meta >> 2) & 3] = ac.reshape(16, K // 4, 2)[..., 1]
    dense = dense.reshape(16, K)
    is_int = s["fmt"] is None
    a_regs = operand_regs(pack_codes(_int_codes(s["fmt"], ac), bits), 16, 4)
    b_regs = split_k_regs(pack_codes(_int_codes(s["fmt"], b), bits))
    idx = sparse_index_regs(meta, K // 16, abid)
    c_m = c.astype(np.int32) if is_int else c.astype(np.float32)
    d = _raw(dev, True, kind, a_regs, b_regs, c_regs_from_matrix(c_m), idx, idx, abid, 0)
    got = matrix_from_d_regs(d, 16, 16, np.int32 if is_int else np.float32)
    assert np.array_equal(got.astype(np.float64), (dense @ b.T + c).astype(np.float64)), s["name"]
