"""Pins the oracle's kernels (CPU only) against what the mathematics fixes: closed forms
of the affine recurrence, numpy restatements written from the definitions in
include/clpeak_mi355.h, exact integer arithmetic in Python, special cases."""
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from oracle import workloads as wl


# ---- global bandwidth --------------------------------------------------------------
@pytest.mark.parametrize("width", [1, 2, 4])
@pytest.mark.parametrize("n,T", [(4096, 64), (4096 + 64, 128), (1000 * 4, 192), (64, 256)])
def test_bandwidth_partials_brute_force(width, n, T):
    data = orc.fill_f32(n, 3, wl.STREAM_BW, 0)
    got = orc.global_bandwidth(width, data, T)
    vec = data.reshape(-1, width)
    ref = np.zeros(T, dtype=np.float32)
    for t in range(T):
        acc = np.zeros(width, dtype=np.float32)
        for v in vec[t::T]:                      # thread t owns vectors t, t+T, ...
            acc = (acc + v).astype(np.float32)
        s = acc[0]
        for c in range(1, width):
            s = np.float32(s + acc[c])
        ref[t] = s
    assert np.array_equal(got, ref)
    # invariant: the grand total does not depend on the vector width (up to fp32 rounding)
    assert abs(float(got.astype(np.float64).sum()) - float(data.astype(np.float64).sum())) < 1e-5 * n


def test_bandwidth_seeded_thread_matches_buffer_version():
    n, T = 1 << 16, 512
    data = orc.fill_f32(n, 77, wl.STREAM_BW, 0)
    for width in (1, 2, 4):
        full = orc.global_bandwidth(width, data, T)
        for t in (0, 1, 255, 511):
            assert orc.global_bandwidth_thread(width, 77, wl.STREAM_BW, n, T, t) == full[t]


# ---- MAD chains ----------------------------------------------------------------------
def _seeds(seed, first, n, per=16, stream=wl.STREAM_MAD):
    return orc.fill_f32(n * per, seed, stream, 1, first=first * per).reshape(n, per).astype(np.float64)


def test_mad_f64_closed_form():
    """x_n = a^n x0 + x0 (a^n - 1)/(a - 1); the double chain tracks it to ~1e-12."""
    n, steps, a = 32, 4096, 1.0001
    got = orc.compute_mad(2, 1, 99, 5, n, steps)
    x0 = _seeds(99, 5, n)
    xn = a ** steps * x0 + x0 * (a ** steps - 1) / (a - 1)
    assert abs(a ** steps - 1.5063) < 1e-3
    assert np.allclose(got, xn.sum(axis=1), rtol=1e-10, atol=1e-9)


def test_mad_f32_closed_form_and_bit_exact_numpy():
    n, steps = 16, 4096
    got = orc.compute_mad(0, 1, 99, 0, n, steps)
    x0 = _seeds(99, 0, n)
    a = float(np.float32(1.0001))
    xn = a ** steps * x0 + x0 * (a ** steps - 1) / (a - 1)
    assert np.allclose(got, xn.sum(axis=1), rtol=2e-3)
    # bit-exact restatement: fp32 FMA = exact product-sum in float64 (24+24 bit product, one
    # add) rounded once to fp32 -- float64 holds a*x exactly, the sum's double rounding cannot
    # bite because the fp64 result keeps >= 29 bits beyond the fp32 mantissa except on exact ties
    # that the 24-bit lattice of a*x + x0 rules out for these magnitudes; checked on short chains.
    steps = 64
    got = orc.compute_mad(0, 1, 99, 0, n, steps)
    x0f = x0.astype(np.float32)
    x = x0f.copy()
    from fractions import Fraction
    for _ in range(steps):
        nxt = np.empty_like(x)
        for idx in np.ndindex(x.shape):
            exact = Fraction(float(x[idx])) * Fraction(float(np.float32(1.0001))) + Fraction(float(x0f[idx]))
            nxt[idx] = _round_fraction_to_f32(exact)
        x = nxt
    ref = np.zeros(n, dtype=np.float32)
    for j in range(16):
        ref = (ref + x[:, j]).astype(np.float32)
    assert np.array_equal(got, ref)


def _round_fraction_to_f32(q):
    """Correctly rounded (nearest even) fp32 of an exact rational."""
    from fractions import Fraction
    if q == 0:
        return np.float32(0.0)
    f = float(q)                       # float(Fraction) is correctly rounded to double
    c = np.float32(f)
    # repair a possible double rounding: compare the neighbours exactly
    cands = [np.nextafter(c, np.float32(-np.inf)), c, np.nextafter(c, np.float32(np.inf))]
    best = min(cands, key=lambda v: (abs(Fraction(float(v)) - q), int(np.float32(v).view(np.uint32)) & 1))
    return np.float32(best)


def test_mad_widths_do_not_change_results():
    for kind in (0, 2, 5):
        ref = orc.compute_mad(kind, 1, 5, 0, 8, 100)
        for w in (2, 4):
            assert np.array_equal(orc.compute_mad(kind, w, 5, 0, 8, 100), ref)


def test_mad_f16_against_numpy_float16():
    """numpy float16 arithmetic through exact float64 intermediates: fma = round16(x*a + x0)."""
    n, steps = 8, 300
    got = orc.compute_mad(1, 1, 21, 0, n, steps)
    x0 = _seeds(21, 0, n).astype(np.float16)
    a = np.float16(1 - 2.0 ** -10)
    x = x0.copy()
    for _ in range(steps):
        x = (x.astype(np.float64) * float(a) + x0.astype(np.float64)).astype(np.float16)  # exact in f64, one rounding
    s = np.zeros(n, dtype=np.float16)
    for j in range(16):
        s = (s.astype(np.float64) + x[:, j].astype(np.float64)).astype(np.float16)
    assert np.array_equal(got, s.view(np.uint16))


def _bf16_round(x):
    """float32 array -> nearest-even bfloat16, returned as float32 (numpy only)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)


def test_mad_mp_against_numpy():
    """x <- fl32(x*a + x0) with half-valued a and x0, through half every 16th step.  x*a + x0 is exact in float64
    (x within a factor 2^10 of x0, 24 + 11 bits of product), so one numpy float32 rounding of the float64 value
    is the fused multiply-add; numpy's float16 is the round trip."""
    n = 32
    u = _seeds(8, 0, n)
    x0 = u.astype(np.float16).astype(np.float32)
    a = np.float32(np.float16(1 - 2.0 ** -10))
    for steps in (1, 15, 16, 17, 100, 4096):
        x = x0.copy()
        for s in range(steps):
            x = (x.astype(np.float64) * np.float64(a) + x0.astype(np.float64)).astype(np.float32)
            if s % 16 == 15:
                x = x.astype(np.float16).astype(np.float32)
        ref = np.zeros(n, dtype=np.float32)
        for j in range(16):
            ref = (ref + x[:, j]).astype(np.float32)
        assert np.array_equal(orc.compute_mad(3, 1, 8, 0, n, steps), ref), steps
    # the recurrence heads for x0 / (1 - a) = 1024 x0: at 4096 steps 1 - a^4097 = 0.982 of it, up to the round trips
    got = orc.compute_mad(3, 1, 8, 0, n, 4096)
    terms = 1024.0 * x0.astype(np.float64) * (1 - float(a) ** 4097)
    assert np.all(np.abs(got - terms.sum(axis=1)) <= 1e-2 * np.abs(terms).sum(axis=1))   # 256 roundings to 11 bits
    # the half operands are visible: an fp32 x0 gives another result
    assert not np.allclose(got, (1024.0 * u * (1 - float(a) ** 4097)).sum(axis=1), rtol=1e-7, atol=0)


def test_mad_bf16_against_numpy_and_every_rounding_of_the_dot_product():
    """acc <- acc + xb*ab + x0b in fp32 (ab = -2^-8), xb <- bf16(acc) every 128th step, restated in numpy with the
    exact three-term sum (float64) rounded once.  The operands keep that sum short enough that the candidate
    roundings of a two-element dot product (exact sum rounded once; two chained fused multiply-adds in either
    order; the product pair rounded before the accumulator is added) all agree, so the workload's result does not
    depend on which one the hardware implements: checked here by running the oracle in each."""
    n = 64
    u = _seeds(8, 0, n)
    x0 = _bf16_round(u.astype(np.float32))
    ab = np.float64(-2.0 ** -8)
    L = orc.lib()
    try:
        for steps in (1, 127, 128, 129, 300, 4096):
            acc, xb = x0.copy(), x0.copy()
            for s in range(steps):
                acc = (acc.astype(np.float64) + xb.astype(np.float64) * ab + x0.astype(np.float64)).astype(np.float32)
                if s % 128 == 127:
                    xb = _bf16_round(acc)
            ref = np.zeros(n, dtype=np.float32)
            for j in range(16):
                ref = (ref + acc[:, j]).astype(np.float32)
            for mode in range(4):
                L.orc_set_dot2_mode(mode)
                assert np.array_equal(orc.compute_mad(4, 1, 8, 0, n, steps), ref), (steps, mode)
    finally:
        L.orc_set_dot2_mode(0)
    # per block the total moves half way to 256 x0b: after 32 blocks it is there
    got = orc.compute_mad(4, 1, 8, 0, n, 4096)
    assert np.allclose(got, (256.0 * x0.astype(np.float64)).sum(axis=1), rtol=2e-2, atol=1.0)
    # 100 steps into the first block: acc = x0b (1 + 100 (1 - 2^-8)) exactly
    got = orc.compute_mad(4, 1, 8, 0, n, 100)
    assert np.allclose(got, (x0.astype(np.float64) * (1 + 100 * (1 - 2.0 ** -8))).sum(axis=1), rtol=1e-6, atol=1e-6)


def test_mad_i32_exact():
    n, steps = 8, 257
    got = orc.compute_mad(5, 1, 4, 3, n, steps)
    for q in range(n):
        total = 0
        for j in range(16):
            x0 = orc.rng_word(4, wl.STREAM_MAD, (3 + q) * 16 + j) >> 32
            # closed form mod 2^32: x_n = x0 * (3^(n+1) - 1) / 2
            xn = (x0 * ((3 ** (steps + 1) - 1) // 2)) % (1 << 32)
            total = (total + xn) % (1 << 32)
        assert int(got[q]) == total


def test_mad_i8dp_exact():
    def sdot4(x, y, acc):
        for b in range(4):
            xb = ((x >> (8 * b)) & 0xff); xb -= 256 * (xb > 127)
            yb = ((y >> (8 * b)) & 0xff); yb -= 256 * (yb > 127)
            acc += xb * yb
        return acc & 0xffffffff
    n, steps = 4, 50
    for chains in (1, 2, 4, 8):
        got = orc.compute_mad(6, chains, 12, 0, n, steps)
        for q in range(n):
            total = 0
            for c in range(chains):
                x = orc.rng_word(12, wl.STREAM_MAD, q * 8 + c) >> 32
                y = orc.rng_word(12, wl.STREAM_MAD_Y, q * 8 + c) >> 32
                acc = 0
                for _ in range(steps):
                    acc = sdot4(x, y, acc)
                    y ^= acc
                total = (total + acc) & 0xffffffff
            assert int(got[q]) & 0xffffffff == total


# ---- matrix instructions ------------------------------------------------------------------
def _unpack(packed, bits, n):
    if bits == 16:
        return packed.view(np.uint16)[:n].astype(np.uint32)
    if bits == 8:
        return packed[:n].astype(np.uint32)
    b = np.unpackbits(packed, bitorder="little")[: n * bits].reshape(n, bits)
    return (b.astype(np.uint32) << np.arange(bits, dtype=np.uint32)).sum(axis=1)


def _dense_reference(kind, A, B, sA, sB, waves, iters):
    """float64 A.B^T per (wave, chain) from the definitions in the C header."""
    s = wl.DENSE[kind]
    M, N, K, units = s["M"], s["N"], s["K"], waves * 4
    if s["fmt"] is None:
        a = A.view(np.int8).astype(np.int64).reshape(units, M, K)
        b = B.view(np.int8).astype(np.int64).reshape(units, N, K)
        return np.einsum("umk,unk->umn", a, b) * iters
    a = orc.decode(s["fmt"], _unpack(A, s["bits"], units * M * K)).reshape(units, M, K)
    b = orc.decode(s["fmt"], _unpack(B, s["bits"], units * N * K)).reshape(units, N, K)
    if s["scaled"]:
        a = a * np.repeat(2.0 ** (sA.astype(np.float64) - 127), 32).reshape(units, M, K)
        b = b * np.repeat(2.0 ** (sB.astype(np.float64) - 127), 32).reshape(units, N, K)
    return np.einsum("umk,unk->umn", a, b) * iters


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
def test_mfma_dense_oracle_against_numpy(kind):
    s = wl.DENSE[kind]
    waves, iters = 4, 1
    A, B, sA, sB = wl.dense_inputs(kind, waves, seed=1234)
    out, ab = orc.mfma_dense(kind, A, B, sA, sB, waves, iters, s["M"] * s["N"], is_int=s["fmt"] is None)
    ref = _dense_reference(kind, A, B, sA, sB, waves, iters).reshape(-1)
    if s["fmt"] is None:
        assert np.array_equal(out.astype(np.int64), ref)
    else:
        assert np.all(np.abs(out - ref) <= 1e-6 * np.abs(ref) + 1e-30)  # one fp32 rounding of an exact sum
        assert np.all(ab >= np.abs(ref) * (1 - 1e-12))


def test_mfma_iterations_accumulate_linearly_for_int8():
    A, B, _, _ = wl.dense_inputs(4, 4, seed=9)
    one, _ = orc.mfma_dense(4, A, B, None, None, 4, 1, 256, is_int=True)
    many, _ = orc.mfma_dense(4, A, B, None, None, 4, 4096, 256, is_int=True)
    assert np.array_equal(many.astype(np.int64), one.astype(np.int64) * 4096)   # no overflow in the seeded range
    assert np.abs(many).max() < 2 ** 31 / 4


def test_mfma_fp32_chain_is_sequential_rounding():
    """acc after n steps is the n-fold fp32 running sum of one product, not n*P rounded once."""
    A, B, _, _ = wl.dense_inputs(0, 4, seed=5)
    one, _ = orc.mfma_dense(0, A, B, None, None, 4, 1, 256)
    n = 1000
    many, _ = orc.mfma_dense(0, A, B, None, None, 4, n, 256)
    exact1 = _dense_reference(0, A, B, None, None, 4, 1).reshape(-1)
    acc = np.zeros_like(one)
    for _ in range(n):
        acc = (acc.astype(np.float64) + exact1).astype(np.float32)
    assert np.array_equal(many, acc)
    assert np.allclose(many, exact1 * n, rtol=1e-4)


def test_mfma_identity_b_reproduces_a():
    """B = identity block (N x K with ones on the diagonal): out[m][n] = A[m][n]."""
    s = wl.DENSE[0]
    A, _, _, _ = wl.dense_inputs(0, 4, seed=3)
    eye = np.zeros((16, 16, 32), dtype=np.float16)  # 16 units
    for n in range(16):
        eye[:, n, n] = 1.0
    out, _ = orc.mfma_dense(0, A, eye.view(np.uint8).reshape(-1), None, None, 4, 1, 256)
    a = A.view(np.float16).reshape(16, 16, 32)[:, :, :16].astype(np.float32)
    assert np.array_equal(out.reshape(16, 16, 16), a)


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
def test_smfmac_oracle_is_dense_on_decompressed_a(kind):
    s = wl.SPARSE[kind]
    waves, K, eb = 4, s["K"], s["bits"] // 8
    Ac, meta, B = wl.sparse_inputs(kind, waves, seed=77)
    out, _ = orc.smfmac(kind, Ac, meta, B, waves, 3, is_int=s["fmt"] is None)
    # decompress in numpy from the metadata definition
    units = waves * 4
    dt = np.uint16 if eb == 2 else np.uint8
    ac = Ac.view(dt).reshape(units, 16, K // 4, 2)
    md = meta.reshape(units, 16, K // 4)
    dense = np.zeros((units, 16, K // 4, 4), dtype=dt)
    u, m, g = np.indices(md.shape)
    dense[u, m, g, md & 3] = ac[..., 0]
    dense[u, m, g, (md >> 2) & 3] = ac[..., 1]
    dense = dense.reshape(units, 16, K)
    b = B.view(dt).reshape(units, 16, K)
    if s["fmt"] is None:
        ref = np.einsum("umk,unk->umn", dense.view(np.int8).astype(np.int64), b.view(np.int8).astype(np.int64)) * 3
        assert np.array_equal(out.astype(np.int64), ref.reshape(-1))
    else:
        ref = np.einsum("umk,unk->umn", orc.decode(s["fmt"], dense), orc.decode(s["fmt"], b)) * 3
        assert np.allclose(out, ref.reshape(-1), rtol=1e-5, atol=1e-12)
    # exactly half of A is kept
    assert np.count_nonzero(md & 3 == (md >> 2) & 3) == 0


def test_smfmac_rejects_repeated_positions():
    Ac, meta, B = wl.sparse_inputs(4, 4, seed=1)
    meta = meta.copy(); meta[0] = 0b0101  # both kept values claim slot 1
    out = np.empty(4 * 4 * 256, dtype=np.int32); ab = np.empty(4 * 4 * 256)
    rc = orc.lib().orc_smfmac(4, Ac.ctypes.data, meta.ctypes.data, B.ctypes.data, out.ctypes.data, ab.ctypes.data, 4, 1)
    assert rc == -2


# ---- GEMM tiles -------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", [orc.FMT_BF16, orc.FMT_E4M3])
def test_gemm_tile_against_numpy_and_special_cases(fmt):
    M = N = 64; K = 256
    if fmt == orc.FMT_BF16:
        A = orc.fill_bf16(M * K, 1, wl.STREAM_GEMM_A, 1); B = orc.fill_bf16(N * K, 1, wl.STREAM_GEMM_B, 1)
    else:
        A = orc.fill_e4m3(M * K, 1, wl.STREAM_GEMM_A, 1, 64.0); B = orc.fill_e4m3(N * K, 1, wl.STREAM_GEMM_B, 1, 64.0)
    a = orc.decode(fmt, A).reshape(M, K); b = orc.decode(fmt, B).reshape(N, K)
    got = orc.gemm_tile(fmt, A, B, K, K, K, 16, 32, 32, 16, scale=0.5)
    assert np.allclose(got, 0.5 * (a[16:48] @ b[32:48].T), rtol=1e-12, atol=1e-12)
    # A = I (as codes): C = B^T
    one = int(orc.encode(fmt, [1.0])[0])
    I = np.zeros((M, K), dtype=A.dtype); I[np.arange(M), np.arange(M)] = one
    got = orc.gemm_tile(fmt, I, B, K, K, K, 0, 0, M, N)
    assert np.array_equal(got, b[:, :M].T)


# --- LDS ping-pong ----------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [1, 2, 4])
@pytest.mark.parametrize("block_size, reps", [(64, 1), (256, 64), (128, 300), (64, 64)])
def test_local_bandwidth_is_a_rotation(width, block_size, reps):
    """After `reps` hand-overs a thread holds the start vector of the thread `reps` places to its
    right, cyclically within its workgroup: out[b*bs + l] is a closed form of the indices.  A wrong
    direction, an off-by-one in the repetition count or a rotation across workgroups all fail this."""
    blocks = 5
    got = orc.local_bandwidth(width, blocks, block_size, reps)
    b, l = np.divmod(np.arange(blocks * block_size, dtype=np.uint32), block_size)
    src = (b * block_size + (l + reps) % block_size).astype(np.uint32)
    comps = [(src + c).astype(np.float32) for c in range(width)]
    want = comps[0]
    for c in comps[1:]:
        want = (want + c).astype(np.float32)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()


def test_local_bandwidth_large_indices_round_like_a_float_conversion():
    # thread ids above 2^24 are not exact in fp32: the start value is the rounded conversion
    got = orc.local_bandwidth(1, (1 << 24) // 256 + 2, 256, 0)
    assert got[-1] == np.float32((1 << 24) + 511) and got[(1 << 24) + 1] == np.float32(1 << 24)


# --- GEMM tiles with mixed operand formats, generic fills -------------------------------------------
def test_gemm_tile2_int8_and_mixed_formats_against_numpy():
    rng = np.random.default_rng(0)
    a = rng.integers(-8, 8, (4, 256), dtype=np.int8)
    b = rng.integers(-8, 8, (5, 256), dtype=np.int8)
    got = orc.gemm_tile2(orc.FMT_I8, orc.FMT_I8, a, b, 256, 256, 256, 0, 0, 4, 5)
    assert np.array_equal(got, a.astype(np.int64) @ b.astype(np.int64).T)
    # an e5m2 A against an e4m3 B (finite codes only), offsets and a scale: transposing the operands or
    # swapping the two decoders changes the result
    ca = rng.integers(0, 256, (6, 128), dtype=np.uint8)
    cb = rng.integers(0, 256, (7, 128), dtype=np.uint8)
    ca[(ca & 0x7f) > 0x7b] = 0x3c
    cb[(cb & 0x7f) == 0x7f] = 0x38
    got = orc.gemm_tile2(orc.FMT_E5M2, orc.FMT_E4M3, ca, cb, 128, 128, 128, 2, 3, 3, 2, 0.5)
    want = 0.5 * (orc.decode(orc.FMT_E5M2, ca[2:5]) @ orc.decode(orc.FMT_E4M3, cb[3:5]).T)
    assert np.allclose(got, want, rtol=1e-12, atol=0)
    swapped = 0.5 * (orc.decode(orc.FMT_E4M3, ca[2:5]) @ orc.decode(orc.FMT_E5M2, cb[3:5]).T)
    assert not np.allclose(got, swapped)
    # f16 against numpy's own half decoding
    ha = rng.standard_normal((3, 64)).astype(np.float16)
    hb = rng.standard_normal((4, 64)).astype(np.float16)
    got = orc.gemm_tile2(orc.FMT_F16, orc.FMT_F16, ha.view(np.uint16), hb.view(np.uint16), 64, 64, 64, 0, 0, 3, 4)
    assert np.allclose(got, ha.astype(np.float64) @ hb.astype(np.float64).T, rtol=1e-12)


def test_generic_fill_matches_library_roundings():
    import torch
    n = 20000
    u = orc.fill_f32(n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1)
    assert np.array_equal(orc.fill_fmt(orc.FMT_F16, n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1), u.astype(np.float16).view(np.uint16))
    assert np.array_equal(orc.fill_fmt(orc.FMT_BF16, n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1), orc.fill_bf16(n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1))
    for scale in (1.0, 3.0, 57344.0):
        want = (torch.from_numpy(u) * scale).to(torch.float8_e5m2).view(torch.uint8).numpy()
        assert np.array_equal(orc.fill_fmt(orc.FMT_E5M2, n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1, scale), want), scale
    # beyond the largest finite value the fill saturates (torch would give inf there)
    sat = orc.fill_fmt(orc.FMT_E5M2, n, wl.DEFAULT_SEED, wl.STREAM_GEMM_A, 1, 1e6)
    assert set(np.unique(sat & 0x7f)) <= set(range(0x7c)) and (sat & 0x7f).max() == 0x7b


def test_gemm_tile2_fp32_and_fp64_against_exact_sums():
    """fp32 / fp64 operands.  The tile sums run in long double: against math.fsum of the exact products
    (products of two fp32 values are exact in double; for fp64 operands the test uses values with 20-bit
    mantissas so that theirs are too) the result is the correctly rounded sum, or next to it."""
    import math
    rng = np.random.default_rng(7)
    a = rng.standard_normal((5, 96)).astype(np.float32)
    b = rng.standard_normal((4, 96)).astype(np.float32)
    got = orc.gemm_tile2(orc.FMT_F32, orc.FMT_F32, a, b, 96, 96, 96, 1, 0, 3, 4)
    want = np.array([[math.fsum(float(x) * float(y) for x, y in zip(a[1 + i], b[j])) for j in range(4)] for i in range(3)])
    assert np.allclose(got, want, rtol=4e-16, atol=0)
    # fp64 with a cancellation a double-only sum gets visibly wrong: 2^40 + (terms with 20 fraction bits) - 2^40
    da = np.round(rng.standard_normal((2, 64)) * 2 ** 10) / 2 ** 10
    db = np.round(rng.standard_normal((3, 64)) * 2 ** 10) / 2 ** 10
    da[:, 0] = 2.0 ** 20; db[:, 0] = 2.0 ** 20; da[:, 63] = -(2.0 ** 20); db[:, 63] = 2.0 ** 20
    got = orc.gemm_tile2(orc.FMT_F64, orc.FMT_F64, da, db, 64, 64, 64, 0, 0, 2, 3, 0.25)
    want = np.array([[0.25 * math.fsum(float(x) * float(y) for x, y in zip(da[i], db[j])) for j in range(3)] for i in range(2)])
    assert np.array_equal(got, want)
    plain = 0.25 * np.array([[sum(float(x) * float(y) for x, y in zip(da[i], db[j])) for j in range(3)] for i in range(2)])
    assert not np.array_equal(plain, want)          # the case does tell a double sum from a wider one
    # transposition or a wrong leading dimension shows: a non-square tile out of a larger matrix
    big_a = rng.standard_normal((8, 32)); big_b = rng.standard_normal((6, 32))
    got = orc.gemm_tile2(orc.FMT_F64, orc.FMT_F64, big_a, big_b, 32, 32, 32, 2, 1, 4, 3)
    assert np.allclose(got, big_a[2:6] @ big_b[1:4].T, rtol=1e-13, atol=1e-13)


# ---- the reference's own operands ---------------------------------------------------------------
def test_oracle_on_the_reference_constants_is_the_closed_form():
    """The reference's kernels run on constants (src/rocm/rocm_kernels/mfma_bf16.hip:16-17, mfma_fp8.hip:17-18,
    mfma_int8.hip:17-18, mfma_mxfp4.hip:23-29, smfmac_fp16.hip:24-27).  Every accumulator element is then
    iterations x terms x constant^2 (x both block scales), exactly; the builders live on the product side."""
    from clpeak_amd import workloads as product_wl
    if not os.path.exists(product_wl.HOST_LIB_PATH):
        pytest.skip("host library not built")
    waves, iters = 4, 257
    for kind, s in product_wl.DENSE.items():
        A, B, sA, sB = product_wl.reference_dense_inputs(kind, waves)
        is_int = s["fmt"] == product_wl.I8
        out, _ = orc.mfma_dense(kind, A, B, sA, sB, waves, iters, s["M"] * s["N"], is_int=is_int)
        v = product_wl.REFERENCE_VALUE[s["fmt"]]
        want = iters * s["K"] * v * v * (2.0 ** (2 * (product_wl.REFERENCE_SCALE - 127)) if s["scaled"] else 1.0)
        assert np.all(out == want), (s["name"], out[:4], want)
    for kind, s in product_wl.SPARSE.items():
        Ac, meta, B = product_wl.reference_sparse_inputs(kind, waves)
        is_int = s["fmt"] == product_wl.I8
        out, _ = orc.smfmac(kind, Ac, np.full_like(meta, 0b0100), B, waves, iters, is_int=is_int)
        v = product_wl.REFERENCE_VALUE[s["fmt"]]
        assert np.all(out == iters * (s["K"] // 2) * v * v), (s["name"], out[:4])


# ---- block-scaled FP4 GEMM tile and the float64 buffer total -----------------------
# e2m1 values by code, written from the OCP Microscaling specification's table (sign bit 3).
_E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def _mx_dense(codes_packed, scales, rows, K):
    """Decoded, scaled operand [rows][K] from packed nibbles (low nibble = even k) and E8M0 bytes."""
    by = codes_packed.reshape(rows, K // 2)
    codes = np.empty((rows, K), dtype=np.uint8)
    codes[:, 0::2] = by & 15
    codes[:, 1::2] = by >> 4
    sc = np.exp2(scales.reshape(rows, K // 32).astype(np.float64) - 127.0)
    return _E2M1[codes] * np.repeat(sc, 32, axis=1)


def test_gemm_mx_tile_against_numpy_product():
    """Non-square tile with offsets, asymmetric scales: every product and every scaled sum is exact in float64
    (4-bit values, power-of-two scales within 2^-4..2^4, K = 96), so the comparison is for equality."""
    rng = np.random.default_rng(11)
    M, N, K = 48, 40, 96
    A = rng.integers(0, 256, size=M * K // 2, dtype=np.uint8)
    B = rng.integers(0, 256, size=N * K // 2, dtype=np.uint8)
    SA = rng.integers(123, 132, size=M * K // 32, dtype=np.uint8)
    SB = rng.integers(123, 128, size=N * K // 32, dtype=np.uint8)      # a different range from SA's
    a, b = _mx_dense(A, SA, M, K), _mx_dense(B, SB, N, K)
    m0, n0, tm, tn = 16, 8, 24, 32
    got = orc.gemm_mx_tile(A, B, SA, SB, K, m0, n0, tm, tn)
    assert np.array_equal(got, a[m0:m0 + tm] @ b[n0:n0 + tn].T)
    # the whole matrix as one tile too
    assert np.array_equal(orc.gemm_mx_tile(A, B, SA, SB, K, 0, 0, M, N), a @ b.T)


def test_gemm_mx_tile_nibble_order_and_scale_index():
    """Cases a swapped nibble order or a swapped scale index (row/block, or A's scales used for B) would fail."""
    M = N = 2
    K = 64
    A = np.zeros(M * K // 2, dtype=np.uint8)
    B = np.zeros(N * K // 2, dtype=np.uint8)
    SA = np.full(M * K // 32, 127, dtype=np.uint8)
    SB = np.full(N * K // 32, 127, dtype=np.uint8)
    # A[0][k=0] = 1.0 (code 2, LOW nibble of byte 0), A[0][k=1] = 6.0 (code 7, HIGH nibble)
    A[0] = 2 | (7 << 4)
    # B[1][k=0] = 0.5 (code 1), B[1][k=1] = 0: with the nibbles swapped the product would pair 6.0 with 0.5
    B[1 * K // 2] = 1
    C = orc.gemm_mx_tile(A, B, SA, SB, K, 0, 0, M, N)
    assert C[0, 1] == 0.5 and C[0, 0] == 0 and C[1, 0] == 0 and C[1, 1] == 0
    # scale of A row 0, block 1 (k = 32..63) only: put a value there and scale that block alone by 2^3
    A[:] = 0; B[:] = 0
    A[0 * K // 2 + 32 // 2] = 2          # A[0][32] = 1.0
    B[1 * K // 2 + 32 // 2] = 4          # B[1][32] = 2.0
    SA[0 * 2 + 1] = 130                  # A row 0, block 1: 2^3
    assert orc.gemm_mx_tile(A, B, SA, SB, K, 0, 0, M, N)[0, 1] == 16.0
    SA[:] = 127
    SA[1 * 2 + 0] = 130                  # row 1 block 0 instead (the transposed index): must not apply
    assert orc.gemm_mx_tile(A, B, SA, SB, K, 0, 0, M, N)[0, 1] == 2.0
    SA[:] = 127
    SB[1 * 2 + 1] = 125                  # B row 1, block 1: 2^-2
    assert orc.gemm_mx_tile(A, B, SA, SB, K, 0, 0, M, N)[0, 1] == 0.5
    # an offset tile sees the same element at its shifted position
    assert orc.gemm_mx_tile(A, B, SA, SB, K, 0, 1, 1, 1)[0, 0] == 0.5


@pytest.mark.parametrize("n", [1, 1000003, (1 << 20) + 7])
def test_sum_u01_against_numpy_float64(n):
    """The float64 total of the bandwidth buffer.  Every element is a multiple of 2^-24 below 1, so the sum of
    up to 2^29 of them is exact in float64 whatever the order: equality with numpy's sum, for lengths that no
    thread count divides."""
    seed, stream = 0x1234, wl.STREAM_BW
    data = orc.fill_f32(n, seed, stream, 0)
    assert orc.sum_u01(seed, stream, n) == float(data.astype(np.float64).sum())
    # and it is a sum over elements 0..n-1 of that stream, not of another stream or another seed
    assert orc.sum_u01(seed, stream + 1, n) != orc.sum_u01(seed, stream, n) or n == 0
