"""GPU parity of the matrix-instruction kernels against the CPU oracle.

Integer kinds are bit-exact.  Floating kinds cannot be: measured on gfx950, the matrix
pipe neither forms the K-long dot product exactly (f16/bf16 and, much more so, fp8/bf8
align the products with a limited number of bits; fp6/fp4 are exact) nor rounds the
running fp32 accumulator to nearest every time.  The oracle accumulates the exact dot
product with one fp32 round-to-nearest per iteration, and the stated tolerance is, per
element,

    |gpu - oracle| <= (DOT_TOL + iters * 2^-23) * iters * sum_k |a_k * b_k|

i.e. 2^-14.6 of the product magnitudes for the dot product plus at most one unit in the
last place of the accumulator per iteration, all in the same direction (the accumulator
never exceeds iters * sum|a*b|).  At 4096 iterations this is 5.3e-4; the observed worst
case is 1.4e-4."""
import numpy as np
import pytest

from clpeak_amd import capi
from clpeak_amd import workloads as product_wl
from oracle import pyoracle as orc
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
SEED = wl.DEFAULT_SEED
DOT_TOL = 4e-5   # relative to sum|a_k * b_k|, one instruction


def _chain0_everywhere(x, waves):
    """What the kernel computes on with MFMA_ONE_OPERAND_SET: every chain of a wave holds chain 0's operand."""
    if x is None:
        return None
    y = np.ascontiguousarray(x).reshape(waves, 4, -1).copy()
    y[:, 1:, :] = y[:, :1, :]
    return y.reshape(x.shape)


def _run_dense(dev, kind, waves, iters, seed=SEED, one_set=False):
    s = wl.DENSE[kind]
    A, B, sA, sB = wl.dense_inputs(kind, waves, seed)
    dA, dB = dev.from_host(A), dev.from_host(B)
    dsA = dev.from_host(sA) if sA is not None else None
    dsB = dev.from_host(sB) if sB is not None else None
    n_out = waves * 4 * s["M"] * s["N"]
    out = dev.alloc(n_out * 4)
    dev.mfma_dense(kind, dA, dB, dsA, dsB, out, waves, iters, one_set=one_set)
    is_int = s["fmt"] is None
    got = out.download(np.int32 if is_int else np.float32, n_out)
    if one_set:   # the device was handed the full arrays; the oracle gets what the flag makes of them
        A, B, sA, sB = (_chain0_everywhere(x, waves) for x in (A, B, sA, sB))
    ref, ab = orc.mfma_dense(kind, A, B, sA, sB, waves, iters, s["M"] * s["N"], is_int=is_int)
    for b in (dA, dB, dsA, dsB, out):
        if b is not None:
            b.free()
    return got, ref, ab, is_int


def _check(got, ref, ab, is_int, what, iters):
    if is_int:
        assert np.array_equal(got, ref), what
    else:
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
        bound = (DOT_TOL + iters * 2.0 ** -23) * ab + 1e-30
        worst = float((err / bound).max())
        assert worst <= 1.0, (what, worst, float(err.max()))
        assert np.count_nonzero(got) > got.size * 0.9, what   # a kernel that wrote nothing must not pass


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_mfma_dense_parity(dev, kind, iters):
    got, ref, ab, is_int = _run_dense(dev, kind, 8, iters)
    _check(got, ref, ab, is_int, (wl.DENSE[kind]["name"], iters), iters)


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_mfma_dense_parity_one_operand_set(dev, kind, iters):
    """The launch the benchmark rows use: the four chains of a wave take chain 0's fragments from the same
    registers (one a and one b for all accumulator chains, as in the reference's kernels).  The four tiles of
    a wave must then be equal among themselves as well as right."""
    got, ref, ab, is_int = _run_dense(dev, kind, 8, iters, one_set=True)
    _check(got, ref, ab, is_int, (wl.DENSE[kind]["name"], iters), iters)
    tiles = got.reshape(8, 4, -1)
    assert all(np.array_equal(tiles[:, 0], tiles[:, c]) for c in (1, 2, 3))


@pytest.mark.parametrize("one_set", [False, True])
@pytest.mark.parametrize("kind", sorted(wl.DENSE))
def test_mfma_dense_full_launch_sampled(dev, kind, one_set):
    """The configured launch: 2048 waves x 4 chains x 4096 iterations.  The oracle replays
    every wave (seconds) and the whole output is compared."""
    got, ref, ab, is_int = _run_dense(dev, kind, 2048, 4096, one_set=one_set)
    _check(got, ref, ab, is_int, wl.DENSE[kind]["name"], 4096)


@pytest.mark.parametrize("seed,waves,iters", [(1, 4, 33), (0xDEADBEEF, 12, 95)])
@pytest.mark.parametrize("one_set", [False, True])
def test_other_seeds_launch_sizes_and_mixed_loop_trips(dev, seed, waves, iters, one_set):
    """Iteration counts that take both loops of a kernel (runs of 32, then single instructions), wave counts
    that are not a power of two, seeds other than the configured one: every dense and sparse kind."""
    for kind in sorted(wl.DENSE):
        got, ref, ab, is_int = _run_dense(dev, kind, waves, iters, seed=seed, one_set=one_set)
        _check(got, ref, ab, is_int, (wl.DENSE[kind]["name"], seed, waves, iters), iters)
    for kind in sorted(wl.SPARSE):
        got, ref, ab, is_int = _run_sparse(dev, kind, waves, iters, seed=seed, one_set=one_set)
        _check(got, ref, ab, is_int, (wl.SPARSE[kind]["name"], seed, waves, iters), iters)


def test_mfma_int8_linearity(dev):
    """Size-independent property: n iterations = n x one iteration (exact in int32)."""
    g1, _, _, _ = _run_dense(dev, capi.MFMA_I8_16x16x64, 64, 1)
    gn, _, _, _ = _run_dense(dev, capi.MFMA_I8_16x16x64, 64, 4096)
    assert np.array_equal(gn.astype(np.int64), g1.astype(np.int64) * 4096)


def _run_sparse(dev, kind, waves, iters, seed=SEED, one_set=False):
    s = wl.SPARSE[kind]
    Ac, meta, B = wl.sparse_inputs(kind, waves, seed)
    dA, dM, dB = dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)
    n_out = waves * 4 * 256
    out = dev.alloc(n_out * 4)
    dev.smfmac(kind, dA, dM, dB, out, waves, iters, one_set=one_set)
    is_int = s["fmt"] is None
    got = out.download(np.int32 if is_int else np.float32, n_out)
    if one_set:
        Ac, meta, B = (_chain0_everywhere(x, waves) for x in (Ac, meta, B))
    ref, ab = orc.smfmac(kind, Ac, meta, B, waves, iters, is_int=is_int)
    for b in (dA, dM, dB, out):
        b.free()
    return got, ref, ab, is_int


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_smfmac_parity(dev, kind, iters):
    got, ref, ab, is_int = _run_sparse(dev, kind, 8, iters)
    _check(got, ref, ab, is_int, (wl.SPARSE[kind]["name"], iters), iters)


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_smfmac_parity_one_operand_set(dev, kind, iters):
    got, ref, ab, is_int = _run_sparse(dev, kind, 8, iters, one_set=True)
    _check(got, ref, ab, is_int, (wl.SPARSE[kind]["name"], iters), iters)
    tiles = got.reshape(8, 4, -1)
    assert all(np.array_equal(tiles[:, 0], tiles[:, c]) for c in (1, 2, 3))


@pytest.mark.parametrize("one_set", [False, True])
@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
def test_smfmac_full_launch(dev, kind, one_set):
    got, ref, ab, is_int = _run_sparse(dev, kind, 2048, 4096, one_set=one_set)
    _check(got, ref, ab, is_int, wl.SPARSE[kind]["name"], 4096)


def _closed_form(fmt, terms, iters, scaled):
    """acc after `iters` instructions that each add `terms` products of the reference's constant with itself."""
    v = float(product_wl.REFERENCE_VALUE[fmt])
    block = 2.0 ** (2 * (product_wl.REFERENCE_SCALE - 127)) if scaled else 1.0
    return iters * terms * v * v * block


@pytest.mark.parametrize("one_set", [False, True])
@pytest.mark.parametrize("kind", sorted(product_wl.DENSE))
def test_mfma_dense_on_the_reference_operands(dev, kind, one_set):
    """The reference's kernels multiply constants (1.0, byte 0x38, byte 0x01, nibble 4 under scales of 0x3f:
    src/rocm/rocm_kernels/mfma_bf16.hip:16-17, mfma_fp8.hip:17-18, mfma_int8.hip:17-18, mfma_mxfp4.hip:23-29).
    On those inputs every element of every accumulator is iterations x K x constant^2 (x both block
    scales), a power of two times an integer below 2^24: exact in fp32 and int32, so the comparison is."""
    s = product_wl.DENSE[kind]
    waves = 8
    A, B, sA, sB = product_wl.reference_dense_inputs(kind, waves)
    n_out = waves * 4 * s["M"] * s["N"]
    for iters in (1, 13, 4096):
        bufs = [dev.from_host(x) if x is not None else None for x in (A, B, sA, sB)]
        out = dev.alloc(n_out * 4)
        dev.mfma_dense(kind, bufs[0], bufs[1], bufs[2], bufs[3], out, waves, iters, one_set=one_set)
        is_int = s["fmt"] == product_wl.I8
        got = out.download(np.int32 if is_int else np.float32, n_out)
        want = _closed_form(s["fmt"], s["K"], iters, s["scaled"])
        assert np.all(got == (np.int32(want) if is_int else np.float32(want))), (s["name"], iters, got[:4], want)
        ref, _ = orc.mfma_dense(kind, A, B, sA, sB, waves, iters, s["M"] * s["N"], is_int=is_int)
        assert np.array_equal(got, ref), (s["name"], iters)
        for b in bufs + [out]:
            if b is not None:
                b.free()


@pytest.mark.parametrize("one_set", [False, True])
@pytest.mark.parametrize("kind", sorted(product_wl.SPARSE))
def test_smfmac_on_the_reference_operands(dev, kind, one_set):
    """Constants and sparsity index 0 (src/rocm/rocm_kernels/smfmac_fp16.hip:24-27, smfmac_fp8.hip:19-21,
    smfmac_int8.hip:18-20): K/2 kept values per row, each against a B element of the same constant.  Index 0
    names position 0 of every group twice, which the oracle refuses as metadata; it is given the first
    proper pattern (positions 0 and 1) instead, which on a constant B selects the same values."""
    s = product_wl.SPARSE[kind]
    waves = 8
    Ac, meta, B = product_wl.reference_sparse_inputs(kind, waves)
    n_out = waves * 4 * 256
    for iters in (1, 13, 4096):
        bufs = [dev.from_host(x) for x in (Ac, meta, B)]
        out = dev.alloc(n_out * 4)
        dev.smfmac(kind, bufs[0], bufs[1], bufs[2], out, waves, iters, one_set=one_set)
        is_int = s["fmt"] == product_wl.I8
        got = out.download(np.int32 if is_int else np.float32, n_out)
        want = _closed_form(s["fmt"], s["K"] // 2, iters, False)
        assert np.all(got == (np.int32(want) if is_int else np.float32(want))), (s["name"], iters, got[:4], want)
        ref, _ = orc.smfmac(kind, Ac, np.full_like(meta, 0b0100), B, waves, iters, is_int=is_int)
        assert np.array_equal(got, ref), (s["name"], iters)
        for b in bufs + [out]:
            b.free()


# --- the diagnosis flags: only some workgroups take part ---------------------------------------------------------
@pytest.mark.parametrize("on_xcds,half_cus", [((0, 1, 2, 3), False), ((0,), False), (None, True), ((0, 5), True)])
def test_matrix_kernels_on_a_subset_of_the_part(dev, on_xcds, half_cus):
    """MI355_MATRIX_ON_XCDS / MI355_MATRIX_ON_HALF_THE_CUS: the workgroups that take part (workgroup index mod 8 among
    the XCDs named; index / 8 mod 32 below 16) give exactly what the whole launch gives, bit for bit, the others leave
    their output tiles untouched; a subset without XCD 0 is refused."""
    waves, iters = 2048, 64
    for sparse, kind in ((False, capi.MFMA_I8_16x16x64), (True, capi.SMFMAC_F16_16x16x64)):
        if sparse:
            Ac, meta, B = wl.sparse_inputs(kind, waves, SEED)
            bufs = [dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)]
            launch = lambda o, **kw: dev.smfmac(kind, bufs[0], bufs[1], bufs[2], o, waves, iters, **kw)
            per_wave, dtype = 4 * 256, np.uint32
        else:
            A, B, _, _ = wl.dense_inputs(kind, waves, SEED)
            bufs = [dev.from_host(A), dev.from_host(B)]
            launch = lambda o, **kw: dev.mfma_dense(kind, bufs[0], bufs[1], None, None, o, waves, iters, **kw)
            per_wave, dtype = 4 * 256, np.uint32
        whole, part = dev.alloc(waves * per_wave * 4), dev.alloc(waves * per_wave * 4)
        dev.memset(whole, 0xa5); dev.memset(part, 0xa5)
        launch(whole)
        launch(part, on_xcds=on_xcds, half_cus=half_cus)
        w = whole.download(dtype, waves * per_wave).reshape(waves // 4, 4 * per_wave)     # one row per workgroup
        p = part.download(dtype, waves * per_wave).reshape(waves // 4, 4 * per_wave)
        wg = np.arange(waves // 4)
        takes_part = np.ones(waves // 4, dtype=bool)
        if on_xcds is not None:
            takes_part &= np.isin(wg % 8, on_xcds)
        if half_cus:
            takes_part &= (wg // 8) % 32 < 16
        assert 0 < takes_part.sum() < waves // 4
        assert np.array_equal(p[takes_part], w[takes_part])
        assert np.all(p[~takes_part] == 0xa5a5a5a5)
        with pytest.raises(capi.Mi355Error, match="XCD 0 must be among"):
            launch(part, on_xcds=(1, 2))
        for b in bufs + [whole, part]:
            b.free()
