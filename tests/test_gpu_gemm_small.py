"""GPU parity of the 8- and 16-bit GEMM on 128x128 tiles (the schedule for products with too few 256x256 tiles to fill
the part), and of the library's choice between the two tilings.

Same oracle, inputs and tolerance as test_gpu_gemm.py, whose checkers run here with the handle switched to the small
tiles: for every checked element |gpu - ref| <= 1e-2*|ref| + 1e-2*rms(ref tile); int8 bit for bit."""
import numpy as np
import pytest

import test_gpu_gemm as big
from clpeak_amd import capi
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
SEED = wl.DEFAULT_SEED
FOUR_TILES = [(0, 0), (0, 128), (128, 0), (128, 128)]


@pytest.fixture(autouse=True, scope="module")
def _on_the_128_tiles(dev):
    dev.gemm_tiling(capi.GEMM_TILING_128)
    yield
    dev.gemm_tiling(capi.GEMM_TILING_AUTO)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("steps", [1, 2, 3, 4, 5, 6, 7, 11, 32])
def test_every_short_k_walk(dev, fp8, steps):
    """The ring holds five steps and the loads run four ahead: walks shorter than, equal to and longer than that."""
    big._check_tiles(dev, fp8, 256, 256, steps * (128 if fp8 else 64), FOUR_TILES, whole_output_finite=True)


@pytest.mark.parametrize("kind", ["f16", "i8", "e5m2"])
@pytest.mark.parametrize("steps", [1, 2, 4, 5, 9])
def test_other_types_short_walks(dev, kind, steps):
    big._check_kind(dev, kind, 256, 256, steps * (64 if kind == "f16" else 128), FOUR_TILES)


@pytest.mark.parametrize("kind", ["bf16", "f16", "e4m3", "e5m2", "i8"])
def test_random_shapes_every_element(dev, kind):
    """The whole of C against a float64 product of the decoded operands on six seeded shapes: a tile or a step of K
    visited twice or never shows, wherever it is in the grid."""
    big.test_gemm_random_shapes_every_element(dev, kind)


@pytest.mark.parametrize("fp8", [False, True])
def test_the_shape_it_is_for_and_more_tiles_than_cus(dev, fp8):
    """2048 cubed (256 small tiles: one per CU) and a grid of 24 x 20 small tiles (480: workgroups queue for a CU)."""
    rng = np.random.default_rng(5)
    tiles = [(int(m) * 128, int(n) * 128) for m, n in zip(rng.integers(0, 16, 10), rng.integers(0, 16, 10))]
    big._check_tiles(dev, fp8, 2048, 2048, 2048, tiles + [(1920, 1920)], whole_output_finite=True)
    big._check_tiles(dev, fp8, 3072, 2560, 640, [(0, 0), (2944, 2432), (1280, 1152), (2944, 0), (0, 2432)], whole_output_finite=True)


def _product(dev, kind, M, N, K, tiling):
    """Bits of C for seeded operands under one tiling."""
    eb = 2 if kind in ("bf16", "f16") else 1
    dA, dB, dC = dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * (4 if kind == "i8" else 2))
    dev.memset(dC, 0xff)
    dev.gemm_tiling(tiling)
    if kind == "bf16":
        dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
        dev.gemm_bf16(dA, dB, dC, M, N, K)
    else:
        dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
        dev.gemm_i8(dA, dB, dC, M, N, K)
    out = dC.download(np.int32 if kind == "i8" else np.uint16, M * N)
    for buf in (dA, dB, dC):
        buf.free()
    dev.gemm_tiling(capi.GEMM_TILING_128)
    return out


def test_int8_is_the_same_on_both_tilings(dev):
    """Integer sums do not depend on their order: the two kernels must agree bit for bit on the whole of C."""
    for M, N, K in [(256, 256, 128), (768, 512, 5 * 128), (2048, 2048, 2048)]:
        assert np.array_equal(_product(dev, "i8", M, N, K, capi.GEMM_TILING_128), _product(dev, "i8", M, N, K, capi.GEMM_TILING_256)), (M, N, K)


def test_the_library_picks_by_the_number_of_tiles(dev):
    """bf16 sums are rounded in an order that differs between the kernels (the 256x256 kernel starts its walk over K at
    a different step on every XCD), so the bits of C say which kernel ran: the small tiles up to half a 256x256 tile per
    CU, the big ones above."""
    cus = dev.props.num_cus
    K = 4096
    few = _product(dev, "bf16", 2048, 2048, K, capi.GEMM_TILING_AUTO)
    small, large = _product(dev, "bf16", 2048, 2048, K, capi.GEMM_TILING_128), _product(dev, "bf16", 2048, 2048, K, capi.GEMM_TILING_256)
    assert not np.array_equal(small, large), "the two kernels cannot be told apart on this shape"
    assert 2 * 64 <= cus and np.array_equal(few, small)
    M = 256 * (cus // 2 // 8 + 1)          # M/256 x 8 tiles: just above half a tile per CU
    many = _product(dev, "bf16", M, 2048, K, capi.GEMM_TILING_AUTO)
    small, large = _product(dev, "bf16", M, 2048, K, capi.GEMM_TILING_128), _product(dev, "bf16", M, 2048, K, capi.GEMM_TILING_256)
    assert not np.array_equal(small, large) and np.array_equal(many, large)


def test_multiples_of_128_that_have_no_256_tiling(dev):
    """M or N a multiple of 128 only: the whole of C against a float64 product of the decoded operands, under the
    library's own choice of tiling (there is only one) as under the pinned one; the 256x256 tiling refuses."""
    for tiling in (capi.GEMM_TILING_AUTO, capi.GEMM_TILING_128):
        dev.gemm_tiling(tiling)
        for M, N, K in [(128, 128, 64), (384, 640, 7 * 64), (2176, 2432, 192)]:
            dA, dB, dC = dev.alloc(M * K * 2), dev.alloc(N * K * 2), dev.alloc(M * N * 2)
            dev.memset(dC, 0xff)
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            dev.gemm_bf16(dA, dB, dC, M, N, K)
            a = (dA.download(np.uint16, M * K).astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(M, K)
            b = (dB.download(np.uint16, N * K).astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(N, K)
            ref = a @ b.T
            got = (dC.download(np.uint16, M * N).astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(M, N)
            rms = float(np.sqrt((ref ** 2).mean()))
            assert np.all(np.isfinite(got)), (M, N, K)
            assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms), (M, N, K, float(np.abs(got - ref).max()), rms)
            for buf in (dA, dB, dC):
                buf.free()
    dev.gemm_tiling(capi.GEMM_TILING_256)
    a = dev.alloc(1 << 20)
    with pytest.raises(capi.Mi355Error) as e:
        dev.gemm_bf16(a, a, a, 384, 256, 64)
    assert "multiples of 256" in str(e.value)
    a.free()
    dev.gemm_tiling(capi.GEMM_TILING_128)


def test_refuses_what_no_tiling_covers(dev):
    a = dev.alloc(1 << 20)
    for M, N, K in [(64, 256, 64), (256, 192, 64), (256, 256, 32), (0, 256, 64)]:
        with pytest.raises(capi.Mi355Error):
            dev.gemm_bf16(a, a, a, M, N, K)
    with pytest.raises(capi.Mi355Error):
        dev.gemm_tiling(7)
    a.free()
