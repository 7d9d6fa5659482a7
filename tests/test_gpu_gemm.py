"""GPU parity of the hand-written GEMM against the oracle's float64 tiles.

Tolerance (from the workload definition): 2e-2 relative.  Stated precisely: for every
checked element |gpu - ref| <= 2e-2*|ref| + 2e-2*rms(ref tile); the observed error is far
smaller (bf16 output rounding, 2^-9 relative) and is asserted at 1e-2 as well."""
import numpy as np
import pytest

from clpeak_amd import capi
from oracle import pyoracle as orc
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
SEED = wl.DEFAULT_SEED
FP8_SCALE = 448.0   # per-tensor scale: uniform [-1,1) * 448 fills the e4m3 range


@pytest.fixture(autouse=True, scope="module")
def _on_the_256_tiles(dev):
    """This file is about the kernels on 256x256 tiles, also at shapes the library would give to the 128x128 kernel
    (test_gpu_gemm_small.py covers that one and the choice between the two)."""
    dev.gemm_tiling(capi.GEMM_TILING_256)
    yield
    dev.gemm_tiling(capi.GEMM_TILING_AUTO)


def _operands(dev, fp8, M, N, K):
    eb = 1 if fp8 else 2
    dA, dB = dev.alloc(M * K * eb), dev.alloc(N * K * eb)
    if fp8:
        dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, FP8_SCALE)
        dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, FP8_SCALE)
    else:
        dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1)
        dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
    return dA, dB


def _rows(buf, fp8, row0, rows, K):
    """Rows [row0, row0+rows) of a device operand (the fills themselves are checked bit-exact
    against the oracle in test_gpu_basic.py)."""
    eb = 1 if fp8 else 2
    return buf.download(np.uint8 if fp8 else np.uint16, rows * K, offset_bytes=row0 * K * eb)


def _check_tiles(dev, fp8, M, N, K, tiles, tile=128, whole_output_finite=False):
    dA, dB = _operands(dev, fp8, M, N, K)
    dC = dev.alloc(M * N * 2)
    dev._check(dev.lib.mi355_memset(dev.h, dC.ptr, 0xff, M * N * 2))   # NaN pattern: unwritten output shows
    if fp8:
        dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0 / FP8_SCALE, 1.0 / FP8_SCALE)
    else:
        dev.gemm_bf16(dA, dB, dC, M, N, K)
    fmt = orc.FMT_E4M3 if fp8 else orc.FMT_BF16
    scale = 1.0 / (FP8_SCALE * FP8_SCALE) if fp8 else 1.0
    if whole_output_finite:
        c = dC.download(np.uint16, M * N)
        assert not np.any((c & 0x7f80) == 0x7f80), "an element of C was never written"
    worst = 0.0
    for (m0, n0) in tiles:
        a = _rows(dA, fp8, m0, tile, K)
        b = _rows(dB, fp8, n0, tile, K)
        ref = orc.gemm_tile(fmt, a, b, K, K, K, 0, 0, tile, tile, scale)
        got = np.empty((tile, tile), dtype=np.float64)
        for i in range(tile):
            row = dC.download(np.uint16, tile, offset_bytes=((m0 + i) * N + n0) * 2)
            got[i] = (row.astype(np.uint32) << 16).view(np.float32)
        rms = float(np.sqrt((ref ** 2).mean()))
        err = np.abs(got - ref)
        assert np.all(np.isfinite(got)), (m0, n0)
        assert np.all(err <= 2e-2 * np.abs(ref) + 2e-2 * rms), (m0, n0, float(err.max()), rms)
        assert np.all(err <= 1e-2 * np.abs(ref) + 1e-2 * rms), (m0, n0, float(err.max()), rms)
        worst = max(worst, float((err / (np.abs(ref) + rms)).max()))
    for b in (dA, dB, dC):
        b.free()
    return worst


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (512, 768, 384), (2048, 2048, 1024)])
def test_gemm_small_all_tiles(dev, fp8, M, N, K):
    tiles = [(m, n) for m in range(0, M, 128) for n in range(0, N, 128)]
    if len(tiles) > 24:
        rng = np.random.default_rng(1)
        tiles = [tiles[i] for i in rng.choice(len(tiles), 24, replace=False)]
    _check_tiles(dev, fp8, M, N, K, tiles)


@pytest.mark.parametrize("fp8", [False, True])
def test_gemm_8192_sampled_tiles(dev, fp8):
    """M=N=K=8192, 64 randomly sampled 128x128 output tiles against the CPU GEMM."""
    rng = np.random.default_rng(2)
    tiles = [(int(m) * 128, int(n) * 128) for m, n in zip(rng.integers(0, 64, 64), rng.integers(0, 64, 64))]
    _check_tiles(dev, fp8, 8192, 8192, 8192, tiles)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("steps", [1, 2, 3, 4, 5, 6, 7, 11])
def test_gemm_every_short_k_walk(dev, fp8, steps):
    """K walks of 1..7 and 11 steps of 128 bytes: the start fills five ring slots, which with fewer than
    three steps already run into the workgroup's next tile (here: wrap to its only tile), and the first
    step of a tile takes the barrier without a load wait.  One 256x256 tile, all four 128x128 quarters."""
    K = steps * (128 if fp8 else 64)
    _check_tiles(dev, fp8, 256, 256, K, [(0, 0), (0, 128), (128, 0), (128, 128)])


@pytest.mark.parametrize("fp8", [False, True])
def test_gemm_non_square_grid_visits_every_tile_once(dev, fp8):
    """3 x 5 tiles (15 is not a multiple of the 8 XCDs: the plain tile order) and 8 x 2 tiles (the
    XCD-banded order with fewer than 4 tile rows per band): every output tile is written, none twice
    with different data (the output starts as a NaN pattern and every checked tile is finite and right)."""
    for M, N in ((768, 1280), (2048, 512)):
        tiles = [(m, n) for m in range(0, M, 256) for n in range(0, N, 256)]
        _check_tiles(dev, fp8, M, N, 512, tiles)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("steps", [1, 2, 5, 9, 16, 19])
def test_gemm_workgroups_walk_several_tiles(dev, fp8, steps):
    """17 x 16 = 272 tiles on a 256-CU part: workgroups are persistent, 16 of them own two tiles and the
    fetch stream runs through the tile boundary (with 1 and 2 steps per tile it is a whole tile
    or more ahead of the tile being multiplied).  From 8 steps on, every XCD starts its walk along K at a place of
    its own and wraps around inside the tile; an odd number of steps makes a workgroup's second tile start on the
    other copy of the step.  Every 256x256 tile is checked on one 128x128 quarter,
    and no element of C keeps the NaN pattern it started with."""
    M, N, K = 17 * 256, 16 * 256, steps * (128 if fp8 else 64)
    assert (M // 256) * (N // 256) > dev.props.num_cus
    tiles = [(m + 128 * ((m // 256 + n // 256) % 2), n + 128 * ((m // 256) % 2)) for m in range(0, M, 256) for n in range(0, N, 256)]
    _check_tiles(dev, fp8, M, N, K, tiles, whole_output_finite=True)


@pytest.mark.parametrize("M, N, K", [(4096, 4096, 128), (4096, 8192, 128), (8192, 4096, 384), (4096, 4096, 19 * 128)])
def test_gemm_rounds_of_16x16_tiles(dev, M, N, K):
    """Grids whose sides are multiples of 16 tiles on a 256-CU part: a round of the part is a square of 16 x 16
    tiles, the squares in serpentine order (one, two side by side, two on top of each other).  Every tile is
    checked on one 128x128 quarter and no element of C keeps the NaN pattern it started with; the int8 product
    of the same shape is compared whole, bit for bit, with an exact numpy product."""
    if dev.props.num_cus != 256:
        pytest.skip("the square rounds are the tile order of a 256-CU part")
    tiles = [(m + 128 * ((m // 256 + n // 256) % 2), n + 128 * ((m // 256) % 2)) for m in range(0, M, 256) for n in range(0, N, 256)]
    _check_tiles(dev, False, M, N, K, tiles, whole_output_finite=True)
    dA, dB, dC = dev.alloc(M * K), dev.alloc(N * K), dev.alloc(M * N * 4)
    dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
    dev.memset(dC, 0xff)
    dev.gemm_i8(dA, dB, dC, M, N, K)
    a = dA.download(np.int8, M * K).reshape(M, K).astype(np.float64)
    b = dB.download(np.int8, N * K).reshape(N, K).astype(np.float64)
    want = (a @ b.T).astype(np.int32)            # |sum| <= 64 K: exact in float64
    got = dC.download(np.int32, M * N).reshape(M, N)
    assert np.array_equal(got, want)
    for buf in (dA, dB, dC):
        buf.free()


# --- the other operand types of the same two kernels -------------------------------------------------
E5M2_SCALE = 57344.0


def _check_kind(dev, kind, M, N, K, tiles, tile=128):
    """kind in f16 / i8 / e5m2 (an e5m2 A against an e4m3 B).  int8 is compared bit for bit."""
    eb = 2 if kind == "f16" else 1
    dA, dB = dev.alloc(M * K * eb), dev.alloc(N * K * eb)
    dC = dev.alloc(M * N * (4 if kind == "i8" else 2))
    dev.memset(dC, 0xff)
    if kind == "f16":
        dev.fill_f16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1)
        dev.fill_f16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
        dev.gemm_f16(dA, dB, dC, M, N, K)
        fa = fb = orc.FMT_F16; scale = 1.0
    elif kind == "i8":
        dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A)
        dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
        dev.gemm_i8(dA, dB, dC, M, N, K)
        fa = fb = orc.FMT_I8; scale = 1.0
    else:
        dev.fill_fp8_e5m2(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, E5M2_SCALE)
        dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, FP8_SCALE)
        dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1.0 / E5M2_SCALE, 1.0 / FP8_SCALE)
        fa, fb = orc.FMT_E5M2, orc.FMT_E4M3; scale = 1.0 / (E5M2_SCALE * FP8_SCALE)
    in_dt = np.uint16 if eb == 2 else np.uint8
    for (m0, n0) in tiles:
        a = dA.download(in_dt, tile * K, offset_bytes=m0 * K * eb)
        b = dB.download(in_dt, tile * K, offset_bytes=n0 * K * eb)
        ref = orc.gemm_tile2(fa, fb, a, b, K, K, K, 0, 0, tile, tile, scale)
        got = np.empty((tile, tile), dtype=np.float64)
        for i in range(tile):
            if kind == "i8":
                got[i] = dC.download(np.int32, tile, offset_bytes=((m0 + i) * N + n0) * 4)
            elif kind == "f16":
                got[i] = dC.download(np.float16, tile, offset_bytes=((m0 + i) * N + n0) * 2)
            else:
                row = dC.download(np.uint16, tile, offset_bytes=((m0 + i) * N + n0) * 2)
                got[i] = (row.astype(np.uint32) << 16).view(np.float32)
        assert np.all(np.isfinite(got)), (m0, n0)
        if kind == "i8":
            assert np.array_equal(got, ref), (m0, n0)      # integers: exact in double, exact on the GPU
        else:
            rms = float(np.sqrt((ref ** 2).mean()))
            err = np.abs(got - ref)
            assert np.all(err <= 1e-2 * np.abs(ref) + 1e-2 * rms), (m0, n0, float(err.max()), rms)
    for b in (dA, dB, dC):
        b.free()


@pytest.mark.parametrize("kind", ["f16", "i8", "e5m2"])
@pytest.mark.parametrize("steps", [1, 2, 3, 4, 5, 9])
def test_gemm_other_types_short_walks(dev, kind, steps):
    K = steps * (64 if kind == "f16" else 128)
    _check_kind(dev, kind, 256, 256, K, [(0, 0), (0, 128), (128, 0), (128, 128)])


@pytest.mark.parametrize("kind", ["f16", "i8", "e5m2"])
def test_gemm_other_types_8192_sampled_tiles(dev, kind):
    rng = np.random.default_rng(3)
    tiles = [(int(m) * 128, int(n) * 128) for m, n in zip(rng.integers(0, 64, 12), rng.integers(0, 64, 12))]
    _check_kind(dev, kind, 8192, 8192, 8192, tiles)


def _decode(fmt, codes):
    """Codes of one of the oracle's formats as float64 (through the oracle's own decoder, which the CPU tests pin)."""
    return orc.decode(fmt, codes).astype(np.float64)


@pytest.mark.parametrize("kind", ["bf16", "f16", "e4m3", "e5m2", "i8", "mx"])
def test_gemm_random_shapes_every_element(dev, kind):
    """Six seeded shapes (tile grids from 1 x 1 to 6 x 5, K walks of 1 to 40 steps, mostly odd): the WHOLE of C against a
    numpy float64 product of the decoded operands.  Catches what sampled tiles cannot: a tile or a K step visited twice
    or never, anywhere in the grid."""
    rng = np.random.default_rng(11)
    eb = 2 if kind in ("bf16", "f16") else 1
    for _ in range(6):
        M, N = 256 * int(rng.integers(1, 7)), 256 * int(rng.integers(1, 6))
        K = int(rng.integers(1, 41)) * (128 // eb)
        if kind == "mx":
            _check_mx_whole(dev, M, N, 2 * K)
            continue
        dA, dB, dC = dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * (4 if kind == "i8" else 2))
        dev.memset(dC, 0xff)
        if kind == "bf16":
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            dev.gemm_bf16(dA, dB, dC, M, N, K); fmt, scale = orc.FMT_BF16, 1.0
        elif kind == "f16":
            dev.fill_f16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_f16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            dev.gemm_f16(dA, dB, dC, M, N, K); fmt, scale = orc.FMT_F16, 1.0
        elif kind == "e4m3":
            dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, FP8_SCALE); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, FP8_SCALE)
            dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0 / FP8_SCALE, 1.0 / FP8_SCALE); fmt, scale = orc.FMT_E4M3, 1.0 / (FP8_SCALE * FP8_SCALE)
        elif kind == "e5m2":   # e5m2 A times e4m3 B, as the reference's row
            dev.fill_fp8_e5m2(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, 57344.0); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, FP8_SCALE)
            dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1.0 / 57344.0, 1.0 / FP8_SCALE); fmt, scale = orc.FMT_E5M2, 1.0 / (57344.0 * FP8_SCALE)
        else:
            dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
            dev.gemm_i8(dA, dB, dC, M, N, K); fmt, scale = None, 1.0
        if kind == "i8":
            a = dA.download(np.int8, M * K).astype(np.float64).reshape(M, K)
            b = dB.download(np.int8, N * K).astype(np.float64).reshape(N, K)
        else:
            in_dt = np.uint16 if eb == 2 else np.uint8
            codes = np.arange(1 << (8 * eb), dtype=np.uint32)
            table = _decode(fmt, codes)            # every code of the format once, then a lookup
            a = table[dA.download(in_dt, M * K)].reshape(M, K)
            b = (_decode(orc.FMT_E4M3, codes) if kind == "e5m2" else table)[dB.download(in_dt, N * K)].reshape(N, K)
        ref = (a @ b.T) * scale
        if kind == "i8":
            got = dC.download(np.int32, M * N).reshape(M, N).astype(np.float64)
            assert np.array_equal(got, ref), (M, N, K)
        else:
            raw = dC.download(np.uint16, M * N)
            got = (raw.view(np.float16) if kind == "f16" else (raw.astype(np.uint32) << 16).view(np.float32)).astype(np.float64).reshape(M, N)
            rms = float(np.sqrt((ref ** 2).mean()))
            assert np.all(np.isfinite(got)), (M, N, K)
            assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms), (M, N, K, float(np.abs(got - ref).max()), rms)
        for buf in (dA, dB, dC):
            buf.free()


# --- fp32 and fp64: the accumulation type is the operand type ---------------------------------------------
def _check_wide(dev, kind, M, N, K, tiles, tile=128):
    """kind in f32 / f64.  Bar: |gpu - ref| <= 4 sqrt(K) eps (|ref| + rms(ref tile)), eps = 2^-24 / 2^-53: K
    roundings of a running sum of the size of the result, adding up like a random walk, times four.  The
    reference sum runs in long double."""
    eb, dt, eps = (4, np.float32, 2.0 ** -24) if kind == "f32" else (8, np.float64, 2.0 ** -53)
    dA, dB, dC = dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * eb)
    dev.memset(dC, 0xff)
    if kind == "f32":
        dev.fill_f32(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1)
        dev.fill_f32(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
        dev.gemm_f32(dA, dB, dC, M, N, K)
    else:
        dev.fill_f64(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1)
        dev.fill_f64(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
        dev.gemm_f64(dA, dB, dC, M, N, K)
    fmt = orc.FMT_F32 if kind == "f32" else orc.FMT_F64
    worst = 0.0
    for (m0, n0) in tiles:
        a = dA.download(dt, tile * K, offset_bytes=m0 * K * eb)
        b = dB.download(dt, tile * K, offset_bytes=n0 * K * eb)
        ref = orc.gemm_tile2(fmt, fmt, a, b, K, K, K, 0, 0, tile, tile, 1.0)
        got = np.empty((tile, tile), dtype=np.float64)
        for i in range(tile):
            got[i] = dC.download(dt, tile, offset_bytes=((m0 + i) * N + n0) * eb)
        assert np.all(np.isfinite(got)), (m0, n0)
        rms = float(np.sqrt((ref ** 2).mean()))
        err = np.abs(got - ref)
        bound = 4.0 * np.sqrt(K) * eps * (np.abs(ref) + rms)
        assert np.all(err <= bound), (m0, n0, float((err / bound).max()))
        worst = max(worst, float((err / bound).max()))
    for b in (dA, dB, dC):
        b.free()
    return worst


def test_fill_f64_is_the_fp32_stream_widened(dev):
    n = (1 << 16) + 5
    buf = dev.alloc(n * 8)
    for dist in (capi.DIST_U01, capi.DIST_UPM1):
        dev.fill_f64(buf, n, SEED, wl.STREAM_GEMM_A, dist)
        got = buf.download(np.float64, n)
        assert np.array_equal(got, orc.fill_f32(n, SEED, wl.STREAM_GEMM_A, dist).astype(np.float64))
    buf.free()


@pytest.mark.parametrize("kind", ["f32", "f64"])
@pytest.mark.parametrize("steps", [1, 2, 3, 4, 5, 9])
def test_gemm_wide_types_short_walks(dev, kind, steps):
    K = steps * (32 if kind == "f32" else 16)
    _check_wide(dev, kind, 256, 256, K, [(0, 0), (0, 128), (128, 0), (128, 128)])


@pytest.mark.parametrize("kind", ["f32", "f64"])
def test_gemm_wide_types_grids_and_full_size(dev, kind):
    """Non-square tile grids (every tile checked), more tiles than CUs with a short K, and 8192^3 on sampled tiles."""
    for M, N in ((768, 1280), (2048, 512)):
        _check_wide(dev, kind, M, N, 256, [(m, n) for m in range(0, M, 128) for n in range(0, N, 128)])
    _check_wide(dev, kind, 17 * 256, 16 * 256, 64, [(m, n + 128 * ((m // 256) % 2)) for m in range(0, 17 * 256, 256) for n in range(0, 16 * 256, 256)])
    rng = np.random.default_rng(5)
    tiles = [(int(m) * 128, int(n) * 128) for m, n in zip(rng.integers(0, 64, 8), rng.integers(0, 64, 8))]
    _check_wide(dev, kind, 8192, 8192, 8192, tiles)


# --- block-scaled FP4 ----------------------------------------------------------------------------------
def _check_mx(dev, M, N, K, tiles, tile=128, whole_output_finite=False):
    dA, dB = dev.alloc(M * K // 2), dev.alloc(N * K // 2)
    dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
    dC = dev.alloc(M * N * 2)
    dev.memset(dC, 0xff)
    dev.fill_bytes(dA, M * K // 2, SEED, wl.STREAM_GEMM_A, 0, 256)        # two uniformly random e2m1 codes per byte
    dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
    dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9)       # 2^-4 .. 2^4
    dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
    dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K)
    if whole_output_finite:
        c = dC.download(np.uint16, M * N)
        assert not np.any((c & 0x7f80) == 0x7f80), "an element of C was never written"
    for (m0, n0) in tiles:
        a = dA.download(np.uint8, tile * K // 2, offset_bytes=m0 * K // 2)
        b = dB.download(np.uint8, tile * K // 2, offset_bytes=n0 * K // 2)
        sa = dSA.download(np.uint8, tile * K // 32, offset_bytes=m0 * K // 32)
        sb = dSB.download(np.uint8, tile * K // 32, offset_bytes=n0 * K // 32)
        ref = orc.gemm_mx_tile(a, b, sa, sb, K, 0, 0, tile, tile)
        got = np.empty((tile, tile), dtype=np.float64)
        for i in range(tile):
            row = dC.download(np.uint16, tile, offset_bytes=((m0 + i) * N + n0) * 2)
            got[i] = (row.astype(np.uint32) << 16).view(np.float32)
        rms = float(np.sqrt((ref ** 2).mean()))
        err = np.abs(got - ref)
        assert np.all(np.isfinite(got)), (m0, n0)
        assert np.all(err <= 1e-2 * np.abs(ref) + 1e-2 * rms), (m0, n0, float(err.max()), rms)
    for b in (dA, dB, dSA, dSB, dC):
        b.free()


def _check_mx_whole(dev, M, N, K):
    """The block-scaled FP4 product, the whole of C against a numpy float64 product of decoded codes times 2^(scale - 127)
    (low nibble = even element; one scale byte per 32 elements of a row; the oracle's tile routine, which the CPU tests
    pin, says the same on the sampled tiles of the other tests)."""
    dA, dB = dev.alloc(M * K // 2), dev.alloc(N * K // 2)
    dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
    dC = dev.alloc(M * N * 2)
    dev.memset(dC, 0xff)
    dev.fill_bytes(dA, M * K // 2, SEED, wl.STREAM_GEMM_A, 0, 256); dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
    dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9); dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
    dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K)
    e2m1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float64)
    e2m1 = np.concatenate([e2m1, -e2m1])

    def operand(buf, sbuf, rows):
        raw = buf.download(np.uint8, rows * K // 2).reshape(rows, K // 2)
        x = np.empty((rows, K), dtype=np.float64)
        x[:, 0::2], x[:, 1::2] = e2m1[raw & 15], e2m1[raw >> 4]
        sc = np.exp2(sbuf.download(np.uint8, rows * K // 32).astype(np.float64) - 127.0).reshape(rows, K // 32)
        return x * np.repeat(sc, 32, axis=1)

    ref = operand(dA, dSA, M) @ operand(dB, dSB, N).T
    got = (dC.download(np.uint16, M * N).astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(M, N)
    rms = float(np.sqrt((ref ** 2).mean()))
    assert np.all(np.isfinite(got)), (M, N, K)
    assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms), (M, N, K, float(np.abs(got - ref).max()), rms)
    for b in (dA, dB, dSA, dSB, dC):
        b.free()


def test_fill_bytes_bit_exact(dev):
    n = (1 << 16) + 3
    buf = dev.alloc(n)
    for lo, span in ((0, 256), (123, 9), (7, 1)):
        dev.fill_bytes(buf, n, SEED, wl.STREAM_SCALE_A, lo, span)
        got = buf.download(np.uint8, n)
        assert np.array_equal(got, orc.fill_bytes(n, SEED, wl.STREAM_SCALE_A, lo, span))
        assert got.min() >= lo and got.max() < lo + span
    buf.free()


@pytest.mark.parametrize("steps", [1, 2, 3, 4, 5, 9, 16, 17, 31])
def test_gemm_mxfp4_short_walks(dev, steps):
    """16, 17 and 31 steps: the scale pre-pass works on groups of 16 steps (one full group, a full group and a
    single step, a full group and one that lacks a step)."""
    _check_mx(dev, 256, 256, steps * 256, [(0, 0), (0, 128), (128, 0), (128, 128)])


def test_gemm_mxfp4_grids_and_full_size(dev):
    _check_mx(dev, 768, 512, 1024, [(m, n) for m in range(0, 768, 128) for n in range(0, 512, 128)])
    rng = np.random.default_rng(4)
    tiles = [(int(m) * 128, int(n) * 128) for m, n in zip(rng.integers(0, 64, 8), rng.integers(0, 64, 8))]
    _check_mx(dev, 8192, 8192, 8192, tiles)


@pytest.mark.parametrize("steps", [1, 2, 5, 9, 16])
def test_gemm_mxfp4_workgroups_walk_several_tiles(dev, steps):
    """272 tiles on a 256-CU part (see test_gemm_workgroups_walk_several_tiles): the A, B and scale streams
    each cross the tile boundary at their own distance ahead of the tile being multiplied."""
    M, N, K = 17 * 256, 16 * 256, steps * 256
    assert (M // 256) * (N // 256) > dev.props.num_cus
    tiles = [(m + 128 * ((m // 256 + n // 256) % 2), n + 128 * ((m // 256) % 2)) for m in range(0, M, 256) for n in range(0, N, 256)]
    _check_mx(dev, M, N, K, tiles, whole_output_finite=True)


@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (768, 512, 17 * 256), (17 * 256, 16 * 256, 2 * 256), (4096, 4096, 4096)])
def test_gemm_mxfp4_prepared_scales_give_the_same_bits(dev, M, N, K):
    """Scales laid out once (mi355_gemm_mxfp4_prepare_scales) and the product on them (mi355_gemm_mxfp4_prepared)
    against the one-call form, which the tests above hold to the oracle: the same bits in every element of C, also on a
    second product with the same prepared scales and new A, and nothing allocated by either call."""
    dA, dB = dev.alloc(M * K // 2), dev.alloc(N * K // 2)
    dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
    prepared = dev.alloc((M + N) * K // 32)
    c_one, c_two = dev.alloc(M * N * 2), dev.alloc(M * N * 2)
    dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
    dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9); dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
    before = dev.scratch_bytes()
    dev.gemm_mxfp4_prepare_scales(dSA, dSB, M, N, K, prepared)
    for salt in (0, 1):
        dev.fill_bytes(dA, M * K // 2, SEED + salt, wl.STREAM_GEMM_A, 0, 256)
        dev.memset(c_two, 0xff)
        dev.gemm_mxfp4_prepared(dA, dB, prepared, c_two, M, N, K)
        assert dev.scratch_bytes() == before
        dev.memset(c_one, 0xff)
        dev.gemm_mxfp4(dA, dB, dSA, dSB, c_one, M, N, K)
        one, two = c_one.download(np.uint16, M * N), c_two.download(np.uint16, M * N)
        assert not np.any((two & 0x7f80) == 0x7f80), "an element of C was never written"
        assert np.array_equal(one, two), salt
    for b in (dA, dB, dSA, dSB, prepared, c_one, c_two):
        b.free()


def test_gemm_mxfp4_refuses_before_it_allocates_or_launches(dev):
    """A call that will be refused (a row of K past the 64 MiB the kernel's offsets reach, a misaligned scale array)
    leaves the handle's scratch as it was: the checks come before the allocation and the pre-pass."""
    small = dev.alloc(1 << 20)
    before = dev.scratch_bytes()
    K = (64 << 20) * 2 + 256           # 64 MiB + 128 bytes per row of two codes per byte
    for call in (lambda: dev.gemm_mxfp4(small, small, small, small, small, 256, 256, K),
                 lambda: dev.gemm_mxfp4_static(small, small, small, small, small, 256, 256, K),
                 lambda: dev.gemm_mxfp4_prepared(small, small, small, small, 256, 256, K)):
        with pytest.raises(capi.Mi355Error) as err:
            call()
        assert err.value.code == capi.ERR_ARG and "at most" in str(err.value)
        assert dev.scratch_bytes() == before
    small.free()


def test_gemm_refuses_rows_longer_than_its_offsets_reach(dev):
    """A lane addresses its wave's 64 rows of a slab with 32-bit offsets: rows of K longer than 64 MiB are refused
    before anything is launched (the buffers here are never touched)."""
    small = dev.alloc(1 << 20)
    K = (64 << 20) // 2 + 64      # bf16: 64 MiB + 128 bytes per row
    with pytest.raises(capi.Mi355Error) as err:
        dev.gemm_bf16(small, small, small, 256, 256, K)
    assert err.value.code == capi.ERR_ARG and "at most" in str(err.value)
    small.free()


# --- the reference's own GEMM inputs ---------------------------------------------------------------------
def _bf16_bits_of(x):
    """Nearest-even bf16 code of a float32 value that is finite (numpy only)."""
    u = np.float32(x).view(np.uint32).astype(np.uint64)
    return int(((u + 0x7fff + ((u >> 16) & 1)) >> 16) & 0xffff)


@pytest.mark.parametrize("kind", ["fp32", "fp64", "fp16", "bf16", "int8", "fp8_e4m3", "fp8_e5m2", "mxf4_e2m1"])
def test_gemm_on_the_reference_fills(dev, kind):
    """The reference's GEMM tests run on buffers set to one byte: 0x3f for every type of its rocBLAS test
    (src/rocm/rocblas.cpp:211-212), 0x38 under block scales of 0x7f in its hipBLASLt test
    (src/rocm/hipblaslt_gemm.cpp:272-273, 417-418).  On those inputs every element of C is K x a x b rounded to
    the output type, with a and b the value that byte pattern has in the operand type; for the narrow types the
    fp32 accumulation is exact at this K, so the whole of C is compared bit for bit with that one number."""
    M, N, K = 512, 768, 1024
    ebytes = {"fp32": 4, "fp64": 8, "fp16": 2, "bf16": 2, "int8": 1, "fp8_e4m3": 1, "fp8_e5m2": 1, "mxf4_e2m1": 0.5}[kind]
    obytes = {"fp32": 4, "fp64": 8, "int8": 4}.get(kind, 2)
    byte = 0x3f if kind in ("fp32", "fp64", "fp16", "bf16", "int8") else 0x38
    dA, dB, dC = dev.alloc(int(M * K * ebytes)), dev.alloc(int(N * K * ebytes)), dev.alloc(M * N * obytes)
    dev.memset(dA, byte); dev.memset(dB, byte); dev.memset(dC, 0xff)
    pattern = np.full(8, byte, dtype=np.uint8)
    if kind == "fp32":
        a = float(pattern.view(np.float32)[0])
        dev.gemm_f32(dA, dB, dC, M, N, K)
        got = dC.download(np.float32, M * N)
        assert np.all(got == got[0]) and abs(float(got[0]) - K * a * a) <= 1e-5 * K * a * a, (got[0], K * a * a)
    elif kind == "fp64":
        a = float(pattern.view(np.float64)[0])
        dev.gemm_f64(dA, dB, dC, M, N, K)
        got = dC.download(np.float64, M * N)
        assert np.all(got == got[0]) and abs(float(got[0]) - K * a * a) <= 1e-12 * K * a * a, (got[0], K * a * a)
    elif kind == "int8":
        dev.gemm_i8(dA, dB, dC, M, N, K)
        assert np.all(dC.download(np.int32, M * N) == K * 63 * 63)
    elif kind == "fp16":
        a = float(pattern.view(np.float16)[0])                      # 1855/1024: K*a*a needs 22 bits, exact in fp32
        dev.gemm_f16(dA, dB, dC, M, N, K)
        want = np.float16(np.float32(K * a * a))
        assert np.float32(K * a * a) == K * a * a
        assert np.all(dC.download(np.uint16, M * N) == want.view(np.uint16)), want
    else:
        if kind == "bf16":
            a = b = float((pattern.view(np.uint16)[:1].astype(np.uint32) << 16).view(np.float32)[0])   # 191/256
            dev.gemm_bf16(dA, dB, dC, M, N, K)
            total = K * a * b
        elif kind == "fp8_e4m3":
            dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0, 1.0)        # 0x38 is 1.0 as e4m3
            total = K * 1.0
        elif kind == "fp8_e5m2":
            dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1.0, 1.0)        # ... and 0.5 as e5m2 (the A operand of this row)
            total = K * 0.5
        else:
            dSA, dSB = dev.alloc(M * K // 32), dev.alloc(N * K // 32)
            dev.memset(dSA, 0x7f); dev.memset(dSB, 0x7f)
            dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K)
            # byte 0x38: even k holds code 8 (-0), odd k code 3 (1.5); scales 2^0
            total = (K // 2) * 1.5 * 1.5
            dSA.free(); dSB.free()
        assert np.float32(total) == total
        assert np.all(dC.download(np.uint16, M * N) == _bf16_bits_of(total)), (kind, total)
    for b in (dA, dB, dC):
        b.free()


@pytest.mark.parametrize("kind", ["bf16", "e4m3", "i8", "mx"])
def test_gemm_same_bits_from_launch_to_launch(dev, kind):
    """4096^3 (256 tiles: every workgroup busy, 64 / 32 / 16 K steps per tile), launched three times back to back, six
    times over: C is the same bits every time.  Nothing in the kernel depends on timing unless a wave reads a slab or
    a fragment before it has landed, or a slot is overwritten while another wave still reads it; such a launch would
    differ from its neighbours now and then."""
    import zlib
    M = N = K = 4096
    eb, cb = (2 if kind == "bf16" else 1), (4 if kind == "i8" else 2)
    if kind == "mx":
        bufs = [dev.alloc(M * K // 2), dev.alloc(N * K // 2), dev.alloc(M * N * 2), dev.alloc(M * K // 32), dev.alloc(N * K // 32)]
        dA, dB, dC, dSA, dSB = bufs
        dev.fill_bytes(dA, M * K // 2, SEED, wl.STREAM_GEMM_A, 0, 256); dev.fill_bytes(dB, N * K // 2, SEED, wl.STREAM_GEMM_B, 0, 256)
        dev.fill_bytes(dSA, M * K // 32, SEED, wl.STREAM_SCALE_A, 123, 9); dev.fill_bytes(dSB, N * K // 32, SEED, wl.STREAM_SCALE_B, 123, 9)
        launch = lambda: dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K)
    else:
        bufs = [dev.alloc(M * K * eb), dev.alloc(N * K * eb), dev.alloc(M * N * cb)]
        dA, dB, dC = bufs
        if kind == "bf16":
            dev.fill_bf16(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1); dev.fill_bf16(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1)
            launch = lambda: dev.gemm_bf16(dA, dB, dC, M, N, K)
        elif kind == "e4m3":
            dev.fill_fp8_e4m3(dA, M * K, SEED, wl.STREAM_GEMM_A, capi.DIST_UPM1, FP8_SCALE); dev.fill_fp8_e4m3(dB, N * K, SEED, wl.STREAM_GEMM_B, capi.DIST_UPM1, FP8_SCALE)
            launch = lambda: dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0 / FP8_SCALE, 1.0 / FP8_SCALE)
        else:
            dev.fill_i8(dA, M * K, SEED, wl.STREAM_GEMM_A); dev.fill_i8(dB, N * K, SEED, wl.STREAM_GEMM_B)
            launch = lambda: dev.gemm_i8(dA, dB, dC, M, N, K)
    seen = set()
    for _ in range(6):
        dev.memset(dC, 0xff)
        for _ in range(3):
            launch()
        dev.sync()
        seen.add(zlib.crc32(dC.download(np.uint8, M * N * cb).tobytes()))
    assert len(seen) == 1, seen
    for b in bufs:
        b.free()
