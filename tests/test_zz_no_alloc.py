"""The entry point that allocates nothing (mi355_gemm_mxfp4_static) against the one it is a variant of
(mi355_gemm_mxfp4): same inputs, same kernels, so the outputs are compared bit for bit; two calls in a row,
the second on a smaller problem, so that what the first left in the shared static array would show."""
import numpy as np
import pytest

from clpeak_amd import capi
from oracle import pyoracle as orc
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
SEED = wl.DEFAULT_SEED


def _problem(dev, M, N, K, salt):
    bufs = [dev.alloc(M * K // 2), dev.alloc(N * K // 2), dev.alloc(M * K // 32), dev.alloc(N * K // 32)]
    dev.fill_bytes(bufs[0], M * K // 2, SEED + salt, wl.STREAM_GEMM_A, 0, 256)
    dev.fill_bytes(bufs[1], N * K // 2, SEED + salt, wl.STREAM_GEMM_B, 0, 256)
    dev.fill_bytes(bufs[2], M * K // 32, SEED + salt, wl.STREAM_SCALE_A, 123, 9)
    dev.fill_bytes(bufs[3], N * K // 32, SEED + salt, wl.STREAM_SCALE_B, 123, 9)
    return bufs


def _both(dev, M, N, K, salt):
    dA, dB, dSA, dSB = _problem(dev, M, N, K, salt)
    c_ref, c_new = dev.alloc(M * N * 2), dev.alloc(M * N * 2)
    dev.memset(c_ref, 0xff); dev.memset(c_new, 0xff)
    print(f"gemm_mxfp4 {M}x{N}x{K}", flush=True)
    dev.gemm_mxfp4(dA, dB, dSA, dSB, c_ref, M, N, K)
    print(f"gemm_mxfp4_static {M}x{N}x{K}", flush=True)
    dev.gemm_mxfp4_static(dA, dB, dSA, dSB, c_new, M, N, K)
    ref, new = c_ref.download(np.uint16, M * N), c_new.download(np.uint16, M * N)
    assert not np.any((new & 0x7f80) == 0x7f80), "an element of C was never written"
    assert np.array_equal(ref, new)
    # and one tile of it against the oracle, so that "equal" is not "equally wrong"
    t = 128
    a, b = dA.download(np.uint8, t * K // 2), dB.download(np.uint8, t * K // 2)
    sa, sb = dSA.download(np.uint8, t * K // 32), dSB.download(np.uint8, t * K // 32)
    want = orc.gemm_mx_tile(a, b, sa, sb, K, 0, 0, t, t)
    got = (new.reshape(M, N)[:t, :t].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    rms = float(np.sqrt((want ** 2).mean()))
    assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-2 * rms)
    for buf in (dA, dB, dSA, dSB, c_ref, c_new):
        buf.free()


def test_static_entry_point_on_a_fresh_handle_allocates_nothing():
    """A handle that has never run the allocating entry point: the static one must work from the static array alone
    (the handle's scratch stays at 0 bytes, the device's free memory does not move), and its result is the one the
    allocating entry point gives afterwards, and the oracle's."""
    fresh = capi.Device(0)
    try:
        M, N, K = 512, 256, 1024
        dA, dB, dSA, dSB = _problem(fresh, M, N, K, salt=7)
        c_new, c_ref = fresh.alloc(M * N * 2), fresh.alloc(M * N * 2)
        fresh.memset(c_new, 0xff); fresh.memset(c_ref, 0xff)
        fresh.sync()
        assert fresh.scratch_bytes() == 0
        fresh.gemm_mxfp4_static(dA, dB, dSA, dSB, c_new, M, N, K)
        fresh.sync()
        assert fresh.scratch_bytes() == 0, "the entry point that allocates nothing grew the handle's scratch"
        new = c_new.download(np.uint16, M * N)
        assert not np.any((new & 0x7f80) == 0x7f80), "an element of C was never written"
        t = 128
        want = orc.gemm_mx_tile(dA.download(np.uint8, t * K // 2), dB.download(np.uint8, t * K // 2),
                                dSA.download(np.uint8, t * K // 32), dSB.download(np.uint8, t * K // 32), K, 0, 0, t, t)
        got = (new.reshape(M, N)[:t, :t].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        rms = float(np.sqrt((want ** 2).mean()))
        assert np.all(np.abs(got - want) <= 1e-2 * np.abs(want) + 1e-2 * rms)
        fresh.gemm_mxfp4(dA, dB, dSA, dSB, c_ref, M, N, K)          # only now does the handle allocate
        assert fresh.scratch_bytes() == (M + N) * K // 32
        assert np.array_equal(c_ref.download(np.uint16, M * N), new)
        for buf in (dA, dB, dSA, dSB, c_new, c_ref):
            buf.free()
    finally:
        fresh.close()


def test_static_entry_point_matches_two_calls_in_a_row(dev):
    _both(dev, 1024, 768, 2048, salt=0)
    _both(dev, 256, 512, 512, salt=1)      # smaller: the array still holds the first call's scales beyond these
    _both(dev, 8192, 8192, 8192, salt=2)   # the largest problem the static array admits


def test_static_entry_point_refuses_what_does_not_fit(dev):
    M, N, K = 8192, 8192 + 256, 8192
    tiny = dev.alloc(256)
    with pytest.raises(capi.Mi355Error, match="exceed the static scratch"):
        dev.gemm_mxfp4_static(tiny, tiny, tiny, tiny, tiny, M, N, K)
    tiny.free()
