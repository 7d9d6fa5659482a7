"""GPU parity of the matrix-instruction kernels against the CPU oracle.

Integer kinds are bit-exact.  Floating kinds: |gpu - oracle| <= TOL * iters*sum|a*b| per
element (the oracle accumulates the exact dot product in fp32 once per iteration; the
matrix pipe rounds inside the dot product too, so a relative-to-magnitude bound is the
honest statement)."""
import numpy as np
import pytest

from clpeak_amd import capi
from oracle import pyoracle as orc
from oracle import workloads as wl

pytestmark = pytest.mark.gpu
SEED = wl.DEFAULT_SEED
TOL = 1e-5   # relative to iters * sum|a_k * b_k|


def _run_dense(dev, kind, waves, iters, seed=SEED):
    s = wl.DENSE[kind]
    A, B, sA, sB = wl.dense_inputs(kind, waves, seed)
    dA, dB = dev.from_host(A), dev.from_host(B)
    dsA = dev.from_host(sA) if sA is not None else None
    dsB = dev.from_host(sB) if sB is not None else None
    n_out = waves * 4 * s["M"] * s["N"]
    out = dev.alloc(n_out * 4)
    dev.mfma_dense(kind, dA, dB, dsA, dsB, out, waves, iters)
    is_int = s["fmt"] is None
    got = out.download(np.int32 if is_int else np.float32, n_out)
    ref, ab = orc.mfma_dense(kind, A, B, sA, sB, waves, iters, s["M"] * s["N"], is_int=is_int)
    for b in (dA, dB, dsA, dsB, out):
        if b is not None:
            b.free()
    return got, ref, ab, is_int


def _check(got, ref, ab, is_int, what):
    if is_int:
        assert np.array_equal(got, ref), what
    else:
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
        bound = TOL * ab + 1e-30
        worst = float((err / bound).max())
        assert worst <= 1.0, (what, worst, float(err.max()))
        assert np.count_nonzero(got) > got.size * 0.9, what   # a kernel that wrote nothing must not pass


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_mfma_dense_parity(dev, kind, iters):
    got, ref, ab, is_int = _run_dense(dev, kind, 8, iters)
    _check(got, ref, ab, is_int, (wl.DENSE[kind]["name"], iters))


@pytest.mark.parametrize("kind", sorted(wl.DENSE))
def test_mfma_dense_full_launch_sampled(dev, kind):
    """The configured launch: 2048 waves x 4 chains x 4096 iterations.  The oracle replays
    every wave (seconds) and the whole output is compared."""
    got, ref, ab, is_int = _run_dense(dev, kind, 2048, 4096)
    _check(got, ref, ab, is_int, wl.DENSE[kind]["name"])


def test_mfma_int8_linearity(dev):
    """Size-independent property: n iterations = n x one iteration (exact in int32)."""
    g1, _, _, _ = _run_dense(dev, capi.MFMA_I8_16x16x64, 64, 1)
    gn, _, _, _ = _run_dense(dev, capi.MFMA_I8_16x16x64, 64, 4096)
    assert np.array_equal(gn.astype(np.int64), g1.astype(np.int64) * 4096)


def _run_sparse(dev, kind, waves, iters, seed=SEED):
    s = wl.SPARSE[kind]
    Ac, meta, B = wl.sparse_inputs(kind, waves, seed)
    dA, dM, dB = dev.from_host(Ac), dev.from_host(meta), dev.from_host(B)
    n_out = waves * 4 * 256
    out = dev.alloc(n_out * 4)
    dev.smfmac(kind, dA, dM, dB, out, waves, iters)
    is_int = s["fmt"] is None
    got = out.download(np.int32 if is_int else np.float32, n_out)
    ref, ab = orc.smfmac(kind, Ac, meta, B, waves, iters, is_int=is_int)
    for b in (dA, dM, dB, out):
        b.free()
    return got, ref, ab, is_int


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
@pytest.mark.parametrize("iters", [1, 13, 4096])
def test_smfmac_parity(dev, kind, iters):
    got, ref, ab, is_int = _run_sparse(dev, kind, 8, iters)
    _check(got, ref, ab, is_int, (wl.SPARSE[kind]["name"], iters))


@pytest.mark.parametrize("kind", sorted(wl.SPARSE))
def test_smfmac_full_launch(dev, kind):
    got, ref, ab, is_int = _run_sparse(dev, kind, 2048, 4096)
    _check(got, ref, ab, is_int, wl.SPARSE[kind]["name"])
