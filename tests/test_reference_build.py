"""The restated calibration helpers and thread pool against the reference's own compiled code.

oracle/ref.mk compiles src/common/common.cpp and src/cpu/thread_pool.cpp of the reference where they
lie (the only two files of this path that build without its build system) into
oracle/_ref/libclpeak_ref.so.  Where that library exists, the host layer's and the CPU harness's
restatements are compared with it call by call; elsewhere these tests skip.
"""
import ctypes as C
import os
import random

import numpy as np
import pytest

from oracle import pyoracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFLIB = os.path.join(ROOT, "oracle", "_ref", "libclpeak_ref.so")
HOSTLIB = os.path.join(ROOT, "clpeak_amd", "libclpeak_host.so")

pytestmark = pytest.mark.skipif(not os.path.exists(REFLIB), reason="reference build (oracle/_ref) not present")


@pytest.fixture(scope="module")
def ref():
    L = C.CDLL(REFLIB)
    L.ref_pick_iters.argtypes = [C.c_double, C.c_uint, C.c_uint, C.c_uint]; L.ref_pick_iters.restype = C.c_uint
    L.ref_target_global_threads.argtypes = [C.c_uint]; L.ref_target_global_threads.restype = C.c_ulonglong
    L.ref_config_for_device.argtypes = [C.c_uint, C.POINTER(C.c_ulonglong)]; L.ref_config_for_device.restype = None
    L.ref_pool_create.argtypes = [C.c_int]; L.ref_pool_create.restype = C.c_void_p
    L.ref_pool_destroy.argtypes = [C.c_void_p]; L.ref_pool_destroy.restype = None
    L.ref_pool_max_threads.argtypes = [C.c_void_p]; L.ref_pool_max_threads.restype = C.c_int
    L.ref_pool_count.argtypes = [C.c_void_p, C.c_int, C.c_ulonglong, C.c_void_p]; L.ref_pool_count.restype = None
    L.ref_lmem_reps.restype = C.c_uint
    L.ref_cancel_requested.restype = C.c_int
    return L


@pytest.fixture(scope="module")
def host():
    L = C.CDLL(HOSTLIB)
    L.clpeak_host_pick_iters.argtypes = [C.c_double, C.c_uint, C.c_uint, C.c_uint]; L.clpeak_host_pick_iters.restype = C.c_uint
    L.clpeak_host_target_global_threads.argtypes = [C.c_uint]; L.clpeak_host_target_global_threads.restype = C.c_ulonglong
    L.clpeak_host_config_for_device.argtypes = [C.c_uint, C.POINTER(C.c_ulonglong)]; L.clpeak_host_config_for_device.restype = None
    L.clpeak_host_cancel_requested.restype = C.c_int
    return L


def test_pick_iters_agrees_everywhere(ref, host):
    rng = random.Random(7)
    cases = [(0.0, 0, 0, 1), (1e-9, 500000, 0, 10000), (1e9, 1, 0, 10000), (1.0, 0, 0, 100000000), (2.5, 1000, 9, 3)]
    for _ in range(5000):
        cases.append((10 ** rng.uniform(-3, 7), rng.choice([0, 1, 1000, 500000, 2000000, rng.randrange(1, 1 << 31)]),
                      rng.choice([0, 0, 0, rng.randrange(1, 100000)]), rng.choice([1, 10000, 100000000, rng.randrange(1, 1 << 31)])))
    for c in cases:
        want = ref.ref_pick_iters(*c)
        assert host.clpeak_host_pick_iters(*c) == want, c
        assert orc.pick_iters(*c) == want, c


def test_launch_width_and_device_config_agree(ref, host):
    for cus in list(range(0, 64)) + [104, 228, 256, 304, 1024, 65535]:
        assert host.clpeak_host_target_global_threads(cus) == ref.ref_target_global_threads(cus)
    for dtype in (1, 2, 4):
        a, b = (C.c_ulonglong * 6)(), (C.c_ulonglong * 6)()
        ref.ref_config_for_device(dtype, a)
        host.clpeak_host_config_for_device(dtype, b)
        assert list(a) == list(b), dtype
    assert ref.ref_lmem_reps() == 64      # repetitions the LDS row is priced with


def test_pool_dispatch_contract_agrees(ref):
    n_max = min(4, len(os.sched_getaffinity(0)))
    rp = ref.ref_pool_create(n_max)
    assert ref.ref_pool_max_threads(rp) == n_max
    with orc.CpuPool(n_max) as mine:
        for n in (-3, 0, 1, 2, n_max, n_max + 9):
            want = np.zeros(n_max, dtype=np.uint64)
            ref.ref_pool_count(rp, n, 11, want.ctypes.data)
            got = mine.count(n, 11)
            assert (got == want).all(), (n, got, want)
    ref.ref_pool_destroy(rp)


def test_cancel_flag_behaves_alike(ref, host):
    for lib, req, reset, get in ((ref, "ref_request_cancel", "ref_reset_cancel", "ref_cancel_requested"),
                                 (host, "clpeak_host_request_cancel", "clpeak_host_reset_cancel", "clpeak_host_cancel_requested")):
        getattr(lib, reset)()
        assert getattr(lib, get)() == 0
        getattr(lib, req)()
        getattr(lib, req)()
        assert getattr(lib, get)() == 1
        getattr(lib, reset)()
        assert getattr(lib, get)() == 0


def test_restated_populate_is_the_reference_s(ref):
    """The harness's buffer fill against the reference's compiled populate() (src/common/common.cpp:76-95),
    bit for bit, over a length that is not a multiple of anything."""
    n = 100_003
    ref.ref_populate.argtypes = [C.c_void_p, C.c_ulonglong]; ref.ref_populate.restype = None
    L = orc.lib()
    L.cpuh_populate.argtypes = [C.c_void_p, C.c_ulonglong]; L.cpuh_populate.restype = None
    a, b = np.zeros(n, dtype=np.float32), np.zeros(n, dtype=np.float32)
    ref.ref_populate(a.ctypes.data, n)
    L.cpuh_populate(b.ctypes.data, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
