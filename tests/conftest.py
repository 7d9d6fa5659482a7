import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    """The opened GPU, through the C ABI.  No fallback: a missing library or GPU is an error."""
    from clpeak_amd import capi
    d = capi.Device(0)
    yield d
    d.close()


def ensure_host_double():
    """Build the host layer's test target (tests/host_double: the host sources against a pretend device) when
    it is not there yet."""
    import subprocess
    d = os.path.join(ROOT, "tests", "host_double")
    if all(os.path.exists(os.path.join(d, f)) for f in ("clpeak-mi355-double", "libclpeak_host_double.so")):
        return
    r = subprocess.run(["make", "-C", d, "-j8"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("tests/host_double did not build:\n" + r.stdout[-4000:])
