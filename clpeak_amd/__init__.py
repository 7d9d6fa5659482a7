"""MI355X (gfx950) compute backend for clpeak: Python view of the C ABI.

The product is the shared library ``libclpeak_mi355.so`` (HIP kernels + C ABI, built
from ``clpeak_amd/csrc``) and the C++ host layer in ``clpeak_amd/host``.  This package
only binds the C ABI with ctypes so that tests and the benchmark driver can call it;
it contains no arithmetic of its own and no CPU fallback: if the library is missing,
importing :mod:`clpeak_amd.capi` raises.
"""
