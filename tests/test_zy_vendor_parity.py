"""This library's GEMMs against the vendor library's on the same operands.

The reference's GEMM rows call rocBLAS / hipBLASLt (src/rocm/rocblas.cpp:122-342, src/rocm/hipblaslt_gemm.cpp:262-520);
the hand-written kernels take their place, so their results are held to that library's here: torch.matmul,
torch._scaled_mm and torch._int_mm reach the same libraries on this image.  All eight rows (bf16, fp16, fp32, fp64, fp8 e4m3, e5m2 x e4m3, int8, block-scaled
FP4), 1024 x 768 x 4096, every element of C: int8 equal, the 16-bit outputs within 1e-2 (relative to the element and to
the rms of C: the two sum in different orders and round once to the output type), fp32 within 1e-5, fp64 within 1e-13.  The block-scaled FP4 case also says that both read the scale bytes as
plain row-major [rows][K / 32] arrays.

The comparison runs in a child process (tests/vendor_parity_child.py): torch's HIP runtime has to be the one that
initialises the device in its process.  The file sorts behind the other GPU tests because the first import of torch on a
machine can take minutes; when it does, the test is skipped rather than failed (a time limit that strikes after torch
has loaded is a failure)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.timeout(260)
def test_gemm_matches_the_vendor_library_on_the_same_operands():
    """Skipped only when torch itself is slow to load or absent; once the child says LOADED, a time limit is a failure
    (a product that hangs must not read as a skip)."""
    child = subprocess.Popen([sys.executable, "-u", os.path.join(ROOT, "tests", "vendor_parity_child.py")], stdout=subprocess.PIPE,
                             stderr=subprocess.PIPE, text=True)
    import threading
    import time
    lines, errs = [], []
    readers = [threading.Thread(target=lambda: lines.extend(iter(child.stdout.readline, "")), daemon=True),
               threading.Thread(target=lambda: errs.extend(iter(child.stderr.readline, "")), daemon=True)]
    for t in readers:
        t.start()
    t0 = time.time()
    load_limit, run_limit = 120.0, 100.0
    loaded_at = None
    while child.poll() is None:
        now = time.time()
        if loaded_at is None and any(l.startswith(("LOADED", "SKIP")) for l in lines):
            loaded_at = now
        if loaded_at is None and now - t0 > load_limit:
            child.kill()
            child.wait()
            pytest.skip(f"torch took more than {load_limit:.0f} s to load here: no comparison with the vendor library this time")
        if loaded_at is not None and now - loaded_at > run_limit:
            child.kill()
            child.wait()
            pytest.fail(f"the comparison did not finish within {run_limit:.0f} s of torch being loaded: " + " | ".join(l.strip() for l in lines))
        time.sleep(0.2)
    for t in readers:
        t.join(timeout=5)
    lines = [l.strip() for l in lines if l.strip() and not l.startswith("LOADED")]
    if lines and lines[0].startswith("SKIP"):
        pytest.skip(lines[0])
    assert child.returncode == 0, "".join(lines)[-2000:] + "".join(errs)[-2000:]
    verdicts = {l.split()[0]: l.split()[1] for l in lines}
    assert "MISMATCH" not in verdicts.values(), lines
    # the 16-bit and int8 products exist in every hipBLASLt this image could carry; fp8 and FP4 may be skipped by an older one
    for kind in ("bf16", "f16", "i8"):
        assert verdicts.get(kind) == "ok", lines
