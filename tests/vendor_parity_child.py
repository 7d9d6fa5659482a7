"""Child process of test_zy_vendor_parity.py: this library's GEMM next to the vendor library's (what the reference's
rocblas-fp / hipblaslt-fp8 / rocblas-int rows call, reached through torch.matmul, torch._scaled_mm and torch._int_mm) on
the SAME operands, every element of C.  A process of its own: torch brings a HIP runtime that has to be the one to
initialise the device in its process, so torch is imported first and this library is loaded behind it.

Prints "LOADED" once torch has initialised the device (the parent tells a slow import from a hung product by it), then
one line per kind, "<kind> ok ..." or "<kind> MISMATCH ...", or "SKIP <reason>"; exit status 0 unless a kind mismatches."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

try:
    import torch
    torch.cuda.init()
except Exception as e:   # no torch, or no device for it
    print(f"SKIP torch not usable: {e!r}")
    sys.exit(0)
print("LOADED", flush=True)
import numpy as np  # noqa: E402

from clpeak_amd import capi  # noqa: E402

M, N, K = 1024, 768, 4096
g = torch.Generator(device="cuda")
g.manual_seed(20240607)
dev = capi.Device(0)
one = torch.ones((), device="cuda")
failed = 0


def host_bytes(t):
    return t.contiguous().view(torch.uint8).cpu().numpy().reshape(-1)


def report(kind, got, ref, exact, tol=1e-2):
    global failed
    if exact:
        ok, worst = bool(np.array_equal(got, ref)), float(np.abs(got - ref).max())
    else:
        rms = float(np.sqrt((ref ** 2).mean()))
        err = np.abs(got - ref)
        ok, worst = bool(np.all(np.isfinite(got)) and np.all(err <= tol * np.abs(ref) + tol * rms)), float(err.max() / rms)
    failed += not ok
    print(f"{kind} {'ok' if ok else 'MISMATCH'} worst {'difference' if exact else 'error / rms'} {worst:.3g}", flush=True)


def as_f64(raw_u16, half):
    return (raw_u16.view(np.float16) if half else (raw_u16.astype(np.uint32) << 16).view(np.float32)).astype(np.float64)


for kind in ("bf16", "f16", "e4m3", "e5m2", "i8", "mx", "f32", "f64"):
    try:
        if kind in ("bf16", "f16"):
            dt = torch.bfloat16 if kind == "bf16" else torch.float16
            A = (torch.rand(M, K, device="cuda", generator=g) * 2 - 1).to(dt)
            B = (torch.rand(N, K, device="cuda", generator=g) * 2 - 1).to(dt)
            ref = torch.matmul(A, B.t())
        elif kind == "e4m3":
            A = ((torch.rand(M, K, device="cuda", generator=g) * 2 - 1) * 448).to(torch.float8_e4m3fn)
            B = ((torch.rand(N, K, device="cuda", generator=g) * 2 - 1) * 448).to(torch.float8_e4m3fn)
            ref = torch._scaled_mm(A, B.t(), scale_a=one / 448, scale_b=one / 448, out_dtype=torch.bfloat16)
        elif kind == "e5m2":   # e5m2 A times e4m3 B, the reference's second fp8 row
            A = ((torch.rand(M, K, device="cuda", generator=g) * 2 - 1) * 57344).to(torch.float8_e5m2)
            B = ((torch.rand(N, K, device="cuda", generator=g) * 2 - 1) * 448).to(torch.float8_e4m3fn)
            ref = torch._scaled_mm(A, B.t(), scale_a=one / 57344, scale_b=one / 448, out_dtype=torch.bfloat16)
        elif kind in ("f32", "f64"):
            dt = torch.float32 if kind == "f32" else torch.float64
            A = (torch.rand(M, K, device="cuda", generator=g, dtype=dt) * 2 - 1)
            B = (torch.rand(N, K, device="cuda", generator=g, dtype=dt) * 2 - 1)
            ref = torch.matmul(A, B.t())
        elif kind == "i8":
            A = torch.randint(-128, 128, (M, K), device="cuda", dtype=torch.int8, generator=g)
            B = torch.randint(-128, 128, (N, K), device="cuda", dtype=torch.int8, generator=g)
            ref = torch._int_mm(A, B.t())
        else:
            A = torch.randint(0, 256, (M, K // 2), device="cuda", dtype=torch.uint8, generator=g).view(torch.float4_e2m1fn_x2)
            B = torch.randint(0, 256, (N, K // 2), device="cuda", dtype=torch.uint8, generator=g).view(torch.float4_e2m1fn_x2)
            SA = torch.randint(123, 132, (M, K // 32), device="cuda", dtype=torch.uint8, generator=g)
            SB = torch.randint(123, 132, (N, K // 32), device="cuda", dtype=torch.uint8, generator=g)
            ref = torch._scaled_mm(A, B.t(), scale_a=SA.view(torch.float8_e8m0fnu), scale_b=SB.view(torch.float8_e8m0fnu),
                                   out_dtype=torch.bfloat16)
        torch.cuda.synchronize()
    except Exception as e:
        print(f"{kind} SKIP the vendor product is not available here: {e!r}"[:300], flush=True)
        continue
    dA, dB = dev.from_host(host_bytes(A)), dev.from_host(host_bytes(B))
    dC = dev.alloc(M * N * {"i8": 4, "f32": 4, "f64": 8}.get(kind, 2))
    dev.memset(dC, 0xff)
    if kind == "bf16":
        dev.gemm_bf16(dA, dB, dC, M, N, K)
    elif kind == "f16":
        dev.gemm_f16(dA, dB, dC, M, N, K)
    elif kind == "e4m3":
        dev.gemm_fp8_e4m3(dA, dB, dC, M, N, K, 1.0 / 448, 1.0 / 448)
    elif kind == "e5m2":
        dev.gemm_fp8_e5m2(dA, dB, dC, M, N, K, 1.0 / 57344, 1.0 / 448)
    elif kind == "i8":
        dev.gemm_i8(dA, dB, dC, M, N, K)
    elif kind == "f32":
        dev.gemm_f32(dA, dB, dC, M, N, K)
    elif kind == "f64":
        dev.gemm_f64(dA, dB, dC, M, N, K)
    else:
        dSA, dSB = dev.from_host(host_bytes(SA)), dev.from_host(host_bytes(SB))
        dev.gemm_mxfp4(dA, dB, dSA, dSB, dC, M, N, K)
    dev.sync()
    if kind == "i8":
        report(kind, dC.download(np.int32, M * N).astype(np.int64), ref.cpu().numpy().reshape(-1).astype(np.int64), exact=True)
    elif kind in ("f32", "f64"):
        ndt = np.float32 if kind == "f32" else np.float64
        report(kind, dC.download(ndt, M * N).astype(np.float64), ref.cpu().numpy().reshape(-1).astype(np.float64), exact=False,
               tol=1e-5 if kind == "f32" else 1e-13)
    else:
        want = as_f64(host_bytes(ref).view(np.uint16), kind == "f16")
        report(kind, as_f64(dC.download(np.uint16, M * N), kind == "f16"), want, exact=False)
dev.close()
sys.exit(1 if failed else 0)
