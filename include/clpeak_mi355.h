/*
 * clpeak_mi355.h -- C ABI of the MI355X (gfx950 / CDNA4) compute backend for clpeak.
 *
 * This is the only door through which host code reaches HIP.  Everything is
 * plain C: opaque device handle, raw device pointers, sizes, int status codes.
 * No C++ types, no exceptions, no torch types.  One handle owns one HIP stream;
 * a handle is not thread-safe, different handles may be used from different
 * threads.  Every `*_launch_*`-style entry point ENQUEUES on the handle's stream
 * and returns without waiting; use mi355_sync() or the timer pair to wait.
 *
 * The reference has no C boundary between a backend and HIP (a backend is a C++
 * class that calls hipModuleLaunchKernel itself), so each entry point below
 * cites the reference code whose work it takes over.  Paths are relative to the
 * reference checkout.
 *
 * Status codes: 0 = ok, negative = failure; mi355_last_error() explains the
 * last failure on that handle (or the last handle-less failure when dev==NULL).
 */
#ifndef CLPEAK_MI355_H
#define CLPEAK_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_OK            0
#define MI355_ERR_ARG      (-1)  /* bad argument / shape the kernels do not support */
#define MI355_ERR_HIP      (-2)  /* a HIP runtime call failed */
#define MI355_ERR_NODEV    (-3)  /* no such device */
#define MI355_ERR_ARCH     (-4)  /* device is not gfx950 */
#define MI355_ERR_OOM      (-5)  /* device allocation failed */

typedef struct mi355_dev mi355_dev;

/* Device facts the reference keeps in rocm_device_info_t
 * (include/rocm/rocm_peak.h:23-40, filled in src/rocm/rocm_device.cpp:42-85). */
typedef struct mi355_props {
  char     name[256];            /* hipDeviceProp_t::name */
  char     arch[64];             /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  char     driver_version[32];   /* hipDriverGetVersion as major.minor.patch */
  char     runtime_version[32];  /* hipRuntimeGetVersion as major.minor.patch */
  int32_t  num_cus;
  int32_t  wave_size;
  int32_t  max_threads_per_block;
  int32_t  clock_khz;
  uint64_t total_mem;            /* bytes */
} mi355_props_t;

/* ---- device / memory / timing ------------------------------------------------ */

/* src/rocm/rocm_peak.cpp:32-49 (initRuntime: hipGetDeviceCount). */
int mi355_device_count(int *count);
/* src/rocm/rocm_device.cpp:42-85 (RocmDevice::init: hipSetDevice, props,
 * non-blocking stream).  Refuses anything that is not gfx950. */
int mi355_open(int ordinal, mi355_dev **out);
/* src/rocm/rocm_device.cpp:87-98 (RocmDevice::cleanup). */
int mi355_close(mi355_dev *dev);
int mi355_get_props(mi355_dev *dev, mi355_props_t *out);
const char *mi355_last_error(mi355_dev *dev);

/* hipMalloc / hipFree / hipMemcpy as the run* tests use them
 * (e.g. src/rocm/global_bandwidth.cpp:26-55, src/rocm/mfma.cpp:139-165). */
int mi355_alloc(mi355_dev *dev, size_t bytes, void **dptr);
int mi355_free(mi355_dev *dev, void *dptr);
int mi355_upload(mi355_dev *dev, void *dst_dev, const void *src_host, size_t bytes);
int mi355_download(mi355_dev *dev, void *dst_host, const void *src_dev, size_t bytes);
int mi355_memset(mi355_dev *dev, void *dptr, int byte, size_t bytes);
int mi355_sync(mi355_dev *dev);

/* The two hipEventRecord brackets of RocmPeak::runKernel's runBatch
 * (src/rocm/rocm_peak.cpp:56-85).  start records on the handle's stream; stop
 * records, waits for the stream and returns the elapsed microseconds. */
int mi355_timer_start(mi355_dev *dev);
int mi355_timer_stop(mi355_dev *dev, float *elapsed_us);

/* ---- seeded inputs generated on the device ---------------------------------- */
/* Counter-based generator: element i of a stream is a pure function of
 * (seed, stream, i):
 *     z = seed + 0x9E3779B97F4A7C15*(i+1) + 0xD6E8FEB86659FD93*stream
 *     z = (z ^ z>>30) * 0xBF58476D1CE4E5B9;  z = (z ^ z>>27) * 0x94D049BB133111EB;  z ^= z>>31
 * (for stream 0 this is the (i+1)-th output of SplitMix64 started at `seed`).
 * Replaces the reference's host-side xorshift fill, populate()
 * (src/common/common.cpp:76-95), which it uploads with hipMemcpy.
 *   dist 0: uniform [0,1)   = (z>>40) * 2^-24
 *   dist 1: uniform [-1,1)  = ((z>>40) - 2^23) * 2^-23                          */
#define MI355_DIST_U01   0
#define MI355_DIST_UPM1  1
int mi355_fill_f32(mi355_dev *dev, float *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist);
/* The same fp32 values widened to fp64 (operands of the fp64 GEMM). */
int mi355_fill_f64(mi355_dev *dev, double *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist);
/* Same values rounded to nearest-even bf16 (GEMM operands). */
int mi355_fill_bf16(mi355_dev *dev, uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist);
/* Same values multiplied by `scale` (fp32) then rounded to nearest-even OCP
 * e4m3fn with saturation to +-448 (fp8 GEMM operands). */
int mi355_fill_fp8_e4m3(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist, float scale);
/* The same for the other GEMM operand types: IEEE half (nearest even), OCP e5m2 with
 * saturation to +-57344, and int8 = (z >> 60) - 8, uniform in [-8, 7]. */
int mi355_fill_f16(mi355_dev *dev, uint16_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist);
int mi355_fill_fp8_e5m2(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream, int dist, float scale);
int mi355_fill_i8(mi355_dev *dev, int8_t *dst, uint64_t n, uint64_t seed, uint32_t stream);

/* Plain device-to-device copy kernel (16 bytes per lane, grid-stride).  No counterpart in
 * the reference; it exists so that the HBM byte counters (FETCH_SIZE / WRITE_SIZE) can be
 * calibrated against a transfer of known size.  bytes must be a multiple of 16 and both
 * pointers 16-byte aligned. */
int mi355_copy(mi355_dev *dev, void *dst, const void *src, size_t bytes);

/* ---- global memory bandwidth -------------------------------------------------- */
/* Takes over global_bandwidth_v1/v2/v4 (src/rocm/rocm_kernels/global_bandwidth.hip:10-67)
 * and their launch in runGlobalBandwidth (src/rocm/global_bandwidth.cpp:6-110).
 * width in {1,2,4} floats per load.  T = blocks*block_size threads; thread t adds
 * vector elements t, t+T, t+2T, ... (component-wise, in that order, fp32) and
 * writes out[t] = ((x+y)+z)+w of its component sums (x for width 1, x+y for 2).
 * n_floats must be a multiple of width; `in` 16-byte aligned; out holds T floats.
 * block_size in {64,128,256,512,1024}. */
int mi355_global_bandwidth(mi355_dev *dev, int width, const float *in, uint64_t n_floats,
                           float *out, uint32_t blocks, uint32_t block_size);

/* ---- local (LDS) memory bandwidth --------------------------------------------- */
/* Takes over local_bandwidth_v1/v2/v4 (src/rocm/rocm_kernels/local_bandwidth.hip:3-66)
 * and their launch in runLocalBandwidth (src/rocm/local_bandwidth.cpp:6-75).  width in
 * {1,2,4} floats per LDS access.  Thread gid starts from (float)gid [, gid+1 [, gid+2,
 * gid+3]]; per repetition it stores its vector to slot lid of the workgroup's LDS array,
 * barrier, loads slot (lid+1) % block_size, barrier.  out[gid] = x [+ y [+ z + w]] of
 * what it holds after `reps` repetitions (the reference runs LMEM_REPS = 64,
 * include/common/common.h:58, and 256 threads per block).  out holds
 * blocks*block_size floats; block_size a multiple of 64 in [64,1024]. */
int mi355_local_bandwidth(mi355_dev *dev, int width, float *out, uint32_t blocks,
                          uint32_t block_size, uint32_t reps);

/* ---- host <-> device transfer bandwidth --------------------------------------- */
/* The pieces of runTransferBandwidth (src/rocm/transfer_bandwidth.cpp:6-122):
 * hipHostMalloc / hipHostFree of the pinned staging buffer (:32-40, :118) and the
 * hipMemcpyAsync on the device stream that its runBatch repeats between two events
 * (:52-60).  copy_async only enqueues; time a batch with mi355_timer_start/stop. */
#define MI355_H2D 0
#define MI355_D2H 1
int mi355_host_alloc(mi355_dev *dev, size_t bytes, void **hptr);
int mi355_host_free(mi355_dev *dev, void *hptr);
int mi355_copy_async(mi355_dev *dev, void *dst, const void *src, size_t bytes, int direction);

/* ---- vector MAD compute ------------------------------------------------------- */
/* Takes over the compute_* kernels (src/rocm/rocm_kernels/compute_sp.hip:18-70,
 * compute_hp.hip, compute_dp.hip, compute_mp.hip, compute_bf16.hip,
 * compute_int32.hip, compute_int8_dp.hip) and their launch in runComputeKernel
 * (src/rocm/compute_kernel.cpp:7-94).  Shape: n_items work-items, each with 16
 * accumulators (as 16/width vectors of `width` lanes) seeded from stream
 * `MI355_STREAM_MAD` element item*16+j, `steps` dependent steps, out[item] = sum of
 * the 16 accumulators in index order (one element of the kernel's type). */
#define MI355_MAD_F32      0  /* x = fma(x, a, x0), a = 1.0001f, x0 uniform[-1,1); widths 1,2,4          */
#define MI355_MAD_F16      1  /* same in IEEE half, a = 1-2^-10 (1.0001 is 1.0 in half), x0 = half(u);
                                 width 1: scalar half FMA, 2: packed half2 FMA; out is half bits        */
#define MI355_MAD_F64      2  /* same in double, a = 1.0001; widths 1,2,4                               */
#define MI355_MAD_MP       3  /* x = fma(x, ah, x0h): x fp32, ah = 1-2^-10 and x0h = half(u) IEEE half operands
                                 widened by the instruction (v_fma_mix_f32), one fp32 rounding; x starts
                                 at x0h; after every 16th step x = float(half(x)), nearest even (the block
                                 round trip of compute_mp.hip:18-23); width 1                           */
#define MI355_MAD_BF16     4  /* acc = acc + xb*ab + x0b*1: one two-element bf16 dot product with an fp32
                                 accumulator per step (v_dot2_f32_bf16, 4 flop); ab = -2^-8, x0b = bf16(u),
                                 xb and acc start at x0b; after every 128th step xb = bf16(acc), nearest
                                 even (the block round trip of compute_bf16.hip:26-31); width 1          */
#define MI355_MAD_I32      5  /* x = x*3 + x0 (wrapping), x0 = high 32 bits of the word; widths 1,2,4   */
#define MI355_MAD_I8DP     6  /* acc = sdot4(x, y, acc); y ^= acc; `width` in {1,2,4,8} = number of
                                 independent chains (x, y from element item*8+chain of streams
                                 MI355_STREAM_MAD / MI355_STREAM_MAD_Y), out = sum of the chains' acc    */
int mi355_compute_mad(mi355_dev *dev, int kind, int width, uint64_t seed,
                      uint64_t n_items, uint32_t steps, void *out, uint32_t block_size);

/* ---- kernel launch latency ---------------------------------------------------- */
/* Takes over kernel_latency_noop (src/rocm/rocm_kernels/kernel_latency.hip:3) and the
 * launch + hipStreamSynchronize wall-clock loop of runKernelLatency
 * (src/rocm/kernel_latency.cpp:40-56).  Does `warmup` untimed and `launches` timed
 * round trips of an empty 1x1x1 kernel; returns the mean in microseconds. */
int mi355_launch_roundtrip(mi355_dev *dev, uint32_t warmup, uint32_t launches, double *mean_us);

/* ---- dense MFMA --------------------------------------------------------------- */
/* Takes over mfma_fp16/bf16/fp8/int8/mxfp4 (src/rocm/rocm_kernels/mfma_*.hip) and
 * their launch in runMfma (src/rocm/mfma.cpp:58-168), on the CDNA4 shapes.
 * Operands are LOGICAL matrices, one set per (wave, chain), 4 chains per wave:
 *   A[wave][chain][M][K]  row-major, K contiguous
 *   B[wave][chain][N][K]  column-major B, K contiguous
 *   out[wave][chain][M][N] row-major fp32 (int32 for I8), C starts at 0 and every
 *   chain does acc = MFMA(A, B, acc) `iters` times.
 * Element storage: f16/bf16 2 bytes; i8/fp8/bf8 1 byte; fp6 packed 4 codes in
 * 3 bytes and fp4 2 codes per byte, little-endian bit order along K.
 * Scaled kinds take scaleA[wave][chain][M][K/32] and scaleB[wave][chain][N][K/32]
 * E8M0 bytes (value 2^(byte-127)); other kinds pass NULL.
 * waves must be a multiple of 4 (a workgroup is 4 waves).
 * clocks (may be NULL): two uint64 in device memory; wave 0 stores the shader-clock
 * ticks and the 100 MHz reference-clock ticks its MFMA loop took, from which the
 * caller derives the clock the chip actually held under this load. */
#define MI355_MFMA_F16_16x16x32     0
#define MI355_MFMA_BF16_16x16x32    1
#define MI355_MFMA_F16_32x32x16     2
#define MI355_MFMA_BF16_32x32x16    3
#define MI355_MFMA_I8_16x16x64      4
#define MI355_MFMA_FP8_16x16x128    5   /* OCP e4m3fn, scales fixed at 1.0 */
#define MI355_MFMA_BF8_16x16x128    6   /* OCP e5m2,   scales fixed at 1.0 */
#define MI355_MFMA_MXFP6_E2M3       7   /* 16x16x128, E8M0 block scales */
#define MI355_MFMA_MXFP6_E3M2       8
#define MI355_MFMA_MXFP4_E2M1       9
#define MI355_MFMA_KIND_COUNT      10
/* OR into `kind` (here and for mi355_smfmac): every chain of a wave takes the operands (A, B, scales /
 * index) of its chain 0, from the same registers, as the reference's kernels use one a and one b for all
 * their accumulator chains (src/rocm/rocm_kernels/mfma_bf16.hip:16-30).  The slots of chains 1..3 in
 * the operand arrays are then not read; all four output tiles of a wave are equal. */
#define MI355_MFMA_ONE_OPERAND_SET 0x100
/* Diagnosis of what holds the clock (no counterpart in the reference; also for mi355_smfmac).  OR into `kind`:
 * MI355_MATRIX_ON_XCDS(mask): only the workgroups that the part places on the XCDs of `mask` (workgroup index mod 8,
 * bit 0 = XCD 0, which must be among them: its wave 0 fills `clocks`) do their work, the others return at once and
 * leave their output tiles untouched.  MI355_MATRIX_ON_HALF_THE_CUS: of every XCD's workgroups only those of the
 * first 16 of its 32 CUs (workgroup index / 8 mod 32 < 16).  Same total work per active wave either way, so the
 * clock an active XCD holds with its neighbours idle, or with half of its own CUs idle, can be read off. */
#define MI355_MATRIX_ON_XCDS(mask) (((mask) & 0xff) << 16)
#define MI355_MATRIX_ON_HALF_THE_CUS 0x200
int mi355_mfma_dense(mi355_dev *dev, int kind, const void *A, const void *B,
                     const uint8_t *scaleA, const uint8_t *scaleB,
                     void *out, uint32_t waves, uint32_t iters, uint64_t *clocks);

/* ---- 2:4 structured-sparse SMFMAC --------------------------------------------- */
/* Takes over smfmac_fp16/bf16/fp8/int8 (src/rocm/rocm_kernels/smfmac_*.hip) and their
 * launch in runSparseMfma (src/rocm/sparse_mfma.cpp:52-151), on the CDNA4 shapes.
 *   Ac[wave][chain][M][K/2]   the two kept values of every group of four, K order
 *   meta[wave][chain][M][K/4] one byte per group: bits[1:0] = position (0..3) of the
 *                             first kept value, bits[3:2] = position of the second
 *   B[wave][chain][N][K]      dense, K contiguous;  out as for mi355_mfma_dense.
 * K is the dense-equivalent depth (64 for 16-bit kinds, 128 for 8-bit kinds).
 * clocks: as for mi355_mfma_dense. */
#define MI355_SMFMAC_F16_16x16x64    0
#define MI355_SMFMAC_BF16_16x16x64   1
#define MI355_SMFMAC_FP8_16x16x128   2
#define MI355_SMFMAC_BF8_16x16x128   3
#define MI355_SMFMAC_I8_16x16x128    4
#define MI355_SMFMAC_KIND_COUNT      5
int mi355_smfmac(mi355_dev *dev, int kind, const void *Ac, const uint8_t *meta, const void *B,
                 void *out, uint32_t waves, uint32_t iters, uint64_t *clocks);

/* One matrix instruction on raw per-lane register images (no reference counterpart:
 * the reference never checks a result, so it never needed to know the operand
 * layouts).  a_regs/b_regs: 64 lanes x 8 dwords (dense) or a 64x4 / b 64x8 dwords
 * (sparse, b holds 8 dwords); c_regs/d_regs: 64 lanes x 16 dwords (only the first 4
 * are used by 16x16 shapes); aux0/aux1: 64 dwords each (scaleA/scaleB for scaled
 * kinds, sparse index / unused for SMFMAC).  sel0/sel1: op_sel for scaled kinds,
 * unused otherwise.  `sparse` selects the kind namespace. */
int mi355_mfma_raw(mi355_dev *dev, int sparse, int kind,
                   const uint32_t *a_regs, const uint32_t *b_regs, const uint32_t *c_regs,
                   const uint32_t *aux0, const uint32_t *aux1, int sel0, int sel1,
                   uint32_t *d_regs);

/* ---- hand-written GEMM -------------------------------------------------------- */
/* Fills the slots of the vendor-library tests runRocblas / runHipblasLt
 * (src/rocm/rocblas.cpp:122-342 row "bf16"; src/rocm/hipblaslt_gemm.cpp:214-525 row
 * "fp8_e4m3"; both with K contiguous in A and B, fp32 accumulation, bf16 output).
 *   A[M][K] row-major, B[N][K] (column-major B), C[M][N] row-major bf16.
 * M, N multiples of 128 (fp32: of 256; see mi355_gemm_tiling), K a multiple of 128 bytes (64 bf16 values, 128 fp8
 * values) and a row of K at most 64 MiB; buffers 16-byte aligned.  fp8: C = scale_a*scale_b * (A.B).  Sums along K are
 * formed in an order that depends on the tile (results agree within rounding; int8 exactly). */
int mi355_gemm_bf16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C,
                    uint32_t M, uint32_t N, uint32_t K);
int mi355_gemm_fp8_e4m3(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C,
                        uint32_t M, uint32_t N, uint32_t K, float scale_a, float scale_b);
/* The other rows of the same two tests, same layouts and shape rules:
 *   "fp16" of runRocblas (src/rocm/rocblas.cpp:265-300: half operands, fp32 accumulate):
 *          C is IEEE half;
 *   "int8" of runRocblas (src/rocm/rocblas.cpp:309-333: i8 operands, i32 accumulate and output):
 *          C is int32, K a multiple of 128;
 *   "fp8_e5m2" of runHipblasLt (src/rocm/hipblaslt_gemm.cpp:393-396: an e5m2 A against an e4m3 B):
 *          C is bf16 = scale_a*scale_b * (A.B). */
int mi355_gemm_f16(mi355_dev *dev, const uint16_t *A, const uint16_t *B, uint16_t *C,
                   uint32_t M, uint32_t N, uint32_t K);
int mi355_gemm_i8(mi355_dev *dev, const int8_t *A, const int8_t *B, int32_t *C,
                  uint32_t M, uint32_t N, uint32_t K);
int mi355_gemm_fp8_e5m2(mi355_dev *dev, const uint8_t *A, const uint8_t *B, uint16_t *C,
                        uint32_t M, uint32_t N, uint32_t K, float scale_a, float scale_b);
/* Which tiling the five calls above take (no counterpart in the reference: the vendor libraries behind its tests
 * pick their own kernel per shape).  256: every workgroup owns a 256x256 tile of C and a whole CU, the schedule for
 * the sizes the reference's tests pick on a part of this many CUs (pickGemmDim, src/rocm/hipblaslt_gemm.cpp:41-55,
 * and pickRocblasGemmDim, src/rocm/rocblas.cpp:71: thousands of rows).  128: one
 * workgroup per 128x128 tile, four times as many workgroups at half the arithmetic per operand byte.  AUTO (the
 * default of a new handle): 128 when the product has at most half a 256x256 tile per CU (2048 cubed: 64 tiles on
 * 256 CUs), 256 otherwise.  The 256 tiling needs M and N to be multiples of 256: a product with a multiple of 128 only
 * runs on the 128 tiling under AUTO and is refused under 256.  Results of the two agree within rounding (int8 exactly). */
#define MI355_GEMM_TILING_AUTO 0
#define MI355_GEMM_TILING_256  1
#define MI355_GEMM_TILING_128  2
int mi355_gemm_tiling(mi355_dev *dev, int tiling);
/*   "fp32" of runRocblas (src/rocm/rocblas.cpp:246-254, rocblas_sgemm): fp32 operands, accumulation
 *          and output, on the fp32 matrix instruction; M, N multiples of 256, K a multiple of 32;
 *   "fp64" of runRocblas (src/rocm/rocblas.cpp:256-263, rocblas_dgemm): all fp64, on the fp64 matrix
 *          instruction; M, N multiples of 128, K a multiple of 16, buffers 32-byte aligned.
 *          Same operand layout as the rows above (K contiguous in A and in B). */
int mi355_gemm_f32(mi355_dev *dev, const float *A, const float *B, float *C,
                   uint32_t M, uint32_t N, uint32_t K);
int mi355_gemm_f64(mi355_dev *dev, const double *A, const double *B, double *C,
                   uint32_t M, uint32_t N, uint32_t K);

/*   "mxf4_e2m1" of runHipblasLt (src/rocm/hipblaslt_gemm.cpp:398-512: block-scaled FP4, one
 *          UE8M0 scale per 32 elements along K, fp32 accumulate, bf16 output).  A[M][K/2] and
 *          B[N][K/2] hold e2m1 codes two per byte (low nibble = even k), K contiguous;
 *          scale_a[M][K/32], scale_b[N][K/32] hold E8M0 bytes (value 2^(byte-127)).
 *          C[m][n] = sum_k A[m][k]*2^sa[m][k/32] * B[n][k]*2^sb[n][k/32].  K a multiple of 256.
 *          A, B, C 16-byte aligned, the scale arrays 8-byte aligned.
 *          Each call first rewrites the scales into the order the kernel loads them (one small
 *          launch, part of the timed work); the copy lives in a scratch buffer of the same size
 *          that the handle allocates on the first call and on growth, and frees in mi355_close. */
int mi355_gemm_mxfp4(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scale_a,
                     const uint8_t *scale_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K);
/*   The same product in two calls, for operands whose scales stay fixed over many products (weights): the
 *          reference's timed loop hands the library the same scale pointers on every call
 *          (src/rocm/hipblaslt_gemm.cpp:438-449 sets them once, :487-505 loops the product).
 *          mi355_gemm_mxfp4_prepare_scales lays scale_a / scale_b out in the order the kernel loads them,
 *          into `prepared` (caller-allocated device memory, (M + N) * K / 32 bytes, 16-byte aligned;
 *          same M, N, K rules); mi355_gemm_mxfp4_prepared multiplies with them and launches nothing else.
 *          The bytes of `prepared` mean something only to this library, for the M, N, K they were
 *          prepared for.  Results are bit for bit those of mi355_gemm_mxfp4. */
int mi355_gemm_mxfp4_prepare_scales(mi355_dev *dev, const uint8_t *scale_a, const uint8_t *scale_b,
                                    uint32_t M, uint32_t N, uint32_t K, uint8_t *prepared);
int mi355_gemm_mxfp4_prepared(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *prepared,
                              uint16_t *C, uint32_t M, uint32_t N, uint32_t K);
/*   The same product for callers that cannot allocate (tight serving loops, harnesses that forbid
 *          hipMalloc).  No counterpart in the reference.  Identical
 *          arguments, checks and result; the lane-ordered scales go into a 4 MiB array that lives in
 *          the library's device image instead of a buffer of the handle, so the call performs no
 *          allocation and frees nothing.  Limit: (M + N) * K / 32 <= 4 MiB (8192^3 just fits);
 *          larger problems are refused with MI355_ERR_ARG and a message.  Every call on a GPU shares
 *          that GPU's array: calls that overlap on one GPU (two handles, two threads) race; calls on
 *          one handle are ordered by its stream.  Nothing in it has to start at zero — each call
 *          overwrites all it reads. */
int mi355_gemm_mxfp4_static(mi355_dev *dev, const uint8_t *A, const uint8_t *B, const uint8_t *scale_a,
                            const uint8_t *scale_b, uint16_t *C, uint32_t M, uint32_t N, uint32_t K);
/* Bytes of device scratch memory the handle has allocated so far (today: the lane-ordered scales of
 * mi355_gemm_mxfp4); 0 on a fresh handle, and unchanged by the entry points that allocate nothing.
 * No counterpart in the reference; no HIP call. */
int mi355_scratch_bytes(mi355_dev *dev, size_t *handle_bytes);
/* Operands for it: dst[i] = lo + floor(span * (z >> 32) / 2^32), a uniform byte in [lo, lo+span)
 * (span 256, lo 0: random code pairs; lo 123, span 9: scales 2^-4 .. 2^4). */
int mi355_fill_bytes(mi355_dev *dev, uint8_t *dst, uint64_t n, uint64_t seed, uint32_t stream,
                     uint32_t lo, uint32_t span);

#ifdef __cplusplus
}
#endif
#endif /* CLPEAK_MI355_H */
