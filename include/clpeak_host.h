/* clpeak_host.h — auxiliary C entry points of libclpeak_host.so.
 *
 * libclpeak_host.so carries two C ABIs.  The embedding ABI (clpeak_ffi.h: the six clpeak_* calls a
 * front end binds) is the reference's.  This header is the second one and has no counterpart in the
 * reference: plain-C windows onto pieces of the C++ host layer that callers without a C++ compiler
 * need — the seeded operand generator that builds the inputs of the matrix rows (bench drivers and
 * tests generate the same operands as the CLI through it), the shared calibration helpers, the
 * result-file converter and the cancel flag.  Nothing here touches a GPU.
 */
#ifndef CLPEAK_HOST_H
#define CLPEAK_HOST_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- calibration (reference: src/common/common.cpp:16-45, include/common/common.h:142-147) ---- */

/* Launches per timed batch: `forced` if non-zero, else target_us / per_iter_us clamped to
 * [1, max_iters] (pickIters, src/common/common.cpp:35-45). */
unsigned clpeak_host_pick_iters(double per_iter_us, unsigned target_us, unsigned forced, unsigned max_iters);

/* Work-items of the vector-compute and bandwidth launches for a device with `num_cus` compute units
 * (targetGlobalThreads, include/common/common.h:142-147). */
unsigned long long clpeak_host_target_global_threads(unsigned num_cus);

/* benchmark_config_t::forDevice(type) (src/common/common.cpp:16-33), type 1 = CPU, 2 = GPU:
 * out = { globalBWMaxSize, computeWgsPerCU, computeDPWgsPerCU, transferBWMaxSize, targetTimeUs,
 *         kernelLatencyIters }. */
void clpeak_host_config_for_device(unsigned type, unsigned long long out[6]);

/* ---- seeded operands of the matrix rows (no reference counterpart: its kernels multiply constants,
 *      src/rocm/rocm_kernels/mfma_bf16.hip:16-17) ---- */

/* n elements of stream `stream` under `seed`, normal(0, sigma) rounded once to the format (int8:
 * uniform in [-8, 7], sigma ignored), packed as the kernels read them (6-bit and 4-bit codes
 * little-endian along the element index).  fmt: 0 f16, 1 bf16, 2 e4m3, 3 e5m2, 4 e2m3, 5 e3m2,
 * 6 e2m1, 7 int8.  Returns the number of bytes written, 0 if `cap` is too small. */
size_t clpeak_host_seeded_operand(int fmt, double sigma, unsigned long long seed, unsigned stream,
                                  unsigned long long n, unsigned char *out, size_t cap);

/* The same formats: n elements of the constant the reference's kernel of that format multiplies
 * (1.0; byte 0x38; byte 0x01; nibble 4).  Returns bytes written, 0 if `cap` is too small. */
size_t clpeak_host_reference_operand(int fmt, unsigned long long n, unsigned char *out, size_t cap);

/* what = 0: n E8M0 scale bytes, exponents uniform in [-4, 4]; what = 1: n bytes of 2:4 metadata (one
 * of the six patterns per group of four: first kept slot | second << 2).  `out` holds n bytes. */
size_t clpeak_host_seeded_bytes(int what, unsigned long long seed, unsigned stream, unsigned long long n,
                                unsigned char *out);

/* ---- result files (reference: src/common/result_store.cpp:145-963) ---- */

/* Load a result file (XML, JSON or CSV by extension) and write it again as fmt (0 XML, 1 JSON,
 * 2 CSV).  Returns the number of rows loaded, -1 when saving failed. */
int clpeak_host_resave(const char *in_path, const char *out_path, int fmt);

/* ---- cancel flag (reference: src/common/common.cpp:10-13) ---- */
int clpeak_host_cancel_requested(void);
void clpeak_host_request_cancel(void);
void clpeak_host_reset_cancel(void);

#ifdef __cplusplus
}
#endif
#endif /* CLPEAK_HOST_H */
