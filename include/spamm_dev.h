/*
 * spamm_dev.h -- measurement aids that are NOT part of the SpAMM engine.
 *
 * Built into a library of its own (libspamm_dev_gfx950.so); the engine
 * (libspamm_gfx950.so, include/spamm.h) neither contains nor needs any of
 * this.  Nothing here has a counterpart in the reference: its only
 * yardstick is a dense cuBLAS run (run_cublas_time, tool.cu:153-226).
 */
#ifndef SPAMM_DEV_H_
#define SPAMM_DEV_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define SPAMM_DEV_API __attribute__((visibility("default")))
#else
#define SPAMM_DEV_API
#endif

/* The rate the matrix pipeline of `device` sustains when every CU issues
 * nothing but independent fp16 32x32x16 MFMAs (iters x 16 per wave, one wave
 * per SIMD), with all-zero operands (random_operands = 0) or uniform [-1,1)
 * operands (1).  The sustained clock under MFMA load depends on the operand
 * values, so the second figure is the ceiling a GEMM on real data can
 * approach; a bench reports it next to the datasheet peak.  Allocates and
 * frees its own buffers, runs on its own stream, synchronises.  Returns 0 or
 * the negative of the failing hipError_t (-1 for bad arguments). */
SPAMM_DEV_API int spamm_dev_mfma_ceiling(int device, int random_operands, int iters, double *tflops,
                                         double *clock_ghz);

/* Read-only reference kernels for reading cache counters of other kernels against: `which` = 0: one
 * pass over 4 GiB with a full grid (every read comes from HBM, queues full); 1: 40 passes over one
 * 96 MiB buffer (misses the 4 MB L2s, stays in the 256 MB memory-side cache); 2 and 3: the same two
 * with 32 workgroups (idle queues: latency rather than bandwidth).  Each runs three times; *gbps is
 * the best.  Kernel names k_dev_read<which> tell them apart in a profile.  Returns 0 or the negative
 * of the failing hipError_t (-1 for bad arguments). */
SPAMM_DEV_API int spamm_dev_read_reference(int device, int which, double *gbps);

#ifdef __cplusplus
}
#endif
#endif /* SPAMM_DEV_H_ */
