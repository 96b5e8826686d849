/*
 * spamm.h -- C ABI of the gfx950 SpAMM engine (sparse approximate matrix
 * multiply: norm map -> tau gate -> gated fp16 tile GEMM with fp32 accumulate).
 *
 * The reference (buaa-hipo/cuSpAMM) has no callable API: its "multiply call" is
 * the timed body of main() (cuSpAMM.cu:458-546) driven by compile-time
 * constants (para.h:1-22, main.h:32-73).  This header turns that body and its
 * parameter vocabulary into run-time entry points.  All matrices are dense
 * row-major (cuSpAMM.cu:352-353,391; main.h:110) and all matrix pointers are
 * DEVICE pointers that stay resident across calls (cuSpAMM.cu:449-461).
 *
 * Every function returns SPAMM_OK (0) or a negative error code; nothing prints
 * or exits.  A context is bound to one device and one stream and is not
 * thread-safe; distinct contexts are independent.
 */
#ifndef SPAMM_H_
#define SPAMM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define SPAMM_API __attribute__((visibility("default")))
#else
#define SPAMM_API
#endif

#define SPAMM_OK 0
#define SPAMM_EINVAL (-1)    /* bad dimension / tile / pointer / flag */
#define SPAMM_ENOMEM (-2)    /* device or host allocation failed */
#define SPAMM_EHIP (-3)      /* a HIP call failed; see spamm_last_hip_error */
#define SPAMM_ESTATE (-4)    /* stage called before the stage it depends on */
#define SPAMM_ENODEV (-5)    /* no usable gfx950 device */

/* Operand roles for the norm-map stage. */
#define SPAMM_ROLE_A 0       /* contraction along columns: A[M x K] */
#define SPAMM_ROLE_B 1       /* contraction along rows:    B[K x N] */

/* spamm_params.flags */
#define SPAMM_FLAG_A_EQ_B 1u     /* A and B are the same matrix (square); reserved */
#define SPAMM_FLAG_TIMING 2u     /* record per-stage HIP events (spamm_get_stats) */

/* Run-time form of the reference's compile-time configuration:
 * M,K,N <- inM,inK,inN (para.h:6-8) already padded to a tile multiple
 * (main.h:54-56); tile <- LoNum (main.h:32); tau <- NormINIT/Norm narrowed to
 * float (para.h:2, cuSpAMM.cu:516). */
typedef struct spamm_params {
    int64_t M, K, N;     /* multiples of tile */
    int32_t tile;        /* 32, 64 or 128 */
    float tau;           /* product kept iff ||A_ik||_F * ||B_kj||_F >= tau (cuSpAMM.cu:305-306) */
    uint32_t flags;
    uint32_t reserved;
} spamm_params;

/* Results of the last spamm_multiply / stage calls on a context. */
typedef struct spamm_stats {
    int64_t total_products;   /* (M/b)(N/b)(K/b) */
    int64_t kept_products;    /* number of (i,j,k) that passed the gate */
    float ms_normmap_a;       /* valid when SPAMM_FLAG_TIMING was set */
    float ms_normmap_b;
    float ms_gate;
    float ms_gemm;
    float ms_total;
    int32_t timing_valid;
} spamm_stats;

typedef struct spamm_ctx spamm_ctx;

/* Replaces the per-device plan set-up (TGPUplan, cuSpAMM.cu:6-12,404-408):
 * binds a context to `device`, creates its stream.  Workspaces (fp16 operand
 * copies, norm maps, lists) are allocated lazily and reused across calls. */
SPAMM_API int spamm_create(spamm_ctx **out, int device);
SPAMM_API int spamm_destroy(spamm_ctx *ctx);

/* Run all stages on a caller-provided hipStream_t (default: the context's own
 * stream).  Pass NULL to return to the context's stream. */
SPAMM_API int spamm_set_stream(spamm_ctx *ctx, void *hip_stream);

/* The multiply call: the timed body of main() (cuSpAMM.cu:461-541) --
 * normmap(B), normmap(A), gate, gated GEMM -- on one stream with no host
 * synchronisation.  dA [M x K] fp32, dB [K x N] fp32, dC [M x N] fp32 (fully
 * overwritten, zeros where nothing is kept).  fp32->fp16 conversion (host side
 * in the reference, tool.cu:418,432) happens on the device inside the
 * norm-map stage. */
SPAMM_API int spamm_multiply(spamm_ctx *ctx, const spamm_params *p, const float *dA, const float *dB,
                   float *dC);

/* Stage 1 -- replaces unroll_get_Fnorm_FP16 / unroll_get_Fnorm_pri
 * (cuSpAMM.cu:74-123, 21-71; launches :478-503) plus the host fp16 conversion:
 * reads fp32 dX [rows x cols], stores the fp16 copy (context-private packed
 * layout) and the tile Frobenius norm map [rows/tile x cols/tile]. */
SPAMM_API int spamm_normmap_f32(spamm_ctx *ctx, int role, const float *dX, int64_t rows, int64_t cols,
                      int32_t tile);

/* Stage 2 -- replaces the gating prologue of get_C_FP16_B32
 * (cuSpAMM.cu:302-334): per output tile the kept-k bitmap, the ascending
 * compacted k list and the count.  Uses the norm maps left by stage 1 (or by
 * spamm_set_normmaps). */
SPAMM_API int spamm_gate(spamm_ctx *ctx, float tau);

/* Stage 3 -- replaces the product loop of get_C_FP16_B32 (cuSpAMM.cu:336-391):
 * C_ij = sum over kept k of A_ik * B_kj, fp16 operands, fp32 accumulate. */
SPAMM_API int spamm_gemm_gated(spamm_ctx *ctx, float *dC);

/* Upload host norm maps (row-major nA [nbM x nbK], nB [nbK x nbN]) so that the
 * gate can be exercised on hand-built maps. */
SPAMM_API int spamm_set_normmaps(spamm_ctx *ctx, const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                       int64_t nbN, int32_t tile);

/* Read-back helpers (host destination buffers; each synchronises the stream).
 *   normmap: row-major, role A [M/b x K/b], role B [K/b x N/b] (cuSpAMM.cu:438-439)
 *   counts:  int32 [nbM*nbN]
 *   klist:   uint16 [nbM*nbN*nbK], first counts[t] entries of each row valid
 *   mask:    uint64 [nbM*nbN*ceil(nbK/64)], bit k of tile t
 *   fp16:    the fp16 copy of an operand un-packed to row-major bit patterns */
SPAMM_API int spamm_get_normmap(spamm_ctx *ctx, int role, float *host_out);
SPAMM_API int spamm_get_counts(spamm_ctx *ctx, int32_t *host_out);
SPAMM_API int spamm_get_klist(spamm_ctx *ctx, uint16_t *host_out);
SPAMM_API int spamm_get_mask(spamm_ctx *ctx, uint64_t *host_out);
SPAMM_API int spamm_get_fp16(spamm_ctx *ctx, int role, uint16_t *host_out);

/* Synchronises and fills `out` (kept-product count as in countValid,
 * tool.cu:493-529; per-stage times replace the whole-iteration cudaEvent pair,
 * cuSpAMM.cu:459-545). */
SPAMM_API int spamm_get_stats(spamm_ctx *ctx, spamm_stats *out);

/* Synthetic inputs on the device (tool.cu:370-436 generators, plus the seeded
 * u_ij * decay(|i-j|) family): dX[i,j] = u_ij * table[|i-j|], u_ij = 1 when
 * random == 0.  `table` is a HOST array of max(rows,cols) floats. */
SPAMM_API int spamm_fill_decay_f32(spamm_ctx *ctx, float *dX, int64_t rows, int64_t cols,
                         const float *host_table, uint64_t seed, int random);

SPAMM_API int spamm_synchronize(spamm_ctx *ctx);
SPAMM_API const char *spamm_strerror(int code);
/* hipError_t of the last failing HIP call on this context, as an int. */
SPAMM_API int spamm_last_hip_error(spamm_ctx *ctx);
/* Library version, major*10000 + minor*100 + patch. */
SPAMM_API int spamm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SPAMM_H_ */
