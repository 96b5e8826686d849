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
#define SPAMM_ELIMIT (-6)    /* spamm_multiply_noalloc: the problem needs more than the fixed workspace */

/* Operand roles for the norm-map stage. */
#define SPAMM_ROLE_A 0       /* contraction along columns: A[M x K] */
#define SPAMM_ROLE_B 1       /* contraction along rows:    B[K x N] */

/* spamm_params.flags */
#define SPAMM_FLAG_A_EQ_B 1u     /* dA == dB, M == K == N (else SPAMM_EINVAL): at tile 32 and 64 the matrix is read once
                                  * for both operand roles (the single pass is reported as ms_normmap_b); at tile 128
                                  * the two ordinary passes run (they are faster there) */
#define SPAMM_FLAG_TIMING 2u     /* record per-stage HIP events (spamm_get_stats) */
#define SPAMM_FLAG_REUSE_A 4u    /* A's fp16 copy and norm map from an earlier call are reused (dA ignored) */
#define SPAMM_FLAG_REUSE_B 8u    /* same for B: e.g. one B against many A, or matrix powers */
#define SPAMM_FLAG_PRUNE 16u     /* tau-aware conversion passes (tau > 0): the fp16 copy of a tile is written only if some
                                  * product can keep it.  A tile A_ik: fl(|A_ik| * max_j |B_kj|) >= tau (B's norms are
                                  * complete when A's pass runs).  B tile B_kj: |B_kj| > 0 (B's pass runs first; a
                                  * tile of norm zero fails the gate against any A).  Exact: fp32 rounding is
                                  * monotone, so every product of a skipped tile fails the gate.  C, mask and counts
                                  * are identical to a call without the flag; the passes write less.  Afterwards the
                                  * copies are incomplete: SPAMM_FLAG_REUSE_A is accepted only together with
                                  * SPAMM_FLAG_REUSE_B and tau' >= tau, SPAMM_FLAG_REUSE_B only with tau' > 0, and
                                  * spamm_get_fp16 and spamm_error_vs_dense_f64 return SPAMM_ESTATE until the
                                  * operand is converted again without the flag.  With SPAMM_FLAG_A_EQ_B (one pass, no
                                  * row maxima yet) only tiles of norm zero are left out, in both copies.  Ignored
                                  * for tau <= 0.  No counterpart in the reference, which converts on the host
                                  * outside its timed region (tool.cu:418,432). */

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

/* Tuning options.  The defaults suit a whole MI355X; nothing here changes C, mask or counts.
 *   SPAMM_OPT_NUM_XCD: number of XCDs (32 CUs sharing an L2) the GEMM schedule deals workgroups to:
 *     1, 2, 4 or 8; 0 = derive from the device's CU count (what spamm_create does; a partitioned
 *     device shows fewer).  Invalidates the gate of the last call.
 *   SPAMM_OPT_GATE_CHUNK_WORDS: the gate walks K in chunks of at most this many 64-k-tile bitmap
 *     words; 0 = as many as fit LDS (one chunk unless K / tile exceeds ~19 500 at tile 32).
 *   SPAMM_OPT_GEMM_RING: LDS stages of the GEMM's operand ring, 3..5; 0 = default (4).
 *   SPAMM_OPT_GEMM_SHAPE: work unit of the gated GEMM: 1 = a workgroup of four waves per 256 x 256
 *     macro tile of C (one workgroup per CU), 2 = four waves per 128 x 256 half (two workgroups per
 *     CU), 3 = eight waves per macro tile, 4 = shape 1 by workgroups that stay on their CU and draw
 *     macro tiles from a ticket counter per XCD; 0 = chosen per call (halves when C has at most
 *     half a macro tile per CU, else 1).  All walk the same lists in the same order: C is
 *     bit-identical.
 * SPAMM_EINVAL for an unknown option or a value outside its range.  The reference has no such
 * knobs: its launch shapes are compile-time constants (main.h:32-73). */
#define SPAMM_OPT_NUM_XCD 1
#define SPAMM_OPT_GATE_CHUNK_WORDS 2
#define SPAMM_OPT_GEMM_RING 3
#define SPAMM_OPT_GEMM_SHAPE 4
SPAMM_API int spamm_set_option(spamm_ctx *ctx, int option, int value);

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

/* The same multiply for operands that already are fp16 (the reference's actual
 * input type, para.h:1, cuSpAMM.cu:486): dAh, dBh are row-major fp16 device
 * arrays.  The norm-map stage then only packs and takes norms. */
SPAMM_API int spamm_multiply_f16(spamm_ctx *ctx, const spamm_params *p, const void *dAh, const void *dBh,
                                 float *dC);

/* spamm_multiply for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * main() allocates everything up front (cuSpAMM.cu:435-439).  Same arguments, same result, but the
 * whole workspace -- fp16 operand copies, norm maps, gate bitmaps and lists, schedule -- lives in one
 * fixed device array of SPAMM_NOALLOC_WORKSPACE_BYTES that is part of the library image (every GPU
 * the library runs on holds it until the process ends), and the call makes no hipMalloc / hipFree.
 * Limit: the buffers for (M, K, N, tile) must fit the array -- 2(MK + KN) bytes of fp16 copies plus
 * ~1 % for the rest, e.g. up to 2048 x 4096 x 2048 or 3072^3 -- else SPAMM_ELIMIT.
 * SPAMM_FLAG_REUSE_A/B are rejected (SPAMM_EINVAL).  All contexts on one GPU share the array and it
 * keeps the last call's contents: calls that overlap in time on one GPU (two contexts, two
 * streams) race; issue them one after the other.  Afterwards the context's read-backs and stage
 * calls refer to this call's results -- until ANY context makes the next spamm_multiply_noalloc
 * on the same GPU: from then on they return SPAMM_ESTATE for this context (the array now holds the
 * other call's bytes).  The next ordinary multiply / norm-map call returns to the context's own
 * workspace, whose contents (and REUSE state) are as it left them. */
#define SPAMM_NOALLOC_WORKSPACE_BYTES (40u << 20)
SPAMM_API int spamm_multiply_noalloc(spamm_ctx *ctx, const spamm_params *p, const float *dA, const float *dB,
                                     float *dC);

/* Stage 1 -- replaces unroll_get_Fnorm_FP16 / unroll_get_Fnorm_pri
 * (cuSpAMM.cu:74-123, 21-71; launches :478-503) plus the host fp16 conversion:
 * reads fp32 dX [rows x cols], stores the fp16 copy (context-private packed
 * layout) and the tile Frobenius norm map [rows/tile x cols/tile]. */
SPAMM_API int spamm_normmap_f32(spamm_ctx *ctx, int role, const float *dX, int64_t rows, int64_t cols,
                      int32_t tile);

SPAMM_API int spamm_normmap_f16(spamm_ctx *ctx, int role, const void *dXh, int64_t rows, int64_t cols,
                                int32_t tile);

/* Stage 2 -- replaces the gating prologue of get_C_FP16_B32
 * (cuSpAMM.cu:302-334): per output tile the kept-k bitmap and the count (the
 * ascending compacted k list of :315-325 is the bitmap's set bits in order;
 * spamm_get_klist materialises it).  Uses the norm maps left by stage 1 (or by
 * spamm_set_normmaps); SPAMM_ESTATE unless both are present for the same K and tile.
 * Shape limit (SPAMM_EINVAL): at most 8192 super tiles of 1024 x 2048 elements of C.  K is not
 * limited beyond the 65535 tiles per dimension: a macro tile's bitmaps are held in LDS, and where
 * they do not fit (K / tile beyond about 19 500 at tile 32) the gate walks K in chunks. */
SPAMM_API int spamm_gate(spamm_ctx *ctx, float tau);

/* Stage 3 -- replaces the product loop of get_C_FP16_B32 (cuSpAMM.cu:336-391):
 * C_ij = sum over kept k of A_ik * B_kj, fp16 operands, fp32 accumulate. */
SPAMM_API int spamm_gemm_gated(spamm_ctx *ctx, float *dC);

/* tau for a target kept ratio -- replaces the host-side tuner that the reference
 * runs inside its timed loop (tuneValidRate, tool.cu:438-490; main.h:35-38).
 * Both use the norm maps left by stage 1 (or spamm_set_normmaps) and leave
 * the gate untouched.
 *   spamm_tau_for_ratio: exact order statistic on the device: tau = the
 *     ceil(ratio*total)-th largest fp32 norm product, so that the products
 *     >= tau are kept (ties may push the achieved ratio above the target); if
 *     fewer positive products exist, the smallest positive one.
 *   spamm_tune_bisect: the reference's bisection, same arithmetic
 *     (tool.cu:445-486): iteration 0 measures the ratio at tau = 0 and moves to the
 *     mean product, later rounds bisect, stop at |ratio - expected| < tol or
 *     after max_rounds (reference: 0.75, 0.01, 20).  Counting runs on the device.
 *   spamm_count_kept: products with (double)product >= threshold, and the
 *     sum of all products (tool.cu:448-463, 505-516). */
SPAMM_API int spamm_tau_for_ratio(spamm_ctx *ctx, double ratio, float *tau_out, double *achieved_out);
SPAMM_API int spamm_tune_bisect(spamm_ctx *ctx, double expected, double tol, int max_rounds, float *tau_out,
                                double *achieved_out);
SPAMM_API int spamm_count_kept(spamm_ctx *ctx, double threshold, int64_t *count_out, double *sum_out);

/* Upload host norm maps (row-major nA [nbM x nbK], nB [nbK x nbN]) so that the
 * gate can be exercised on hand-built maps. */
SPAMM_API int spamm_set_normmaps(spamm_ctx *ctx, const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                       int64_t nbN, int32_t tile);

/* Read-back helpers (host destination buffers; each synchronises the stream).
 *   normmap: row-major, role A [M/b x K/b], role B [K/b x N/b] (cuSpAMM.cu:438-439)
 *   counts:  int32 [nbM*nbN]
 *   klist:   uint16 [nbM*nbN*nbK], first counts[t] entries of each row valid (built from the
 *            mask by this call; the rest of each row is unspecified)
 *   mask:    uint64 [nbM*nbN*ceil(nbK/64)], bit k of tile t
 *   fp16:    the fp16 copy of an operand un-packed to row-major bit patterns */
SPAMM_API int spamm_get_normmap(spamm_ctx *ctx, int role, float *host_out);
SPAMM_API int spamm_get_counts(spamm_ctx *ctx, int32_t *host_out);
SPAMM_API int spamm_get_klist(spamm_ctx *ctx, uint16_t *host_out);
SPAMM_API int spamm_get_mask(spamm_ctx *ctx, uint64_t *host_out);
SPAMM_API int spamm_get_fp16(spamm_ctx *ctx, int role, uint16_t *host_out);
/* The work list the gate built for the GEMM (the reference has none: every block re-gates its own
 * tile, cuSpAMM.cu:302-334): per macro tile of C (256 x 256 elements, row-major over
 * ceil(M/256) x ceil(N/256)) host_counts[2 m] = k tiles kept by at least one of its output tiles
 * (the length of the list its workgroup walks), host_counts[2 m + 1] = of which kept by all of
 * them; host_sched (optional, 16 ints): per XCD x the number of macro tiles with work [x] and of
 * all macro tiles [8 + x] in its sequence. */
SPAMM_API int spamm_get_macro_counts(spamm_ctx *ctx, int32_t *host_counts, int32_t *host_sched);

/* Synchronises and fills `out` (kept-product count as in countValid,
 * tool.cu:493-529; per-stage times replace the whole-iteration cudaEvent pair,
 * cuSpAMM.cu:459-545). */
SPAMM_API int spamm_get_stats(spamm_ctx *ctx, spamm_stats *out);

/* Synthetic inputs on the device (tool.cu:370-436 generators, plus the seeded
 * u_ij * decay(|i-j|) family): dX[i,j] = u_ij * table[|i-j|], u_ij = 1 when
 * random == 0.  `table` is a HOST array of max(rows,cols) floats. */
SPAMM_API int spamm_fill_decay_f32(spamm_ctx *ctx, float *dX, int64_t rows, int64_t cols,
                         const float *host_table, uint64_t seed, int random);

/* Error report (check_simple_gpu / COUNTERRTRANS, tool.cu:227-280, 6-24, with an
 * exact fp64 product of the resident fp16 operands instead of cuBLAS):
 * out3 = { ||C - C_dense||_F, ||C_dense||_F, ||C||_F } over rows [row0, row1)
 * (multiples of 64; N a multiple of 64).  The dense product is never stored. */
SPAMM_API int spamm_error_vs_dense_f64(spamm_ctx *ctx, const float *dC, int64_t row0, int64_t row1,
                                       double *out3);
/* tau-derived bound on that error: sqrt(sum_ij s_ij^2) with s_ij = sum_{k dropped} nA[i,k]*nB[k,j],
 * the bound on ||C_ij - (A B)_ij||_F of output tile (i,j).  spamm_dropped_bound_tiles returns the
 * per-tile s_ij themselves, row-major [M/b x N/b] doubles in a HOST buffer (where the error sits,
 * which the reference's single printed norm, tool.cu:6-24, does not tell).  Both use the norm maps
 * of stage 1 and take tau as an argument (the gate need not have run). */
SPAMM_API int spamm_dropped_bound(spamm_ctx *ctx, float tau, double *out);
SPAMM_API int spamm_dropped_bound_tiles(spamm_ctx *ctx, float tau, double *host_out);

/* Input adapters (host): dense CSV, one matrix row per line (getMatrixFromCSV,
 * tool.cu:329-366), and "row col val" triples, 1-based, first line skipped
 * (getMatrixFromMTX, tool.cu:282-327).  host_out is rows x ld, zero-filled
 * first, so ld/rows may be the tile-padded sizes (main.h:54-56). */
SPAMM_API int spamm_load_csv_f32(const char *path, int64_t rows, int64_t cols, int64_t ld, float *host_out);
SPAMM_API int spamm_load_mtx_f32(const char *path, int64_t rows, int64_t cols, int64_t ld, float *host_out);

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
