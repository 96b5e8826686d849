/*
 * spamm_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Plain host C (C99 + OpenMP) restatement of the cuSpAMM algorithm:
 * tile Frobenius norm maps, the tau gate, and the gated tile product with
 * fp16 operands and fp32 accumulation.  It is the correctness checker for the
 * HIP library and the reported CPU baseline.  Only tests, the smoke check and
 * the bench's cpu_baseline leg may load it; the product library never does.
 *
 * Reference lines each function follows (paths are in the cuSpAMM tree):
 *   orc_fill_decay      tool.cu:409-436   (decay generators; seeded u_ij added)
 *   orc_f32_to_f16      tool.cu:418       (__float2half, round-to-nearest-even)
 *   orc_normmap         cuSpAMM.cu:21-71, 74-123 (sqrt of tile sum of squares,
 *                       row-major map [rows/b x cols/b]); accumulation is fp32
 *                       in the fixed order documented below, NOT the reference's
 *                       fp16 WMMA column sums (cuSpAMM.cu:86,98-102)
 *   orc_gate            cuSpAMM.cu:303-311 (fp32 product, >= tau),
 *                       cuSpAMM.cu:315-325 (ascending compaction),
 *                       cuSpAMM.cu:328-334 (count); tool.cu:493-529 (kept count)
 *   orc_gemm_gated      cuSpAMM.cu:358-375 (sum of kept tile products, fp16
 *                       operands, fp32 accumulator, ascending k), :391 (C layout);
 *                       loop structure of the authors' commented-out CPU check
 *                       tool.cu:85-118
 *   orc_gemm_dense_f64  tool.cu:227-280   (dense comparison product; here fp64)
 *   orc_frob_diff       tool.cu:6-24      (error / dense / spamm Frobenius norms)
 *   orc_tau_for_ratio   tool.cu:438-490   (tau for a target kept ratio; exact
 *                       order statistic instead of bisection)
 *   orc_tune_bisect     tool.cu:438-490   (the reference's bisection, verbatim
 *                       semantics)
 *
 * Parity pins (see tests/test_oracle_*.py): the reference ships no tests or
 * golden vectors, so each function is pinned by mathematics: conversion against
 * numpy's IEEE float16 cast; norm maps against closed forms (all-ones, identity,
 * geometric decay), the sum-of-squares invariant and fp64 brute force; the gate
 * against tau=0 / tau=inf, monotonicity, hand-built maps with products equal to
 * tau, and a numpy restatement of countValid; the gated product against fp64
 * dense GEMM at tau=0, all-ones, identity and block-diagonal inputs, brute force
 * on tiny inputs, and the dropped-norm error bound.
 *
 * What stays unpinned: the reference's own fp16-rounded norm values
 * (cuSpAMM.cu:86,98-102) and therefore its exact mask for products within
 * rounding distance of tau.  This restatement deliberately uses the clean fp32
 * Frobenius norm instead.
 *
 * Canonical norm accumulation order (shared with the HIP kernel so that the
 * norm maps, and hence the kept mask, are bit-identical):
 *   - the contraction axis of a tile is its column axis for the A operand
 *     (role 0) and its row axis for the B operand (role 1); the other axis is
 *     the "free" axis r in [0,b).
 *   - chunk(r,q), q in [0,b/8): s = 0; s = s + x*x over the 8 consecutive
 *     elements 8q..8q+7 along the contraction axis (x is an fp16 value, so x*x
 *     is exact in fp32 and only the additions round).
 *   - chunk index c = r*(b/8)+q; lane L = c % 64, step it = c / 64;
 *     partial[L] = chunk(it=0) + chunk(it=1) + ... in ascending it.
 *   - butterfly: for s in 1,2,4,8,16,32: partial[L] = partial[L] + partial[L^s].
 *   - norm = sqrtf(partial[0]) (correctly rounded).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ utils */

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORC_API void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> fp16 bit pattern, IEEE round-to-nearest-even, subnormals kept,
 * overflow to infinity, NaN stays NaN (quiet). */
static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7fffffffu;
    if (abs >= 0x7f800000u) {                      /* inf / nan */
        if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((abs >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (abs >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  /* rounds to >= 65520 -> inf */
    if (abs >= 0x38800000u) {                      /* normal fp16 range: |f| >= 2^-14 */
        uint32_t mant = abs & 0x7fffffu;
        uint32_t exp = (abs >> 23) - 112u;         /* rebias 127 -> 15 */
        uint32_t h = (exp << 10) | (mant >> 13);
        uint32_t rem = mant & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;   /* may carry into exponent: correct */
        return (uint16_t)(sign | h);
    }
    if (abs < 0x33000000u) return (uint16_t)sign;  /* |f| < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
    /* subnormal fp16: value = m * 2^-24, m in [0,1024) */
    {
        uint32_t e = abs >> 23;                    /* 102..112 */
        uint32_t mant = (abs & 0x7fffffu) | 0x800000u;   /* 24-bit significand */
        uint32_t shift = 126u - e;                 /* 14..24: mant * 2^(e-150) / 2^-24 = mant >> (126-e) */
        uint32_t h = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
}

static inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    if (exp == 0) {
        if (mant == 0) return bits_f32(sign);
        /* subnormal: mant * 2^-24, exact in fp32 */
        float v = (float)mant * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (mant << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

ORC_API void orc_f32_to_f16(const float *x, int64_t n, uint16_t *h) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) h[i] = f32_to_f16_bits(x[i]);
}

ORC_API void orc_f16_to_f32(const uint16_t *h, int64_t n, float *x) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) x[i] = f16_bits_to_f32(h[i]);
}

/* ------------------------------------------------------------ generators */

/* Counter-based uniform: 24 random bits k -> k*2^-23 - 1 in [-1,1), exact in fp32. */
static inline float hash_uniform(uint64_t seed, uint64_t idx) {
    uint64_t z = idx + seed * 0x9E3779B97F4A7C15ull + 0x632BE59BD9B4E019ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    uint32_t k = (uint32_t)(z >> 40);
    return (float)k * 1.1920928955078125e-07f - 1.0f;
}

/* X[i,j] = u_ij * table[|i-j|], u_ij = seeded uniform in [-1,1) when
 * random != 0, else 1.  table has max(rows,cols) fp32 entries computed once by
 * the caller in fp64 (so host and device inputs are bit-identical).
 * Covers the reference generators (tool.cu:409-436: table = c*v^d or
 * c/(d^v+1), random = 0; tool.cu:370-403: table = 1) and the seeded
 * u_ij*decay(|i-j|) family. */
ORC_API void orc_fill_decay(float *X, int64_t rows, int64_t cols, const float *table,
                            uint64_t seed, int random) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; i++) {
        for (int64_t j = 0; j < cols; j++) {
            int64_t d = i > j ? i - j : j - i;
            float u = random ? hash_uniform(seed, (uint64_t)(i * cols + j)) : 1.0f;
            X[i * cols + j] = u * table[d];
        }
    }
}

/* -------------------------------------------------------------- norm map */

/* H: fp16 bit patterns, row-major [rows x cols]; b in {32,64,128};
 * role 0 = A operand (contraction along columns), 1 = B operand (along rows).
 * nm: row-major [rows/b x cols/b]. */
ORC_API int orc_normmap(const uint16_t *H, int64_t rows, int64_t cols, int b, int role, float *nm) {
    if (b != 32 && b != 64 && b != 128) return -1;
    if (rows % b || cols % b) return -1;
    const int64_t nbr = rows / b, nbc = cols / b;
    const int qn = b / 8;
    const int steps = b * b / 8 / 64;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t I = 0; I < nbr; I++) {
        for (int64_t J = 0; J < nbc; J++) {
            float partial[64], tmp[64];
            const uint16_t *T = H + I * b * cols + J * b;
            for (int it = 0; it < steps; it++) {
                for (int L = 0; L < 64; L++) {
                    int c = it * 64 + L;
                    int r = c / qn, q = c % qn;
                    float s = 0.0f;
                    for (int e = 0; e < 8; e++) {
                        int k = 8 * q + e;
                        uint16_t hb = role == 0 ? T[(int64_t)r * cols + k] : T[(int64_t)k * cols + r];
                        float x = f16_bits_to_f32(hb);
                        float sq = x * x;          /* exact */
                        s = s + sq;
                    }
                    partial[L] = it == 0 ? s : partial[L] + s;
                }
            }
            for (int s = 1; s < 64; s <<= 1) {
                for (int L = 0; L < 64; L++) tmp[L] = partial[L] + partial[L ^ s];
                memcpy(partial, tmp, sizeof(partial));
            }
            nm[I * nbc + J] = sqrtf(partial[0]);
        }
    }
    return 0;
}

/* A MODEL of the reference's own fp16 norm kernel (unroll_get_Fnorm_FP16,
 * cuSpAMM.cu:74-123; tile 32 only, as there), used by one CPU test to count how
 * many gate decisions would differ from the clean fp32 norm above.  Not used
 * for parity: what a WMMA unit does inside an fp16-accumulator product is not
 * specified, so this function is PARITY UNPINNED by construction.
 * Per 16 x 16 quarter of the tile (one warp, :93-94): every element is squared
 * in fp32 and rounded to fp16 (:98-101); ones(16x16) x squares with an fp16
 * accumulator gives the 16 column sums (:102) -- modelled as an exact sum of the
 * 16 fp16 squares rounded once to fp16; the column sums times ones with an fp32
 * accumulator gives their total (:109-112, element 0 is read at :116) --
 * modelled as fp32 additions in ascending column order.  The four quarter
 * totals are added in warp order and the square root taken in fp32 (:120). */
ORC_API int orc_normmap_ref16_model(const uint16_t *H, int64_t rows, int64_t cols, float *nm) {
    const int b = 32;
    if (rows % b || cols % b) return -1;
    const int64_t nbr = rows / b, nbc = cols / b;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t I = 0; I < nbr; I++) {
        for (int64_t J = 0; J < nbc; J++) {
            float warp_total[4];
            for (int w = 0; w < 4; w++) {
                const uint16_t *T = H + (I * b + (w / 2) * 16) * cols + J * b + (w % 2) * 16;
                float tot = 0.0f;
                for (int c = 0; c < 16; c++) {
                    double col = 0.0;                       /* exact: 16 fp16 values */
                    for (int r = 0; r < 16; r++) {
                        const float x = f16_bits_to_f32(T[(int64_t)r * cols + c]);
                        col += (double)f16_bits_to_f32(f32_to_f16_bits(x * x));
                    }
                    tot = tot + f16_bits_to_f32(f32_to_f16_bits((float)col));
                }
                warp_total[w] = tot;
            }
            nm[I * nbc + J] = sqrtf(((warp_total[0] + warp_total[1]) + warp_total[2]) + warp_total[3]);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ gate */

/* nA [nbM x nbK], nB [nbK x nbN] row-major.  keep(i,j,k) = nA[i,k]*nB[k,j] >= tau,
 * fp32 multiply and fp32 compare.  Outputs (any may be NULL):
 *   counts [nbM*nbN]            kept k per output tile
 *   klist  [nbM*nbN*nbK]        ascending kept k, first counts[t] entries valid
 *   mask   [nbM*nbN*words]      bit k of tile t = keep, words = (nbK+63)/64
 * Returns the total number of kept products. */
ORC_API int64_t orc_gate(const float *nA, const float *nB, int64_t nbM, int64_t nbK, int64_t nbN,
                         float tau, int32_t *counts, uint16_t *klist, uint64_t *mask) {
    const int64_t words = (nbK + 63) / 64;
    int64_t total = 0;
#pragma omp parallel for schedule(static) reduction(+ : total)
    for (int64_t i = 0; i < nbM; i++) {
        for (int64_t j = 0; j < nbN; j++) {
            const int64_t t = i * nbN + j;
            int32_t cnt = 0;
            if (mask) memset(mask + t * words, 0, (size_t)words * 8);
            for (int64_t k = 0; k < nbK; k++) {
                volatile float p = nA[i * nbK + k] * nB[k * nbN + j];
                if (p >= tau) {
                    if (klist) klist[t * nbK + cnt] = (uint16_t)k;
                    if (mask) mask[t * words + (k >> 6)] |= 1ull << (k & 63);
                    cnt++;
                }
            }
            if (counts) counts[t] = cnt;
            total += cnt;
        }
    }
    return total;
}

/* ----------------------------------------------------------- gated GEMM */

/* Af [M x K], Bf [K x N]: fp32 arrays holding fp16-representable values.
 * C [M x N] fp32, fully overwritten for tile rows [ti0, ti1) (zeros where
 * nothing is kept).  counts/klist as produced by orc_gate (klist stride nbK).
 * Accumulation: fp32, kept k ascending, then the b inner products ascending. */
__attribute__((target_clones("avx2", "default")))
static void tile_fma(float *restrict acc, const float *restrict Arow0, int64_t lda,
                     const float *restrict Brow0, int64_t ldb, int b) {
    for (int r = 0; r < b; r++) {
        float *restrict out = acc + (int64_t)r * b;
        const float *restrict ar = Arow0 + (int64_t)r * lda;
        for (int kk = 0; kk < b; kk++) {
            const float a = ar[kk];
            const float *restrict br = Brow0 + (int64_t)kk * ldb;
            for (int c = 0; c < b; c++) out[c] += a * br[c];
        }
    }
}

ORC_API int orc_gemm_gated(const float *Af, const float *Bf, int64_t M, int64_t K, int64_t N, int b,
                           const int32_t *counts, const uint16_t *klist, float *C,
                           int64_t ti0, int64_t ti1) {
    if (M % b || K % b || N % b) return -1;
    const int64_t nbK = K / b, nbN = N / b;
#pragma omp parallel
    {
        float *acc = (float *)malloc(sizeof(float) * b * b);
#pragma omp for schedule(dynamic, 1) collapse(2)
        for (int64_t i = ti0; i < ti1; i++) {
            for (int64_t j = 0; j < nbN; j++) {
                const int64_t t = i * nbN + j;
                memset(acc, 0, sizeof(float) * b * b);
                for (int32_t e = 0; e < counts[t]; e++) {
                    const int64_t k = klist[t * nbK + e];
                    tile_fma(acc, Af + i * b * K + k * b, K, Bf + k * b * N + j * b, N, b);
                }
                for (int r = 0; r < b; r++)
                    memcpy(C + (i * b + r) * N + j * b, acc + (int64_t)r * b, sizeof(float) * b);
            }
        }
        free(acc);
    }
    return 0;
}

/* Dense fp64 product of the same fp16-rounded operands for rows [r0, r1);
 * Cd holds (r1-r0) x N doubles. */
ORC_API void orc_gemm_dense_f64(const float *Af, const float *Bf, int64_t K, int64_t N,
                                int64_t r0, int64_t r1, double *Cd) {
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t r = r0; r < r1; r++) {
        double *out = Cd + (r - r0) * N;
        for (int64_t c = 0; c < N; c++) out[c] = 0.0;
        for (int64_t k = 0; k < K; k++) {
            const double a = (double)Af[r * K + k];
            if (a == 0.0) continue;
            const float *br = Bf + k * N;
            for (int64_t c = 0; c < N; c++) out[c] += a * (double)br[c];
        }
    }
}

/* --------------------------------------------------------------- metrics */

/* out[0] = ||X - Y||_F, out[1] = ||Y||_F, out[2] = ||X||_F, fp64 accumulation
 * (the reference's error triple, tool.cu:6-24, printed in fp32 there). */
ORC_API void orc_frob_diff(const float *X, const double *Y, int64_t n, double *out) {
    double e = 0, y = 0, x = 0;
#pragma omp parallel for schedule(static) reduction(+ : e, y, x)
    for (int64_t i = 0; i < n; i++) {
        double d = (double)X[i] - Y[i];
        e += d * d;
        y += Y[i] * Y[i];
        x += (double)X[i] * (double)X[i];
    }
    out[0] = sqrt(e); out[1] = sqrt(y); out[2] = sqrt(x);
}

ORC_API void orc_frob_diff_f32(const float *X, const float *Y, int64_t n, double *out) {
    double e = 0, y = 0, x = 0;
#pragma omp parallel for schedule(static) reduction(+ : e, y, x)
    for (int64_t i = 0; i < n; i++) {
        double d = (double)X[i] - (double)Y[i];
        e += d * d;
        y += (double)Y[i] * (double)Y[i];
        x += (double)X[i] * (double)X[i];
    }
    out[0] = sqrt(e); out[1] = sqrt(y); out[2] = sqrt(x);
}

/* tau-derived bound on ||C_spamm - C_exact||_F from the dropped norm products:
 * sqrt( sum_ij ( sum_{k dropped} nA[i,k]*nB[k,j] )^2 ), tile rows [ti0,ti1). */
ORC_API double orc_dropped_bound(const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                                 int64_t nbN, float tau, int64_t ti0, int64_t ti1) {
    double tot = 0;
    (void)nbM;
#pragma omp parallel for schedule(static) reduction(+ : tot)
    for (int64_t i = ti0; i < ti1; i++) {
        for (int64_t j = 0; j < nbN; j++) {
            double s = 0;
            for (int64_t k = 0; k < nbK; k++) {
                volatile float p = nA[i * nbK + k] * nB[k * nbN + j];
                if (!(p >= tau)) s += (double)nA[i * nbK + k] * (double)nB[k * nbN + j];
            }
            tot += s * s;
        }
    }
    return sqrt(tot);
}

/* The same sums per output tile: out[i*nbN + j] = sum over dropped k of nA[i,k]*nB[k,j] (the bound
 * on the Frobenius error of tile (i,j)); orc_dropped_bound is the root of the sum of their squares. */
ORC_API void orc_dropped_bound_tiles(const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                                     int64_t nbN, float tau, double *out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nbM; i++) {
        for (int64_t j = 0; j < nbN; j++) {
            double s = 0;
            for (int64_t k = 0; k < nbK; k++) {
                volatile float p = nA[i * nbK + k] * nB[k * nbN + j];
                if (!(p >= tau)) s += (double)nA[i * nbK + k] * (double)nB[k * nbN + j];
            }
            out[i * nbN + j] = s;
        }
    }
}

/* ---------------------------------------------------------- tau selection */

static int cmp_float_desc(const void *a, const void *b) {
    float x = *(const float *)a, y = *(const float *)b;
    return x < y ? 1 : (x > y ? -1 : 0);
}

/* Smallest-error tau for a target kept ratio: the ceil(ratio*total)-th largest
 * fp32 norm product (so that exactly the products >= tau are kept; ties may
 * push the achieved ratio above the target).  Returns tau; *achieved gets the
 * kept ratio at that tau.  If fewer positive products exist than requested the
 * smallest positive product is returned (tau = 0 would keep everything). */
ORC_API float orc_tau_for_ratio(const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                                int64_t nbN, double ratio, double *achieved) {
    const int64_t total = nbM * nbN * nbK;
    float *p = (float *)malloc(sizeof(float) * (size_t)total);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nbM; i++)
        for (int64_t j = 0; j < nbN; j++)
            for (int64_t k = 0; k < nbK; k++) {
                volatile float v = nA[i * nbK + k] * nB[k * nbN + j];
                p[(i * nbN + j) * nbK + k] = v;
            }
    qsort(p, (size_t)total, sizeof(float), cmp_float_desc);
    int64_t want = (int64_t)ceil(ratio * (double)total);
    if (want < 1) want = 1;
    if (want > total) want = total;
    float tau = p[want - 1];
    if (!(tau > 0.0f)) {            /* ran into the zero tail: take the smallest positive */
        int64_t lo = 0, hi = want - 1;
        while (lo < hi) { int64_t mid = (lo + hi) / 2; if (p[mid] > 0.0f) lo = mid + 1; else hi = mid; }
        tau = lo > 0 ? p[lo - 1] : 0.0f;
    }
    int64_t kept = 0;
    for (int64_t i = 0; i < total; i++) if (p[i] >= tau) kept++; else break;
    if (achieved) *achieved = (double)kept / (double)total;
    free(p);
    return tau;
}

/* The reference's bisection (tool.cu:438-490): iteration 0 measures the ratio at
 * tau = 0 and sets tau to the mean product; later rounds bisect between
 * down/up, doubling `up` while the ratio is still too high; stops when
 * |ratio - expected| < tol or after max_rounds.  Products and comparisons are
 * in double as there (norm is a double product of two floats). */
ORC_API float orc_tune_bisect(const float *nA, const float *nB, int64_t nbM, int64_t nbK, int64_t nbN,
                              double expected, double tol, int max_rounds, double *achieved) {
    const int64_t total = nbM * nbN * nbK;
    double Norm = 0, up = 0, down = 0, rate = 0;
    for (int Ti = 0; Ti < max_rounds; Ti++) {
        int64_t count = 0;
        double ave = 0;
#pragma omp parallel for schedule(static) reduction(+ : count, ave)
        for (int64_t i = 0; i < nbM; i++)
            for (int64_t j = 0; j < nbN; j++)
                for (int64_t k = 0; k < nbK; k++) {
                    double norm = (double)(float)(nA[i * nbK + k] * nB[k * nbN + j]);
                    ave += norm;
                    if (norm >= Norm) count++;
                }
        rate = (double)(float)((float)count / (float)total);
        if (fabs(rate - expected) < tol) break;
        if (Ti == 0) { Norm = ave / (double)total; up = Norm; continue; }
        if (rate > expected) {
            if (up == Norm) up *= 2;
            down = Norm;
            Norm = (Norm + up) / 2;
        } else {
            up = Norm;
            Norm = (Norm + down) / 2;
        }
    }
    if (achieved) *achieved = rate;
    return (float)Norm;
}
