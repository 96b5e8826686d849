// spamm_main: the reference's main() (cuSpAMM.cu:395-560) on top of the C ABI of
// include/spamm.h, with the compile-time configuration of para.h / main.h as
// command-line options.  Same flow: build or load A and B on the host
// (tool.cu:282-436), pad to a tile multiple (main.h:54-56), upload, then TESTTIME
// timed multiplies with the first WARMUP + 1 left out of the mean
// (cuSpAMM.cu:458-556), and print the reference's two lines.  Extras the reference
// keeps behind macros: the valid-ratio tuner (tuneValidRate, tool.cu:438-490) and
// the error check (check_simple_gpu, tool.cu:227-280), here against an exact fp64
// product.
//
//   spamm_main [--M m] [--K k] [--N n] [--tile 32|64|128] [--tau t | --ratio r | --tune r]
//              [--gen exp|alg|ones] [--c c] [--v v] [--a-csv f --b-csv f | --a-mtx f --b-mtx f]
//              [--testtime n] [--warmup n] [--check | --prune] [--noalloc | --half] [--device d]
// --half: the operands are rounded to fp16 on the host and resident as fp16 before the timed
// multiplies, as in the reference (USINGHALF 1, para.h:1; __float2half in its generators,
// tool.cu:418,432); without it the fp32 -> fp16 conversion is part of every timed multiply.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/spamm.h"

static int fail(const char *what, int rc) {
    fprintf(stderr, "spamm_main: %s: %s (%d)\n", what, spamm_strerror(rc), rc);
    return 1;
}

int main(int argc, char **argv) {
    long long inM = 2048, inK = 2048, inN = 2048;      // para.h:6-8
    int tile = 32;                                     // LoNum, main.h:32
    double norm_init = 1.548969;                       // NormINIT, para.h:2
    double ratio = -1.0, tune = -1.0;
    std::string gen = "alg";                           // MATRIXALG 1, para.h:14
    float c = 0.1f, v = 0.1f;                          // getDecayMatrixAlg(h, 0.1, 0.1, ...), cuSpAMM.cu:430-431
    bool cv_given = false;
    std::string a_csv, b_csv, a_mtx, b_mtx;
    int testtime = 10, warmup = 5, device = 0;         // TESTTIME, WARMUP, para.h:4-5
    bool check = false, prune = false, noalloc = false, half_in = false;
    for (int i = 1; i < argc; i++) {
        const std::string o = argv[i];
        auto val = [&]() -> const char * { return i + 1 < argc ? argv[++i] : ""; };
        if (o == "--M") inM = atoll(val());
        else if (o == "--K") inK = atoll(val());
        else if (o == "--N") inN = atoll(val());
        else if (o == "--tile") tile = atoi(val());
        else if (o == "--tau") norm_init = atof(val());
        else if (o == "--ratio") ratio = atof(val());
        else if (o == "--tune") tune = atof(val());
        else if (o == "--gen") gen = val();
        else if (o == "--c") { c = (float)atof(val()); cv_given = true; }
        else if (o == "--v") { v = (float)atof(val()); cv_given = true; }
        else if (o == "--a-csv") a_csv = val();
        else if (o == "--b-csv") b_csv = val();
        else if (o == "--a-mtx") a_mtx = val();
        else if (o == "--b-mtx") b_mtx = val();
        else if (o == "--testtime") testtime = atoi(val());
        else if (o == "--warmup") warmup = atoi(val());
        else if (o == "--device") device = atoi(val());
        else if (o == "--check") check = true;
        else if (o == "--prune") prune = true;
        else if (o == "--half") half_in = true;
        else if (o == "--noalloc") noalloc = true;        // the timed multiplies run in the library's fixed workspace
        else { fprintf(stderr, "spamm_main: unknown option %s\n", o.c_str()); return 2; }
    }
    if (gen == "exp" && !cv_given) { c = 1.0f; v = 0.1f; }    // getDecayMatrixExp(h, 1, 0.1, ...), cuSpAMM.cu:426-427
    if (tile != 32 && tile != 64 && tile != 128) { fprintf(stderr, "spamm_main: tile must be 32, 64 or 128\n"); return 2; }
    if (check && prune) { fprintf(stderr, "spamm_main: --check needs A's complete fp16 copy, --prune leaves tiles out\n"); return 2; }
    if (half_in && noalloc) { fprintf(stderr, "spamm_main: --noalloc takes fp32 operands, not --half\n"); return 2; }
    if (inM <= 0 || inK <= 0 || inN <= 0 || testtime <= warmup + 1) { fprintf(stderr, "spamm_main: bad sizes\n"); return 2; }
    // padded dimensions (main.h:54-56)
    const long long M = (inM + tile - 1) / tile * tile, K = (inK + tile - 1) / tile * tile, N = (inN + tile - 1) / tile * tile;
    printf("input parameters: M=%lld K=%lld N=%lld Norm=%f USINGHALF=%d\n", M, K, N, norm_init, 1);

    spamm_ctx *ctx = nullptr;
    int rc = spamm_create(&ctx, device);
    if (rc) return fail("spamm_create", rc);
    float *dA = nullptr, *dB = nullptr, *dC = nullptr;
    if (hipMalloc(&dA, sizeof(float) * M * K) != hipSuccess || hipMalloc(&dB, sizeof(float) * K * N) != hipSuccess ||
        hipMalloc(&dC, sizeof(float) * M * N) != hipSuccess) {
        fprintf(stderr, "spamm_main: out of device memory\n");
        return 1;
    }

    if (!a_csv.empty() || !a_mtx.empty()) {
        // dense CSV (CNN, tool.cu:282-318) or "row col val" (DECAY, tool.cu:320-366), zero padded
        std::vector<float> hA((size_t)M * K), hB((size_t)K * N);
        const bool csv = !a_csv.empty();
        rc = csv ? spamm_load_csv_f32(a_csv.c_str(), inM, inK, K, hA.data()) : spamm_load_mtx_f32(a_mtx.c_str(), inM, inK, K, hA.data());
        if (rc) return fail("loading A", rc);
        rc = csv ? spamm_load_csv_f32(b_csv.c_str(), inK, inN, N, hB.data()) : spamm_load_mtx_f32(b_mtx.c_str(), inK, inN, N, hB.data());
        if (rc) return fail("loading B", rc);
        if (hipMemcpy(dA, hA.data(), sizeof(float) * M * K, hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(dB, hB.data(), sizeof(float) * K * N, hipMemcpyHostToDevice) != hipSuccess) {
            fprintf(stderr, "spamm_main: upload failed\n");
            return 1;
        }
    } else {
        // the reference's generators are functions of |i - j| only (tool.cu:370-436): one table
        const long long n = M > K ? (M > N ? M : N) : (K > N ? K : N);
        std::vector<float> table((size_t)n);
        for (long long d = 0; d < n; d++) {
            if (gen == "exp") table[d] = c * (float)pow((double)v, (double)d);               // tool.cu:413
            else if (gen == "alg") table[d] = c / ((float)pow((double)d, (double)v) + 1.0f);  // tool.cu:430
            else if (gen == "ones") table[d] = 1.0f;                                          // getNormMatrix, tool.cu:370-403
            else { fprintf(stderr, "spamm_main: --gen must be exp, alg or ones\n"); return 2; }
        }
        if ((rc = spamm_fill_decay_f32(ctx, dA, M, K, table.data(), 0, 0))) return fail("generating A", rc);
        if ((rc = spamm_fill_decay_f32(ctx, dB, K, N, table.data(), 0, 0))) return fail("generating B", rc);
    }

    spamm_params p;
    memset(&p, 0, sizeof(p));
    p.M = M; p.K = K; p.N = N; p.tile = tile; p.tau = (float)norm_init; p.flags = SPAMM_FLAG_TIMING | (prune ? SPAMM_FLAG_PRUNE : 0u);
    if (ratio >= 0.0 || tune >= 0.0) {
        // valid-ratio driven tau: exact order statistic, or the reference's bisection (main.h:35-38)
        if ((rc = spamm_normmap_f32(ctx, SPAMM_ROLE_B, dB, K, N, tile))) return fail("norm map of B", rc);
        if ((rc = spamm_normmap_f32(ctx, SPAMM_ROLE_A, dA, M, K, tile))) return fail("norm map of A", rc);
        float tau = 0.0f;
        double achieved = 0.0;
        rc = ratio >= 0.0 ? spamm_tau_for_ratio(ctx, ratio, &tau, &achieved) : spamm_tune_bisect(ctx, tune, 0.01, 20, &tau, &achieved);
        if (rc) return fail("tau selection", rc);
        printf("tuned Norm=%e valid ratio=%f\n", (double)tau, achieved);
        p.tau = tau;
    }

    void *dAh = nullptr, *dBh = nullptr;
    if (half_in) {
        // host-side rounding to fp16 (round to nearest even, what __float2half does), then upload
        auto to_half = [&](const float *dsrc, size_t n, void **dst) -> bool {
            std::vector<float> h32(n);
            std::vector<_Float16> h16(n);
            if (hipMemcpy(h32.data(), dsrc, n * 4, hipMemcpyDeviceToHost) != hipSuccess) return false;
            for (size_t i = 0; i < n; i++) h16[i] = (_Float16)h32[i];
            return hipMalloc(dst, n * 2) == hipSuccess && hipMemcpy(*dst, h16.data(), n * 2, hipMemcpyHostToDevice) == hipSuccess;
        };
        if (!to_half(dA, (size_t)M * K, &dAh) || !to_half(dB, (size_t)K * N, &dBh)) {
            fprintf(stderr, "spamm_main: fp16 copies of the operands failed\n");
            return 1;
        }
    }

    double sum = 0.0;
    spamm_stats st;
    memset(&st, 0, sizeof(st));
    for (int i = 0; i < testtime; i++) {
        if ((rc = half_in ? spamm_multiply_f16(ctx, &p, dAh, dBh, dC)
                          : (noalloc ? spamm_multiply_noalloc(ctx, &p, dA, dB, dC) : spamm_multiply(ctx, &p, dA, dB, dC))))
            return fail(half_in ? "spamm_multiply_f16" : (noalloc ? "spamm_multiply_noalloc" : "spamm_multiply"), rc);
        if ((rc = spamm_get_stats(ctx, &st))) return fail("spamm_get_stats", rc);
        if (i > warmup) sum += st.ms_total * 1e-3;       // cuSpAMM.cu:548
    }
    printf("SpAMM time=%fs\n", sum / (testtime - warmup - 1));
    printf("valid products=%lld of %lld (ratio %f)\n", (long long)st.kept_products, (long long)st.total_products,
           st.total_products ? (double)st.kept_products / (double)st.total_products : 0.0);
    printf("stages: normmap B %.4f ms, normmap A %.4f ms, gate %.4f ms, multiply %.4f ms\n", st.ms_normmap_b,
           st.ms_normmap_a, st.ms_gate, st.ms_gemm);
    if (check) {
        double e3[3] = {0, 0, 0}, bound = 0.0;
        if (M % 64 || N % 64) { fprintf(stderr, "spamm_main: --check needs M and N to be multiples of 64\n"); return 2; }
        if ((rc = spamm_error_vs_dense_f64(ctx, dC, 0, M, e3))) return fail("spamm_error_vs_dense_f64", rc);
        if ((rc = spamm_dropped_bound(ctx, p.tau, &bound))) return fail("spamm_dropped_bound", rc);
        // the reference prints ||C_dense - C||_F, ||C_dense||_F, ||C||_F (tool.cu:270-276)
        printf("error check: |C_dense-C|_F=%e |C_dense|_F=%e |C|_F=%e bound=%e\n", e3[0], e3[1], e3[2], bound);
    }
    if (dAh) (void)hipFree(dAh);
    if (dBh) (void)hipFree(dBh);
    (void)hipFree(dA);
    (void)hipFree(dB);
    (void)hipFree(dC);
    spamm_destroy(ctx);
    return 0;
}
