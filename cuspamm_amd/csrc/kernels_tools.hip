// Error-report tooling around the multiply (not on the hot path).
//
// The reference compares SpAMM against a dense cuBLAS product and prints
// ||C_dense - C_spamm||_F, ||C_dense||_F, ||C_spamm||_F (check_simple_gpu,
// tool.cu:227-280; COUNTERRTRANS, tool.cu:6-24).  Here the dense product is
// an exact fp64 product of the same fp16 operands, formed on the fp64 matrix
// pipeline (v_mfma_f64_16x16x4_f64) block by block and reduced on the fly (it is
// never stored), next to the tau-derived bound
// sqrt(sum_ij (sum_{k dropped} nA[i,k]*nB[k,j])^2).
#include "spamm_internal.h"

namespace spamm {

typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2t __attribute__((ext_vector_type(2)));

// One workgroup (4 waves, 2 x 2) per 64 x 64 block of C; a wave owns 32 x 32 = 2 x 2 blocks of
// v_mfma_f64_16x16x4_f64 (16 accumulator doubles per lane).  Operands come straight from the packed
// fp16 copies: a packed 16-byte vector holds 8 consecutive k of one row (A) / column (B), and the
// four lanes that share a row in the MFMA's 16 x 4 operand take one aligned pair of halves each
// (lane group q = lane / 16 takes k = 8 G + 2 q and 8 G + 2 q + 1 of k-group G), so a k-group is
// two MFMA steps per block and one 4-byte load per lane per operand block.  Which k goes to which
// step is the same for A and B, and the sum over k does not care.  fp16 -> fp64 is exact.
__global__ __launch_bounds__(256) void k_error_dense(const _Float16 *__restrict__ pA, const _Float16 *__restrict__ pB,
                                                     int64_t K, int64_t N, int tile, const float *__restrict__ C,
                                                     int64_t row0, int64_t nblk_n, double *__restrict__ out3) {
    __shared__ double red[3];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int64_t br = row0 + (int64_t)(blockIdx.x / nblk_n) * 64 + wr * 32, bc = (int64_t)(blockIdx.x % nblk_n) * 64 + wc * 32;
    const int64_t nbK = K / tile;
    const int64_t tile_halves = (int64_t)tile * tile;
    const int l16 = lane & 15, q = lane >> 4;
    if (threadIdx.x < 3) red[threadIdx.x] = 0.0;
    // per operand block t (16 rows / columns): offset in halves of this lane's pair inside k-group 0 of k tile 0
    int64_t offA[2], offB[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int64_t r = br + t * 16 + l16, cn = bc + t * 16 + l16;
        offA[t] = (r / tile) * nbK * tile_halves + (r % tile) * 8 + 2 * q;
        offB[t] = (cn / tile) * nbK * tile_halves + (cn % tile) * 8 + 2 * q;
    }
    f64x4 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) acc[a][b] = f64x4{0.0, 0.0, 0.0, 0.0};
    const int qn = tile / 8;                    // k-groups per k tile
    for (int64_t kt = 0; kt < nbK; kt++) {
        for (int g = 0; g < qn; g++) {
            const int64_t koff = kt * tile_halves + (int64_t)g * tile * 8;
            half2t a[2], b[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                a[t] = *reinterpret_cast<const half2t *>(pA + offA[t] + koff);
                b[t] = *reinterpret_cast<const half2t *>(pB + offB[t] + koff);
            }
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int ta = 0; ta < 2; ta++)
#pragma unroll
                    for (int tb = 0; tb < 2; tb++)
                        acc[ta][tb] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)(float)a[ta][s], (double)(float)b[tb][s],
                                                                           acc[ta][tb], 0, 0, 0);
        }
    }
    // accumulator i of lane l in block (ta, tb): row 4 i + l / 16, column l % 16
    double e2 = 0, d2 = 0, c2 = 0;
#pragma unroll
    for (int ta = 0; ta < 2; ta++)
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const double c = (double)C[(br + ta * 16 + 4 * i + q) * N + bc + tb * 16 + l16];
                const double d = acc[ta][tb][i];
                e2 += (c - d) * (c - d);
                d2 += d * d;
                c2 += c * c;
            }
    for (int off = 32; off > 0; off >>= 1) {
        e2 += __shfl_down(e2, off, 64);
        d2 += __shfl_down(d2, off, 64);
        c2 += __shfl_down(c2, off, 64);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&red[0], e2);
        atomicAdd(&red[1], d2);
        atomicAdd(&red[2], c2);
    }
    __syncthreads();
    if (threadIdx.x < 3) atomicAdd(&out3[threadIdx.x], red[threadIdx.x]);
}

__global__ __launch_bounds__(256) void k_dropped_bound(const float *__restrict__ nA, const float *__restrict__ nBt,
                                                       int nbM, int nbK, int nbN, float tau,
                                                       double *__restrict__ out, double *__restrict__ per_tile) {
    // one wave per output tile
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= (int64_t)nbM * nbN) return;
    const int64_t i = t / nbN, j = t % nbN;
    double s = 0.0;
    for (int k = lane; k < nbK; k += 64) {
        const float a = nA[i * nbK + k], b = nBt[j * nbK + k];
        const float p = a * b;
        if (!(p >= tau)) s += (double)a * (double)b;
    }
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off, 64);
    if (lane == 0) {
        atomicAdd(out, s * s);
        if (per_tile) per_tile[t] = s;
    }
}

__global__ void k_clear_f64(double *p, int n) {
    if ((int)threadIdx.x < n) p[threadIdx.x] = 0.0;
}

hipError_t launch_error_vs_dense(const void *packedA, const void *packedB, int64_t M, int64_t K, int64_t N,
                                 int tile, const float *C, int64_t row0, int64_t row1, double *out3,
                                 hipStream_t s) {
    (void)M;
    const int64_t nblk_n = N / 64, nblk_m = (row1 - row0) / 64;
    k_clear_f64<<<1, 64, 0, s>>>(out3, 3);
    k_error_dense<<<(unsigned)(nblk_m * nblk_n), 256, 0, s>>>((const _Float16 *)packedA, (const _Float16 *)packedB, K,
                                                              N, tile, C, row0, nblk_n, out3);
    return hipGetLastError();
}

hipError_t launch_dropped_bound(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN,
                                float tau, double *out1, double *per_tile, hipStream_t s) {
    k_clear_f64<<<1, 64, 0, s>>>(out1, 1);
    const int64_t nt = nbM * nbN;
    k_dropped_bound<<<(unsigned)((nt + 3) / 4), 256, 0, s>>>(nA, nBt, (int)nbM, (int)nbK, (int)nbN, tau, out1, per_tile);
    return hipGetLastError();
}

}  // namespace spamm
