// Error-report tooling around the multiply (not on the hot path).
//
// The reference compares SpAMM against a dense cuBLAS product and prints
// ||C_dense - C_spamm||_F, ||C_dense||_F, ||C_spamm||_F (check_simple_gpu,
// tool.cu:227-280; COUNTERRTRANS, tool.cu:6-24).  Here the dense product is
// an exact fp64 product of the same fp16 operands, formed tile by tile and
// reduced on the fly (it is never stored), next to the tau-derived bound
// sqrt(sum_ij (sum_{k dropped} nA[i,k]*nB[k,j])^2).
#include "spamm_internal.h"

namespace spamm {

// fp16 value of element (free index r, contraction index k) of a packed operand
// whose tiles are `tile` wide; `t_major` is the tile row (A) / tile column (B).
__device__ __forceinline__ double packed_at(const _Float16 *p, int64_t nbK, int tile, int64_t r, int64_t k) {
    const int64_t tr = r / tile, tk = k / tile;
    const int ri = (int)(r % tile), ki = (int)(k % tile);
    const int64_t base = (tr * nbK + tk) * (int64_t)tile * tile;
    return (double)p[base + ((int64_t)(ki >> 3) * tile + ri) * 8 + (ki & 7)];
}

// One workgroup per 64 x 64 block of C; thread (ty,tx) owns a 4 x 4 patch.
__global__ __launch_bounds__(256) void k_error_dense(const _Float16 *__restrict__ pA, const _Float16 *__restrict__ pB,
                                                     int64_t K, int64_t N, int tile, const float *__restrict__ C,
                                                     int64_t row0, int64_t nblk_n, double *__restrict__ out3) {
    __shared__ double sA[16][64 + 1];    // [k][row]
    __shared__ double sB[16][64 + 1];    // [k][col]
    __shared__ double red[3];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int64_t br = row0 + (int64_t)(blockIdx.x / nblk_n) * 64, bc = (int64_t)(blockIdx.x % nblk_n) * 64;
    const int64_t nbK = K / tile;
    double acc[4][4] = {};
    if (threadIdx.x < 3) red[threadIdx.x] = 0.0;
    for (int64_t k0 = 0; k0 < K; k0 += 16) {
        __syncthreads();
        for (int e = threadIdx.x; e < 16 * 64; e += 256) {
            const int kk = e & 15, rr = e >> 4;
            sA[kk][rr] = packed_at(pA, nbK, tile, br + rr, k0 + kk);
            sB[kk][rr] = packed_at(pB, nbK, tile, bc + rr, k0 + kk);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
            double a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) { a[i] = sA[kk][ty * 4 + i]; b[i] = sB[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
    }
    double e2 = 0, d2 = 0, c2 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const double c = (double)C[(br + ty * 4 + i) * N + bc + tx * 4 + j];
            const double d = acc[i][j];
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
