// tau selection on the device (the reference tunes tau on the host inside the
// timed loop: tuneValidRate, tool.cu:438-490, over managed-memory norm maps).
//
//  - select: exact order statistic.  The fp32 norm products are non-negative,
//    so their bit patterns order like the values; a 3-pass radix select
//    (11 + 11 + 10 bits, most significant first) over the nbM*nbN*nbK products,
//    recomputed from the norm maps in every pass, finds the want-th largest.
//  - count:  number of products >= a threshold and their sum, the two
//    quantities one round of the reference's bisection needs.
#include "spamm_internal.h"

namespace spamm {

__device__ __forceinline__ uint32_t product_key(float a, float b) {
    const float p = a * b;
    return p > 0.0f ? __builtin_bit_cast(uint32_t, p) : 0u;       // NaN and -0 count as 0
}

// Histogram of the `nbits`-wide digit at `shift` over the products whose
// higher bits equal state->prefix.  One workgroup per (i, 16 consecutive j).
__global__ __launch_bounds__(256) void k_tau_hist(const float *__restrict__ nA, const float *__restrict__ nBt,
                                                  int nbM, int nbK, int nbN, int shift, int nbits, int hi_bits,
                                                  const TauState *__restrict__ state,
                                                  unsigned long long *__restrict__ hist) {
    __shared__ unsigned int lh[2048];
    const int nbins = 1 << nbits;
    for (int b = threadIdx.x; b < nbins; b += 256) lh[b] = 0;
    __syncthreads();
    const int jb = (nbN + 15) / 16;
    const int i = blockIdx.x / jb, j0 = (blockIdx.x % jb) * 16;
    const uint32_t prefix = hi_bits ? state->prefix : 0u;
    for (int jj = 0; jj < 16; jj++) {
        const int j = j0 + jj;
        if (j >= nbN) break;
        for (int k = threadIdx.x; k < nbK; k += 256) {
            const uint32_t key = product_key(nA[(int64_t)i * nbK + k], nBt[(int64_t)j * nbK + k]);
            if (hi_bits == 0 || (key >> (shift + nbits)) == prefix) atomicAdd(&lh[(key >> shift) & (nbins - 1)], 1u);
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += 256)
        if (lh[b]) atomicAdd(&hist[b], (unsigned long long)lh[b]);
}

// Walks the histogram from the top bin down to the one holding the wanted
// rank, extends the prefix, clears the histogram for the next pass.
__global__ __launch_bounds__(256) void k_tau_pick(TauState *state, unsigned long long *hist, int nbits, int first,
                                                  int last, unsigned long long want0) {
    const int nbins = 1 << nbits;
    if (threadIdx.x == 0) {
        unsigned long long want = first ? want0 : state->want;
        if (first) state->greater = 0;
        unsigned long long above = 0;
        int bin = nbins - 1;
        for (; bin > 0; bin--) {
            if (above + hist[bin] >= want) break;
            above += hist[bin];
        }
        state->greater += above;
        state->want = want - above;           // rank inside `bin`
        state->prefix = first ? (uint32_t)bin : ((state->prefix << nbits) | (uint32_t)bin);
        if (last) {
            state->tau_bits = state->prefix;
            state->kept = state->greater + hist[bin];
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < nbins; b += 256) hist[b] = 0;
}

// count of products with (double)p >= thr, count of products > 0, and the
// double sum of all products (tool.cu:448-463).
__global__ __launch_bounds__(256) void k_tau_count(const float *__restrict__ nA, const float *__restrict__ nBt,
                                                   int nbM, int nbK, int nbN, double thr,
                                                   unsigned long long *__restrict__ out_count,
                                                   unsigned long long *__restrict__ out_pos,
                                                   double *__restrict__ out_sum) {
    __shared__ unsigned long long s_cnt, s_pos;
    __shared__ double s_sum;
    if (threadIdx.x == 0) { s_cnt = 0; s_pos = 0; s_sum = 0.0; }
    __syncthreads();
    const int jb = (nbN + 15) / 16;
    const int i = blockIdx.x / jb, j0 = (blockIdx.x % jb) * 16;
    unsigned long long c = 0, pz = 0;
    double sum = 0.0;
    for (int jj = 0; jj < 16; jj++) {
        const int j = j0 + jj;
        if (j >= nbN) break;
        for (int k = threadIdx.x; k < nbK; k += 256) {
            const float p = nA[(int64_t)i * nbK + k] * nBt[(int64_t)j * nbK + k];
            if ((double)p >= thr) c++;
            if (p > 0.0f) pz++;
            sum += (double)p;
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        c += __shfl_down(c, off, 64);
        pz += __shfl_down(pz, off, 64);
        sum += __shfl_down(sum, off, 64);
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&s_cnt, c);
        atomicAdd(&s_pos, pz);
        atomicAdd(&s_sum, sum);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(out_count, s_cnt);
        atomicAdd(out_pos, s_pos);
        atomicAdd(out_sum, s_sum);
    }
}

__global__ void k_tau_clear(unsigned long long *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

size_t tau_workspace_bytes() { return sizeof(TauState) + 2048 * 8 + 64; }

// workspace layout: [TauState][pad to 64][hist 2048 x u64][count, pos, sum]
hipError_t launch_tau_select(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN,
                             unsigned long long want, void *workspace, hipStream_t s) {
    TauState *st = (TauState *)workspace;
    unsigned long long *hist = (unsigned long long *)((char *)workspace + 64);
    const int jb = (int)((nbN + 15) / 16);
    const unsigned grid = (unsigned)(nbM * jb);
    k_tau_clear<<<(2048 + 8 + 255) / 256, 256, 0, s>>>((unsigned long long *)workspace, 8 + 2048);
    const int bits[3] = {11, 11, 10};
    int shift = 32;
    for (int pass = 0; pass < 3; pass++) {
        shift -= bits[pass];
        k_tau_hist<<<grid, 256, 0, s>>>(nA, nBt, (int)nbM, (int)nbK, (int)nbN, shift, bits[pass], pass, st, hist);
        k_tau_pick<<<1, 256, 0, s>>>(st, hist, bits[pass], pass == 0, pass == 2, want);
    }
    return hipGetLastError();
}

hipError_t launch_tau_count(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN, double thr,
                            void *workspace, hipStream_t s) {
    unsigned long long *out = (unsigned long long *)((char *)workspace + 64 + 2048 * 8);
    const int jb = (int)((nbN + 15) / 16);
    k_tau_clear<<<1, 256, 0, s>>>(out, 3);
    k_tau_count<<<(unsigned)(nbM * jb), 256, 0, s>>>(nA, nBt, (int)nbM, (int)nbK, (int)nbN, thr, out, out + 1,
                                                    (double *)(out + 2));
    return hipGetLastError();
}

}  // namespace spamm
