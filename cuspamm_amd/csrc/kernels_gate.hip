// Stage 2: the tau gate.
//
// Replaces the gating prologue that the reference re-runs inside every
// multiply block (cuSpAMM.cu:302-334): bitmap of nA[i,k]*nB[k,j] >= tau
// (fp32 multiply, fp32 compare, :305-306), serial O(n^2) compaction
// (:315-325) and a shared-memory tree count (:328-334).  Here one workgroup
// owns one macro tile (256 x 256 elements of C = MT x MT output tiles):
//   phase 1  each wave takes output tiles of the macro tile in turn; 64 k per
//            ballot, popcount/mbcnt gives every kept k its slot in the
//            ascending list; per-tile bitmap, list and count go to memory and
//            the bitmap words also to LDS;
//   phase 2  union of the MT*MT bitmaps per 64-k word, popcount per word, an
//            LDS prefix sum over the words, then every kept k of the union is
//            written at its prefix position together with the bit set of
//            tiles that keep it.  The union list is what the gated GEMM walks;
//            its length and the kept-product total are the work counts used to
//            order macro tiles for load balance.
#include "spamm_internal.h"

namespace spamm {

__global__ __launch_bounds__(256) void k_gate(GateBuffers g, int nbM, int nbK, int nbN, int MT,
                                              int nMacN, float tau) {
    extern __shared__ uint64_t smem[];
    const int words = (nbK + 63) >> 6;
    const int NT = MT * MT;
    uint64_t *lmask = smem;                                   // [NT][words]
    int *wsum = reinterpret_cast<int *>(smem + (size_t)NT * words);   // [words + 1] prefix
    __shared__ int s_work;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int macro = blockIdx.x;
    const int mi = macro / nMacN, mj = macro % nMacN;
    if (threadIdx.x == 0) s_work = 0;
    __syncthreads();

    // ---- phase 1: per output tile bitmap + ascending list + count
    int my_work = 0;
    for (int t = wave; t < NT; t += 4) {
        const int i = mi * MT + t / MT, j = mj * MT + t % MT;
        const bool inside = i < nbM && j < nbN;
        const float *ra = g.nA + (int64_t)i * nbK;
        const float *rb = g.nBt + (int64_t)j * nbK;
        const int64_t tid = (int64_t)i * nbN + j;
        int base = 0;
        for (int w = 0; w < words; w++) {
            const int k = w * 64 + lane;
            bool keep = false;
            if (inside && k < nbK) {
                const float p = ra[k] * rb[k];
                keep = p >= tau;
            }
            const uint64_t m = __ballot(keep);
            if (keep) {
                const int pos = base + __builtin_popcountll(m & ((1ull << lane) - 1ull));
                g.klist[tid * nbK + pos] = (uint16_t)k;
            }
            base += __builtin_popcountll(m);
            if (lane == 0) {
                lmask[(size_t)t * words + w] = m;
                if (inside) g.mask[tid * words + w] = m;
            }
        }
        if (inside && lane == 0) g.counts[tid] = base;
        my_work += base;
    }
    if (lane == 0) atomicAdd(&s_work, my_work);
    __syncthreads();

    // ---- phase 2: union list with per-tile bits
    for (int w = threadIdx.x; w < words; w += 256) {
        uint64_t u = 0;
        for (int t = 0; t < NT; t++) u |= lmask[(size_t)t * words + w];
        wsum[w + 1] = __builtin_popcountll(u);
    }
    if (threadIdx.x == 0) wsum[0] = 0;
    __syncthreads();
    // inclusive scan over words (Hillis-Steele in LDS; words is small)
    for (int off = 1; off <= words; off <<= 1) {
        int add[4];
        int n = 0;
        for (int w = threadIdx.x; w <= words; w += 256) add[n++] = w >= off ? wsum[w - off] : 0;
        __syncthreads();
        n = 0;
        for (int w = threadIdx.x; w <= words; w += 256) wsum[w] += add[n++];
        __syncthreads();
    }
    for (int k = threadIdx.x; k < nbK; k += 256) {
        const int w = k >> 6, b = k & 63;
        uint64_t u = 0, bits = 0;
        for (int t = 0; t < NT; t++) {
            const uint64_t m = lmask[(size_t)t * words + w];
            u |= m;
            bits |= ((m >> b) & 1ull) << t;
        }
        if ((u >> b) & 1ull) {
            const int pos = wsum[w] + __builtin_popcountll(u & ((1ull << b) - 1ull));
            uint32_t need = 0;
            for (int a = 0; a < MT; a++) {
                const uint32_t rowbits = (uint32_t)(bits >> (a * MT)) & ((1u << MT) - 1u);
                if (rowbits) need |= 1u << a;
                need |= rowbits << 8;
            }
            MacroEntry en;
            en.k = (uint32_t)k;
            en.need = need;
            en.mask_lo = (uint32_t)bits;
            en.mask_hi = (uint32_t)(bits >> 32);
            g.macro_list[(int64_t)macro * nbK + pos] = en;
        }
    }
    if (threadIdx.x == 0) {
        g.macro_count[macro] = wsum[words];
        g.macro_work[macro] = s_work;
    }
}

// Orders macro tiles by descending work (counting sort over quantised work)
// and totals the kept products.  One workgroup; n_macro is at most a few tens
// of thousands.
__global__ __launch_bounds__(1024) void k_order(GateBuffers g, int n_macro, int max_work) {
    constexpr int NB = 1024;
    __shared__ int hist[NB];
    __shared__ int start[NB];
    __shared__ unsigned long long total;
    for (int b = threadIdx.x; b < NB; b += blockDim.x) hist[b] = 0;
    if (threadIdx.x == 0) total = 0;
    __syncthreads();
    unsigned long long mine = 0;
    for (int m = threadIdx.x; m < n_macro; m += blockDim.x) {
        const int wk = g.macro_work[m];
        mine += (unsigned long long)wk;
        const int key = (int)(((int64_t)wk * (NB - 1)) / max_work);
        atomicAdd(&hist[NB - 1 - key], 1);          // bucket 0 = heaviest
    }
    atomicAdd(&total, mine);
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        for (int b = 0; b < NB; b++) { start[b] = acc; acc += hist[b]; }
        *g.kept_total = (int64_t)total;
    }
    __syncthreads();
    for (int m = threadIdx.x; m < n_macro; m += blockDim.x) {
        const int wk = g.macro_work[m];
        const int key = (int)(((int64_t)wk * (NB - 1)) / max_work);
        const int pos = atomicAdd(&start[NB - 1 - key], 1);
        g.order[pos] = m;
    }
}

size_t gate_lds_bytes(int tile, int64_t nbK) {
    const int MT = macro_dim(tile);
    const size_t words = (size_t)((nbK + 63) / 64);
    return (size_t)MT * MT * words * 8 + (words + 1) * 4 + 8;
}

hipError_t launch_gate(const GateBuffers &g, int64_t nbM, int64_t nbK, int64_t nbN, int tile,
                       float tau, hipStream_t s) {
    const int MT = macro_dim(tile);
    const int nMacM = (int)((nbM + MT - 1) / MT), nMacN = (int)((nbN + MT - 1) / MT);
    const int n_macro = nMacM * nMacN;
    const size_t lds = gate_lds_bytes(tile, nbK);
    k_gate<<<n_macro, 256, lds, s>>>(g, (int)nbM, (int)nbK, (int)nbN, MT, nMacN, tau);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int max_work = (int)(MT * MT * nbK);
    k_order<<<1, 1024, 0, s>>>(g, n_macro, max_work);
    return hipGetLastError();
}

}  // namespace spamm
