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
    int *wsum = reinterpret_cast<int *>(smem + (size_t)NT * words);   // 2 x [words + 1] prefixes
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
        // four 64-k words per step: their norm loads are in flight together (each is a cache round trip)
        for (int w0 = 0; w0 < words; w0 += 4) {
            float pa[4], pb[4];
            uint64_t mword = 0;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int k = (w0 + u) * 64 + lane;
                const bool live = inside && k < nbK;
                pa[u] = live ? ra[k] : 0.0f;
                pb[u] = live ? rb[k] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int w = w0 + u;
                if (w >= words) break;
                const int k = w * 64 + lane;
                bool keep = false;
                if (inside && k < nbK) {
                    const float p = pa[u] * pb[u];
                    keep = p >= tau;
                }
                const uint64_t m = __ballot(keep);
                if (keep) {
                    const int pos = base + __builtin_popcountll(m & ((1ull << lane) - 1ull));
                    g.klist[tid * nbK + pos] = (uint16_t)k;
                }
                base += __builtin_popcountll(m);
                if (lane == u) mword = m;              // lane u keeps word w0 + u
            }
            // one store of up to four words per step instead of one per word
            if (lane < 4 && w0 + lane < words) {
                lmask[(size_t)t * words + w0 + lane] = mword;
                if (inside) g.mask[tid * words + w0 + lane] = mword;
            }
        }
        if (inside && lane == 0) g.counts[tid] = base;
        my_work += base;
    }
    if (lane == 0) atomicAdd(&s_work, my_work);
    __syncthreads();

    // ---- phase 2: union list with per-tile bits.  Entries whose k is kept by
    // every tile of the macro tile ("full") come first, then the partial ones,
    // each group in ascending k: the GEMM runs a branch-free loop over the
    // first group.
    int *wfull = wsum;                       // [words + 1] prefix of full entries
    int *wpart = wsum + (words + 1);         // [words + 1] prefix of partial entries
    for (int w = threadIdx.x; w < words; w += 256) {
        uint64_t u = 0, f = ~0ull;
        for (int t = 0; t < NT; t++) {
            const uint64_t m = lmask[(size_t)t * words + w];
            u |= m;
            f &= m;
        }
        wfull[w + 1] = __builtin_popcountll(f);
        wpart[w + 1] = __builtin_popcountll(u & ~f);
    }
    if (threadIdx.x == 0) { wfull[0] = 0; wpart[0] = 0; }
    __syncthreads();
    // inclusive scans over words (Hillis-Steele in LDS; words is small)
    for (int off = 1; off <= words; off <<= 1) {
        int addf[5], addp[5];        // words <= 1024: at most 5 per thread
        int n = 0;
        for (int w = threadIdx.x; w <= words; w += 256) {
            addf[n] = w >= off ? wfull[w - off] : 0;
            addp[n] = w >= off ? wpart[w - off] : 0;
            n++;
        }
        __syncthreads();
        n = 0;
        for (int w = threadIdx.x; w <= words; w += 256) {
            wfull[w] += addf[n];
            wpart[w] += addp[n];
            n++;
        }
        __syncthreads();
    }
    const int n_full = wfull[words];
    const int n_part = wpart[words];
    // Each group is rotated to start at an anchor k shared by the whole super
    // tile (the k where its diagonal would sit): the workgroups of a super
    // tile run together on one XCD, and walking k from a common start keeps
    // them on the same A row panels and B column panels at the same time.
    int rot_f = 0, rot_p = 0;              // entries of each group below the anchor
    {
        const int mMT = nMacN > 0 ? MT : MT;
        const int sm = mi / SUPER_M, sn = mj / SUPER_N;
        const float ic = ((sm * SUPER_M + 0.5f * SUPER_M) * mMT) / (float)nbM;
        const float jc = ((sn * SUPER_N + 0.5f * SUPER_N) * mMT) / (float)nbN;
        float fa = 0.5f * (ic + jc) * (float)nbK - 0.5f * SUPER_N * mMT;
        int anchor = (int)fa;
        anchor = anchor < 0 ? 0 : (anchor > nbK - 1 ? nbK - 1 : anchor);
        const int wa = anchor >> 6, ba = anchor & 63;
        uint64_t u = 0, f = ~0ull;
        for (int t = 0; t < NT; t++) {
            const uint64_t m = lmask[(size_t)t * words + wa];
            u |= m;
            f &= m;
        }
        const uint64_t below = (1ull << ba) - 1ull;
        rot_f = wfull[wa] + __builtin_popcountll(f & below);
        rot_p = wpart[wa] + __builtin_popcountll(u & ~f & below);
    }
    for (int k = threadIdx.x; k < nbK; k += 256) {
        const int w = k >> 6, b = k & 63;
        uint64_t u = 0, f = ~0ull, bits = 0;
        for (int t = 0; t < NT; t++) {
            const uint64_t m = lmask[(size_t)t * words + w];
            u |= m;
            f &= m;
            bits |= ((m >> b) & 1ull) << t;
        }
        if ((u >> b) & 1ull) {
            const uint64_t below = (1ull << b) - 1ull;
            int pos;
            if ((f >> b) & 1ull) {
                pos = wfull[w] + __builtin_popcountll(f & below) - rot_f;
                if (pos < 0) pos += n_full;
            } else {
                pos = wpart[w] + __builtin_popcountll(u & ~f & below) - rot_p;
                if (pos < 0) pos += n_part;
                pos += n_full;
            }
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
        g.macro_count[2 * macro] = n_full + n_part;
        g.macro_count[2 * macro + 1] = n_full;
        g.macro_work[macro] = s_work;
    }
}

// Schedule for the GEMM.  Macro tiles are grouped into super tiles of
// SUPER_M x SUPER_N (= 32, one per CU of an XCD); workgroups are dispatched
// round-robin over the 8 XCDs, so workgroup b runs on XCD b % 8 and is the
// (b / 8)-th workgroup that XCD starts.
//   1. Super tiles are ranked by descending kept-product count and dealt to
//      the XCDs in snake order: every XCD owns whole super tiles, so the
//      workgroups sharing one L2 share A row panels and B column panels, and
//      the XCDs get equal work.
//   2. Inside an XCD the macro tiles are ordered by work level (SCHED_LEVELS
//      classes of the kept-product count, heaviest first) and, inside a
//      level, in super-tile order.  With two levels (computing / nothing
//      kept) the computing macro tiles simply run super tile by super tile:
//      measured on banded inputs, finer heaviest-first classes did not
//      shorten the tail but pulled neighbours apart (10 % more L2 misses).
//   3. Macro tiles with nothing kept come last in each XCD's sequence: their
//      workgroups only write zeros and start when CUs fall idle at the end.
// Output: order[x * P + q] = macro tile id of XCD x's q-th workgroup,
// sched[x] = number of computing items, sched[8 + x] = number of all items.
// One workgroup; O(n^2) ranking over at most a few thousand super tiles.
__global__ __launch_bounds__(1024) void k_order(GateBuffers g, int nMacM, int nMacN, int nSupN,
                                                int n_super, int rounds) {
    extern __shared__ int swork[];               // [n_super] work, then reused: [n_super] id by rank
    int *srank_id = swork + n_super;
    __shared__ unsigned long long total;
    __shared__ int maxwork;
    const int P = rounds * SUPER_M * SUPER_N;
    if (threadIdx.x == 0) { total = 0; maxwork = 1; }
    __syncthreads();
    unsigned long long mine = 0;
    int mymax = 0;
    for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) {
        const int sm = sid / nSupN, sn = sid % nSupN;
        int w = 0;
        for (int a = 0; a < SUPER_M; a++)
            for (int b = 0; b < SUPER_N; b++) {
                const int mi = sm * SUPER_M + a, mj = sn * SUPER_N + b;
                if (mi < nMacM && mj < nMacN) {
                    const int mw = g.macro_work[mi * nMacN + mj];
                    w += mw;
                    mymax = mw > mymax ? mw : mymax;
                }
            }
        swork[sid] = w;
        mine += (unsigned long long)w;
    }
    atomicAdd(&total, mine);
    atomicMax(&maxwork, mymax);
    __syncthreads();
    for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) {
        const int w = swork[sid];
        int rank = 0;
        for (int j = 0; j < n_super; j++) {
            const int wj = swork[j];
            rank += (wj > w) || (wj == w && j < sid);
        }
        srank_id[rank] = sid;
    }
    for (int i = threadIdx.x; i < NUM_XCD * P; i += blockDim.x) g.order[i] = -1;
    __syncthreads();

    // item of XCD x at raw position p (round-major, then slot), or -1; level of that item
    const int mw_max = maxwork;
    auto item_at = [&](int x, int p, int &level) -> int {
        const int round = p / (SUPER_M * SUPER_N), slot = p % (SUPER_M * SUPER_N);
        const int sr = round * NUM_XCD + ((round & 1) ? NUM_XCD - 1 - x : x);
        if (sr >= n_super) return -1;
        const int sid = srank_id[sr];
        const int mi = (sid / nSupN) * SUPER_M + slot / SUPER_N, mj = (sid % nSupN) * SUPER_N + slot % SUPER_N;
        if (mi >= nMacM || mj >= nMacN) return -1;
        const int m = mi * nMacN + mj;
        const int mw = g.macro_work[m];
        level = mw > 0 ? 1 + (int)(((int64_t)(mw - 1) * (SCHED_LEVELS - 1)) / mw_max) : 0;
        return m;
    };
    // raw sequence (round-major, slot-minor) with the level in the top byte, in the upper half of `order`
    int32_t *raw = g.order + NUM_XCD * P;
    for (int i = threadIdx.x; i < NUM_XCD * P; i += blockDim.x) {
        int level = 0;
        const int m = item_at(i / P, i % P, level);
        raw[i] = m >= 0 ? (m | (level << 24)) : -1;
    }
    __syncthreads();
    // one wave per XCD: count per level, prefix (heaviest level first, empty tiles last), stable scatter
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (wave < NUM_XCD) {
        const int x = wave;
        const int32_t *rx = raw + x * P;
        int mycnt = 0;                       // lane lv < SCHED_LEVELS keeps the count of level lv
        // (loads of UN chunks are issued together: the wave is alone here and each one is an L2 round trip)
        constexpr int UN = 8;
        for (int p0 = 0; p0 < P; p0 += 64 * UN) {
            int vv[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int p = p0 + u * 64 + lane;
                vv[u] = p < P ? rx[p] : -1;
            }
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int level = vv[u] >= 0 ? (vv[u] >> 24) : -1;
#pragma unroll
                for (int lv = 0; lv < SCHED_LEVELS; lv++) {
                    const int c = __builtin_popcountll(__ballot(level == lv));
                    if (lane == lv) mycnt += c;
                }
            }
        }
        // exclusive prefix over levels in descending order: base(lv) = sum of counts of levels > lv
        int base = 0, ncomp = 0, nall = 0;
#pragma unroll
        for (int lv = SCHED_LEVELS - 1; lv >= 0; lv--) {
            const int c = __shfl(mycnt, lv, 64);
            if (lane == lv) base = nall;
            if (lv == 0) ncomp = nall;
            nall += c;
        }
        if (lane == 0) {
            g.sched[x] = ncomp;
            g.sched[NUM_XCD + x] = nall;
        }
        for (int p0 = 0; p0 < P; p0 += 64 * UN) {
            int vv[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int p = p0 + u * 64 + lane;
                vv[u] = p < P ? rx[p] : -1;
            }
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const int v = vv[u];
                const int level = v >= 0 ? (v >> 24) : -1;
                int pos = -1;
#pragma unroll
                for (int lv = 0; lv < SCHED_LEVELS; lv++) {
                    const uint64_t bal = __ballot(level == lv);
                    const int b0 = __shfl(base, lv, 64);
                    if (level == lv) pos = b0 + __builtin_popcountll(bal & ((1ull << lane) - 1ull));
                    if (lane == lv) base += __builtin_popcountll(bal);
                }
                if (pos >= 0) g.order[x * P + pos] = v & 0xffffff;
            }
        }
    }
    if (threadIdx.x == 0) g.kept_total[0] = (int64_t)total;
}

size_t gate_lds_bytes(int tile, int64_t nbK) {
    const int MT = macro_dim(tile);
    const size_t words = (size_t)((nbK + 63) / 64);
    return (size_t)MT * MT * words * 8 + 2 * (words + 1) * 4 + 8;
}

// k_gate may use all of a CU's LDS for the macro tile's bitmaps (its workgroups are short)
hipError_t gate_init() {
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gate), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)gate_lds_limit());
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
    const int nSupM = (nMacM + SUPER_M - 1) / SUPER_M, nSupN = (nMacN + SUPER_N - 1) / SUPER_N;
    const int n_super = nSupM * nSupN;
    const int rounds = (n_super + NUM_XCD - 1) / NUM_XCD;
    k_order<<<1, 1024, (size_t)n_super * 2 * sizeof(int), s>>>(g, nMacM, nMacN, nSupN, n_super, rounds);
    return hipGetLastError();
}

}  // namespace spamm
