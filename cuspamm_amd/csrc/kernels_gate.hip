// Stage 2: the tau gate.
//
// Replaces the gating prologue that the reference re-runs inside every
// multiply block (cuSpAMM.cu:302-334): bitmap of nA[i,k]*nB[k,j] >= tau
// (fp32 multiply, fp32 compare, :305-306), serial O(n^2) compaction
// (:315-325) and a shared-memory tree count (:328-334).  Here one workgroup
// owns one macro tile (256 x 256 elements of C = MT x MT output tiles):
//   phase 1  a wave takes a block of up to 4 x 4 output tiles and 64 k at a
//            time: it loads the 4 + 4 norms once per lane, forms the 16
//            products in registers and ballots each comparison into the
//            tile's 64-bit bitmap word, kept in LDS;
//   phase 2  per-tile counts and the bitmaps go to memory; then every 64-k
//            word of the MT*MT bitmaps is transposed across a wave (lane =
//            k), which gives each k the bit set of tiles that keep it, the
//            union and the kept-by-all word; an LDS prefix sum over the words
//            places every kept k of the union in the macro tile's list.  The
//            union list is what the gated GEMM walks; its length and the
//            kept-product total are the work counts used to order macro tiles
//            for load balance.
// The reference's compacted per-tile list (offset[], :315-325) is the bitmap's
// set bits in ascending order; nothing downstream reads it, so it is produced
// from the bitmap only when asked for (k_klist).
#include <type_traits>

#include "spamm_internal.h"

namespace spamm {

// 64 x 64 bit-matrix transpose across a wave: lane t holds row t; on return
// lane b holds column b (bit t of the result = bit b of lane t's input).
// Six butterfly steps, each swapping the off-diagonal j x j blocks of lane
// pairs (l, l ^ j).
__device__ __forceinline__ uint64_t transpose64(uint64_t x, int lane) {
    constexpr uint64_t MASKS[6] = {0x00000000FFFFFFFFull, 0x0000FFFF0000FFFFull, 0x00FF00FF00FF00FFull,
                                   0x0F0F0F0F0F0F0F0Full, 0x3333333333333333ull, 0x5555555555555555ull};
#pragma unroll
    for (int s = 0; s < 6; s++) {
        const int j = 32 >> s;
        const uint64_t y = (uint64_t)__shfl_xor((long long)x, j, 64);
        const bool upper = (lane & j) == 0;              // this lane is the row without bit j
        const uint64_t ru = upper ? x : y, rl = upper ? y : x;
        const uint64_t t = ((ru >> j) ^ rl) & MASKS[s];
        x ^= upper ? (t << j) : t;
    }
    return x;
}

// lo[lane idx] = low word, hi[lane idx] = high word of a wave-uniform 64-bit m; idx must fold to
// a constant (unrolled loops).  On gfx90a and later a VALU instruction that reads an SGPR needs
// two wait states after the VALU instruction that wrote it (here: the compare behind the ballot).
// The compiler inserts them only around instructions it can see, not around inline assembly, so
// the s_nop is part of it.
__device__ __forceinline__ void set_lane2(int &lo, int &hi, uint64_t m, int idx) {
    // (readfirstlane: under register pressure the compiler may hold the uniform words in VGPRs)
    const int mlo = __builtin_amdgcn_readfirstlane((int)(uint32_t)m);
    const int mhi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(m >> 32));
    asm("s_nop 1\n\tv_writelane_b32 %0, %2, %4\n\tv_writelane_b32 %1, %3, %4"
        : "+v"(lo), "+v"(hi)
        : "s"(mlo), "s"(mhi), "n"(idx));
}

template <int MT>
struct GateCfg {
    static constexpr int NT = MT * MT;             // output tiles per macro tile
    static constexpr int NTP = NT < 8 ? 8 : NT;    // bitmap rows per 64-k word in LDS (a transposed word needs 64 * NTP bits)
    static constexpr int BT = MT < 4 ? MT : 4;     // a wave's block of tiles per dimension
    static constexpr int QD = MT / BT;
    static constexpr int NQ = QD * QD;
    static constexpr uint64_t FULL = NT == 64 ? ~0ull : ((1ull << NT) - 1ull);
};

// NTH threads per workgroup: 256, or 64 for macro tiles of 2 x 2 output tiles (tile 128), whose
// four tiles give three of four waves nothing to do: one wave per macro tile lets four times as
// many macro tiles be in flight on a CU, and this kernel's time is memory latency.
template <int MT, bool ONE, int NTH = (MT == 2 ? 64 : 256)>
__global__ __launch_bounds__(NTH) void k_gate(GateBuffers g, int nbM, int nbK, int nbN, int nMacN, float tau, int cw_arg) {
    using G = GateCfg<MT>;
    constexpr int NW = NTH / 64;
    constexpr int NT = G::NT, NTP = G::NTP, BT = G::BT;
    extern __shared__ uint64_t smem[];
    const int words = (nbK + 63) >> 6;
    // LDS holds the tile bitmaps of `cw` 64-k words at a time (cw = words unless K / tile is so
    // large that a macro tile's bitmaps exceed a CU's LDS: then the k range is walked in chunks,
    // twice -- once to count, once to place the list entries -- and the bitmaps of a chunk are
    // recomputed for the second walk); the per-word summaries below cover all words.  ONE: the
    // instantiation for cw = words, straight-line code without the chunk loop.
    constexpr bool one_chunk = ONE;
    const int cw = ONE ? words : cw_arg;
    uint64_t *lmask = smem;                                  // [cw][NTP]: tile bitmaps, later transposed in place
    uint64_t *luf = smem + (size_t)cw * NTP;                 // [words][2]: union word, kept-by-all word
    int *wfull = reinterpret_cast<int *>(luf + 2 * (size_t)words);   // [words + 1] prefix of full entries
    int *wpart = wfull + (words + 1);                        // [words + 1] prefix of partial entries

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int macro = blockIdx.x;
    const int mi = macro / nMacN, mj = macro % nMacN;

    // ---- phase 1: bitmaps.  Item = (64-k word, block of BT x BT tiles); two items per step so
    // that their norm loads are in flight together (each is a cache round trip).  Loads are
    // unconditional from clamped addresses; what lies outside the matrix is masked after the
    // ballot (k per lane, tile rows / columns per wave).
    struct Item {
        float pa[BT], pb[BT];
    };
    auto load_item = [&](int w0, int item, Item &it) {
        const int q = item % G::NQ, w = w0 + item / G::NQ;
        const int k = w * 64 + lane;
        const int kc = k < nbK ? k : nbK - 1;
#pragma unroll
        for (int a = 0; a < BT; a++) {
            const int i = mi * MT + (q / G::QD) * BT + a;
            it.pa[a] = g.nA[(int64_t)(i < nbM ? i : nbM - 1) * nbK + kc];
        }
#pragma unroll
        for (int b = 0; b < BT; b++) {
            const int j = mj * MT + (q % G::QD) * BT + b;
            it.pb[b] = g.nBt[(int64_t)(j < nbN ? j : nbN - 1) * nbK + kc];
        }
    };
    // whole macro tile inside the matrix: only the last k word may need masking
    const bool interior = (mi + 1) * MT <= nbM && (mj + 1) * MT <= nbN;
    auto gate_item = [&](int w0, int item, const Item &it) {
        const int q = item % G::NQ, wl = item / G::NQ, w = w0 + wl;
        const int ti0 = (q / G::QD) * BT, tj0 = (q % G::QD) * BT;
        int mlo = 0, mhi = 0;                 // lane a*BT+b collects the word of tile (a, b)
        if (interior && (w + 1) * 64 <= nbK) {
#pragma unroll
            for (int a = 0; a < BT; a++)
#pragma unroll
                for (int b = 0; b < BT; b++) {
                    const uint64_t m = __ballot(it.pa[a] * it.pb[b] >= tau);
                    set_lane2(mlo, mhi, m, a * BT + b);
                }
        } else {
            const uint64_t kmask = __ballot(w * 64 + lane < nbK);
#pragma unroll
            for (int a = 0; a < BT; a++)
#pragma unroll
                for (int b = 0; b < BT; b++) {
                    // wave-uniform all-ones / zero: is tile (a, b) of the block inside the matrix
                    const uint64_t inside =
                        0ull - (uint64_t)((mi * MT + ti0 + a < nbM) & (mj * MT + tj0 + b < nbN));
                    const uint64_t m = __ballot(it.pa[a] * it.pb[b] >= tau) & kmask & inside;
                    set_lane2(mlo, mhi, m, a * BT + b);
                }
        }
        if (lane < BT * BT)
            lmask[(size_t)wl * NTP + (ti0 + lane / BT) * MT + tj0 + lane % BT] =
                ((uint64_t)(uint32_t)mhi << 32) | (uint32_t)mlo;
    };
    auto build_bitmaps = [&](int w0, int cwn) {
        const int n_items = G::NQ * cwn;
        for (int it0 = wave; it0 < n_items; it0 += 2 * NW) {
            const int it1 = it0 + NW;
            Item i0, i1;
            load_item(w0, it0, i0);
            if (it1 < n_items) load_item(w0, it1, i1);
            gate_item(w0, it0, i0);
            if (it1 < n_items) gate_item(w0, it1, i1);
        }
    };
    // ---- phase 2b: transpose every word in place: entry b of word w becomes the set of tiles
    // (bit t = tile t of the macro tile) that keep k = 64 w + b, NTP bits wide
    auto tile_bits = [&](int wl, int b) -> uint64_t {
        if constexpr (NTP == 64) return lmask[(size_t)wl * 64 + b];
        else if constexpr (NTP == 16) return reinterpret_cast<const uint16_t *>(lmask + (size_t)wl * 16)[b];
        else return reinterpret_cast<const uint8_t *>(lmask + (size_t)wl * 8)[b];
    };
    auto transpose_words = [&](int w0, int cwn, bool record) {
        for (int wl = wave; wl < cwn; wl += NW) {
            const uint64_t row = lane < NT ? lmask[(size_t)wl * NTP + lane] : 0ull;
            const uint64_t bits = transpose64(row, lane);
            const uint64_t u = __ballot(bits != 0ull), f = __ballot(bits == G::FULL);
            // the wave has read all rows of the word before any lane writes its column
            if constexpr (NTP == 64) lmask[(size_t)wl * 64 + lane] = bits;
            else if constexpr (NTP == 16) reinterpret_cast<uint16_t *>(lmask + (size_t)wl * 16)[lane] = (uint16_t)bits;
            else reinterpret_cast<uint8_t *>(lmask + (size_t)wl * 8)[lane] = (uint8_t)bits;
            if (record && lane == 0) {
                const int w = w0 + wl;
                luf[2 * w] = u;
                luf[2 * w + 1] = f;
                wfull[w + 1] = __builtin_popcountll(f);
                wpart[w + 1] = __builtin_popcountll(u & ~f);
            }
        }
    };

    int cnt = 0;                               // wave 0, lane < NT: kept k of tile `lane`
    int n_full = 0, n_part = 0, rot_f = 0, rot_p = 0;
    // One walk over the k chunks; `pass` is a compile-time tag: 0 counts, 1 places.
    auto walk = [&](auto pass_tag) {
        constexpr int pass = decltype(pass_tag)::value;
        int w0 = 0;
        do {
            const int cwn = words - w0 < cw ? words - w0 : cw;
            if constexpr (pass == 0 || !one_chunk) {
                build_bitmaps(w0, cwn);
                __syncthreads();
            }
            if constexpr (pass == 0) {
                // ---- phase 2a: per-tile counts and the bitmaps to memory
                if (wave == 0 && lane < NT)
                    for (int wl = 0; wl < cwn; wl++) cnt += __builtin_popcountll(lmask[(size_t)wl * NTP + lane]);
                const float inv_words = 1.0f / (float)cwn;     // e < 2^16, cwn <= 1024: the quotient below is exact
                for (int e = threadIdx.x; e < NT * cwn; e += NTH) {
                    const int t = (int)(((float)e + 0.5f) * inv_words), wl = e - t * cwn;
                    const int i = mi * MT + t / MT, j = mj * MT + t % MT;
                    if (i < nbM && j < nbN) g.mask[((int64_t)i * nbN + j) * words + w0 + wl] = lmask[(size_t)wl * NTP + t];
                }
                __syncthreads();
            }
            if constexpr (pass == 0 || !one_chunk) {
                transpose_words(w0, cwn, pass == 0);
                __syncthreads();
            }
            if constexpr (pass == 1) {
                // ---- phase 2c: union list with per-tile bits.  Entries whose k is kept by every
                // tile of the macro tile ("full") come first, then the partial ones, each group
                // in ascending k rotated to the anchor: the GEMM runs a branch-free loop over the
                // first group.
                const int k1 = (w0 + cwn) * 64 < nbK ? (w0 + cwn) * 64 : nbK;
                for (int k = w0 * 64 + threadIdx.x; k < k1; k += NTH) {
                    const int w = k >> 6, b = k & 63;
                    const uint64_t bits = tile_bits(w - w0, b);
                    if (bits != 0ull) {
                        const uint64_t u = luf[2 * w], f = luf[2 * w + 1];
                        const uint64_t below = (1ull << b) - 1ull;
                        int pos;
                        if (bits == G::FULL) {
                            pos = wfull[w] + __builtin_popcountll(f & below) - rot_f;
                            if (pos < 0) pos += n_full;
                        } else {
                            pos = wpart[w] + __builtin_popcountll(u & ~f & below) - rot_p;
                            if (pos < 0) pos += n_part;
                            pos += n_full;
                        }
                        uint32_t need = 0;
#pragma unroll
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
                if constexpr (!one_chunk) __syncthreads();     // the next chunk's bitmaps overwrite these
            }
            w0 += cw;
        } while (!ONE && w0 < words);
    };
    walk(std::integral_constant<int, 0>{});
    // ---- between the walks: inclusive scans over the words give each word's offset in its group
    if (threadIdx.x == 0) { wfull[0] = 0; wpart[0] = 0; }
    __syncthreads();
    if (words < 64) {
        if (wave == 0) {
            int vf = lane <= words ? wfull[lane] : 0, vp = lane <= words ? wpart[lane] : 0;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int tf = __shfl_up(vf, off, 64), tp = __shfl_up(vp, off, 64);
                if (lane >= off) { vf += tf; vp += tp; }
            }
            if (lane <= words) { wfull[lane] = vf; wpart[lane] = vp; }
        }
        __syncthreads();
    } else {
        // Hillis-Steele in LDS
        for (int off = 1; off <= words; off <<= 1) {
            int addf[1024 / NTH + 1], addp[1024 / NTH + 1];        // words <= 1024
            int n = 0;
            for (int w = threadIdx.x; w <= words; w += NTH) {
                addf[n] = w >= off ? wfull[w - off] : 0;
                addp[n] = w >= off ? wpart[w - off] : 0;
                n++;
            }
            __syncthreads();
            n = 0;
            for (int w = threadIdx.x; w <= words; w += NTH) {
                wfull[w] += addf[n];
                wpart[w] += addp[n];
                n++;
            }
            __syncthreads();
        }
    }
    n_full = wfull[words];
    n_part = wpart[words];
    // Each group is rotated to start at an anchor k shared by the whole super
    // tile (the k where its diagonal would sit): the workgroups of a super
    // tile run together on one XCD, and walking k from a common start keeps
    // them on the same A row panels and B column panels at the same time.
    {
        const int sm = mi / SUPER_M, sn = mj / SUPER_N;
        const float ic = ((sm * SUPER_M + 0.5f * SUPER_M) * MT) / (float)nbM;
        const float jc = ((sn * SUPER_N + 0.5f * SUPER_N) * MT) / (float)nbN;
        const float fa = 0.5f * (ic + jc) * (float)nbK - 0.5f * SUPER_N * MT;
        int anchor = (int)fa;
        anchor = anchor < 0 ? 0 : (anchor > nbK - 1 ? nbK - 1 : anchor);
        const int wa = anchor >> 6, ba = anchor & 63;
        const uint64_t u = luf[2 * wa], f = luf[2 * wa + 1];
        const uint64_t below = (1ull << ba) - 1ull;
        rot_f = wfull[wa] + __builtin_popcountll(f & below);     // entries of each group below the anchor
        rot_p = wpart[wa] + __builtin_popcountll(u & ~f & below);
    }
    walk(std::integral_constant<int, 1>{});
    // per-tile counts and the macro tile's kept-product total
    int work = 0;
    if (wave == 0) {
        if (lane < NT) {
            const int i = mi * MT + lane / MT, j = mj * MT + lane % MT;
            if (i < nbM && j < nbN) g.counts[(int64_t)i * nbN + j] = cnt;
        }
        work = cnt;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) work += __shfl_xor(work, off, 64);
    }
    if (threadIdx.x == 0) {
        g.macro_count[2 * macro] = n_full + n_part;
        g.macro_count[2 * macro + 1] = n_full;
        g.macro_work[macro] = work;
    }
}

// Schedule for the GEMM.  Macro tiles are grouped into super tiles of
// SUPER_M x SUPER_N (= 32, one per CU of an XCD); workgroups are dispatched
// round-robin over the n_xcd XCDs of the device, so workgroup b runs on XCD
// b % n_xcd and is the (b / n_xcd)-th workgroup that XCD starts (n_xcd = 1: one
// flat sequence, for devices that are not whole XCDs of 32 CUs).
//   1. Super tiles are ranked by descending length (entries of their macro
//      tiles' union lists: that, not the kept-product count, is the time a
//      workgroup takes) and dealt to the XCDs: every XCD owns whole super
//      tiles, so the workgroups sharing one L2 share A row panels and B column
//      panels.  Up to LPT_MAX_SUPER super tiles are dealt greedily, each to the
//      XCD with the least length so far (at most `rounds` per XCD, the size
//      the grid and the order buffer are laid out for); a plain snake deal by
//      rank leaves XCDs up to 18 % apart when a problem has only a few super
//      tiles per XCD, and the slowest XCD sets the kernel's time.  Beyond that
//      size the deal is the snake (the serial greedy loop would take longer
//      than it saves, and many super tiles per XCD even out by themselves).
//   2. Inside an XCD the computing macro tiles run super tile by super tile
//      (measured on banded inputs, heaviest-first classes inside an XCD did
//      not shorten the tail but pulled neighbours apart: 10 % more L2 misses).
//   3. Macro tiles with nothing kept come last in each XCD's sequence: their
//      workgroups only write zeros and start when CUs fall idle at the end.
// Output: order[x * P + q] = macro tile id of XCD x's q-th workgroup for
// q < sched[8 + x] (entries beyond are not written), sched[x] = number of
// computing items, sched[8 + x] = number of all items.
// One workgroup; O(n^2) ranking over at most a few thousand super tiles.
__global__ __launch_bounds__(1024) void k_order(GateBuffers g, int nMacM, int nMacN, int nSupN,
                                                int n_super, int rounds, int n_xcd) {
    extern __shared__ __attribute__((aligned(16))) int swork[];               // [n_super] length, then [n_super] super tile origin by rank,
    int *srank_id = swork + n_super;             // then (greedy deal only) [n_xcd][rounds] rank of each XCD's r-th super tile
    uint16_t *sdeal = reinterpret_cast<uint16_t *>(srank_id + n_super);
    __shared__ unsigned long long total;
    __shared__ int s_nonempty;
    const int P = rounds * SUPER_M * SUPER_N;
    if (threadIdx.x == 0) { total = 0; s_nonempty = 0; }
    // (this kernel is one workgroup on an idle GPU: its run time is memory round trips and
    // instruction fetch, so every thread takes one macro tile row of one super tile -- all loads
    // of the kernel's first step are in flight at once -- and the code is kept small)
    for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) swork[sid] = 0;
    __syncthreads();
    unsigned long long mine = 0;
    for (int e = threadIdx.x; e < n_super * SUPER_M; e += blockDim.x) {
        const int sid = e / SUPER_M, a = e % SUPER_M;
        const int mi = (sid / nSupN) * SUPER_M + a, mj0 = (sid % nSupN) * SUPER_N;
        int w = 0, len = 0;
#pragma unroll
        for (int b = 0; b < SUPER_N; b++)
            if (mi < nMacM && mj0 + b < nMacN) {
                w += g.macro_work[mi * nMacN + mj0 + b];
                len += g.macro_count[2 * (mi * nMacN + mj0 + b)];
            }
        if (len) atomicAdd(&swork[sid], len);
        mine += (unsigned long long)w;
    }
    if (mine) atomicAdd(&total, mine);
    __syncthreads();
    // How the super tiles are dealt to the XCDs (sdeal, or the snake formula in macro_at):
    //   DEAL_LPT    few super tiles hold work: ranked by length, each goes to the XCD with the
    //               least length so far (pure balance; ~0.2 us of serial work per super tile);
    //   DEAL_BAND   at most BAND_DEAL_MAX super tiles hold work (the deal is serial, ~1.2 us
    //               per group; at N = 65536 it cost more than it gained) and they are at most
    //               60 % of all (a narrow band): ranked in
    //               row-major order, those with work first; every group of n_xcd consecutive
    //               ones -- neighbours along the band that read the same operand panels -- runs
    //               at the same time, one per XCD, and inside a group the heaviest goes to the
    //               XCD with the least length so far.  Measured against the snake: -4 to -6 %
    //               GEMM time on exponential-decay bands that keep 10 % (N = 16384), -2 % at
    //               N = 32768, but +1 to +3 % when most super tiles hold work (algebraic decay,
    //               30 % kept), hence the condition;
    //   DEAL_SNAKE  ranked by length, dealt in snake order (no table: any number of super tiles).
    //   DEAL_FLAT   fewer super tiles than XCDs (C of at most 7 x 32 macro tiles): whole super tiles
    //               would leave XCDs empty -- 2048^3 at tile 32 is two of them, 64 workgroups on a
    //               quarter of the chip -- so the macro tiles themselves are dealt, consecutive
    //               ones in row-major order (neighbours along a row share the A panel) in equal
    //               chunks, one per XCD; no ranking (the problem is a few microseconds long).
    enum { DEAL_LPT, DEAL_BAND, DEAL_SNAKE, DEAL_FLAT };
    {
        int ne = 0;
        for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) ne += swork[sid] > 0;
        if (ne) atomicAdd(&s_nonempty, ne);
    }
    __syncthreads();
    const int n_ne = s_nonempty;
    const int deal = n_super < n_xcd ? DEAL_FLAT
                     : n_super > LPT_MAX_SUPER ? DEAL_SNAKE
                     : (n_ne <= LPT_GREEDY_MAX ? DEAL_LPT
                        : (n_ne <= BAND_DEAL_MAX && 5 * n_ne <= 3 * n_super ? DEAL_BAND : DEAL_SNAKE));
    const int flat_chunk = (nMacM * nMacN + n_xcd - 1) / n_xcd;      // <= P: n_super < n_xcd super tiles of 32
    // Ranking: larger key first, equal keys by smaller index; the key is the length, or in the
    // band deal just "holds work".  srank_id[rank] becomes the super tile's origin.
    //   up to RANK_SORT_MIN super tiles: rank = number of super tiles that come first, n_super^2
    //   comparisons with the j range cut into `parts` pieces so that all 1024 threads take part
    //   (partial ranks meet in srank_id, used as a counter first);
    //   beyond: a bitonic sort of the indices in LDS (padded to a power of two with indices
    //   >= n_super, which sort last): log^2 steps of one compare-exchange per thread instead of
    //   n_super comparisons per super tile on this one CU (150 us at 2048 super tiles).
    constexpr int RANK_SORT_MIN = 512;
    if (deal == DEAL_FLAT) {
        // nothing to rank
    } else if (n_super <= RANK_SORT_MIN) {
        const bool band = deal == DEAL_BAND;
        int parts = 2;
        while (parts < 32 && n_super * parts * 2 <= (int)blockDim.x) parts *= 2;
        for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) srank_id[sid] = 0;
        __syncthreads();
        const int chunk = (n_super + parts - 1) / parts;
        // (two copies of the loop, one per key, so that the inner loop is a read, two compares and an add)
        auto count_first = [&](auto key) {
            for (int e = threadIdx.x; e < n_super * parts; e += blockDim.x) {
                const int sid = e % n_super, part = e / n_super;
                const int w = key(swork[sid]);
                const int j1 = (part + 1) * chunk < n_super ? (part + 1) * chunk : n_super;
                int rank = 0;
                for (int j = part * chunk; j < j1; j++) {
                    const int kj = key(swork[j]);
                    rank += (kj > w) || (kj == w && j < sid);
                }
                if (rank) atomicAdd(&srank_id[sid], rank);
            }
        };
        if (band) count_first([](int v) { return (int)(v > 0); });
        else count_first([](int v) { return v; });
        __syncthreads();
        const int sid = threadIdx.x;              // n_super <= RANK_SORT_MIN < blockDim.x: one super tile per thread
        const int rank = sid < n_super ? srank_id[sid] : 0;
        __syncthreads();
        if (sid < n_super) {
            srank_id[rank] = ((sid / nSupN) * SUPER_M) << 16 | ((sid % nSupN) * SUPER_N);   // first macro tile row, column
            if (deal != DEAL_SNAKE) sdeal[sid] = (uint16_t)rank;       // parked: rank of super tile sid (read back below)
        }
    } else {
        int np2 = 2 * RANK_SORT_MIN;
        while (np2 < n_super) np2 <<= 1;
        int *sidx = srank_id;                     // [np2]: runs into sdeal's space, which is not in use yet
        for (int i = threadIdx.x; i < np2; i += blockDim.x) sidx[i] = i;
        __syncthreads();
        auto sort_by = [&](auto key) {
            for (int k = 2; k <= np2; k <<= 1)
                for (int j = k >> 1; j > 0; j >>= 1) {
                    for (int t = threadIdx.x; t < np2 / 2; t += blockDim.x) {
                        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), l = i | j;
                        const int a = sidx[i], b = sidx[l];
                        const int ka = a < n_super ? key(swork[a]) : -1, kb = b < n_super ? key(swork[b]) : -1;
                        const bool a_first = ka > kb || (ka == kb && a < b);
                        if (a_first != ((i & k) == 0)) { sidx[i] = b; sidx[l] = a; }
                    }
                    __syncthreads();
                }
        };
        if (deal == DEAL_BAND) sort_by([](int v) { return (int)(v > 0); });
        else sort_by([](int v) { return v; });
        // sidx[rank] = super tile; every thread turns its own slots into origins
        for (int r = threadIdx.x; r < n_super; r += blockDim.x) {
            const int sid = sidx[r];
            srank_id[r] = ((sid / nSupN) * SUPER_M) << 16 | ((sid % nSupN) * SUPER_N);
            if (deal != DEAL_SNAKE) sdeal[sid] = (uint16_t)r;
        }
    }
    __syncthreads();
    if (deal != DEAL_SNAKE && deal != DEAL_FLAT) {
        // lengths by rank, then the deal by one wave
        int mylen[(LPT_MAX_SUPER + 1023) / 1024], myrank[(LPT_MAX_SUPER + 1023) / 1024];
        int n = 0;
        for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) { mylen[n] = swork[sid]; myrank[n] = sdeal[sid]; n++; }
        __syncthreads();
        n = 0;
        for (int sid = threadIdx.x; sid < n_super; sid += blockDim.x) { swork[myrank[n]] = mylen[n]; n++; }
        __syncthreads();
        if (threadIdx.x < 64 && deal == DEAL_LPT) {
            // lane x < n_xcd keeps XCD x's length so far and its number of super tiles; the
            // least-loaded XCD with room is the minimum of (length, lane) over the lanes
            // (lengths stay far below 2^28: at most LPT_GREEDY_MAX super tiles of 32 lists)
            const int x = threadIdx.x;
            uint32_t load = 0;
            int cnt = 0;
            for (int r = 0; r < n_ne; r++) {
                uint32_t key = (x < n_xcd && cnt < rounds) ? (load << 3) | (uint32_t)x : ~0u;
#pragma unroll
                for (int off = 1; off < MAX_XCD; off <<= 1) {
                    const uint32_t o = (uint32_t)__shfl_xor((int)key, off, 64);
                    key = o < key ? o : key;
                }
                if ((int)(key & 7u) == x) {
                    sdeal[x * rounds + cnt] = (uint16_t)r;
                    cnt++;
                    load += (uint32_t)swork[r];
                }
            }
            // super tiles with nothing kept (ranks n_ne ..) fill the XCDs' remaining slots in lane order
            const int room = x < n_xcd ? rounds - cnt : 0;
            int before = room;
#pragma unroll
            for (int off = 1; off < MAX_XCD; off <<= 1) {
                const int o = __shfl_up(before, off, 64);
                if (x >= off) before += o;
            }
            before -= room;
            for (int c = 0; c < room; c++) {
                const int r = n_ne + before + c;
                sdeal[x * rounds + cnt + c] = r < n_super ? (uint16_t)r : (uint16_t)0xffffu;   // 0xffff: no super tile
            }
        }
        if (threadIdx.x < 64 && deal == DEAL_BAND) {
            // lane x < 8 holds the x-th super tile of the group and the length of XCD x so far; the
            // 64 lanes compare all pairs at once (lane 8 i + j: i against j), so that the ranks of
            // the eight super tiles (heaviest first) and of the eight XCDs (shortest first) are
            // byte-wise popcounts of two ballots, and the match -- the super tile whose rank is the
            // XCD's rank -- the lowest set bit of a third
            const int x = threadIdx.x;
            const int pi = x >> 3, pj = x & 7;
            int load = 0, cnt = 0;
            const int ngroups = (n_ne + n_xcd - 1) / n_xcd;
            for (int g2 = 0; g2 < ngroups; g2++) {
                const int r = g2 * n_xcd + x;
                const int w = (x < n_xcd && r < n_ne) ? swork[r] : -1;           // -1: no super tile
                const int wi = __shfl(w, pi, 64), wj = __shfl(w, pj, 64);
                const int li = __shfl(load, pi, 64), lj = __shfl(load, pj, 64);
                const uint64_t heavier = __ballot((wj > wi) || (wj == wi && pj < pi));
                const uint64_t shorter = __ballot(pj < n_xcd && ((lj < li) || (lj == li && pj < pi)));
                const int irank_j = __builtin_popcountll((heavier >> (8 * pj)) & 0xffull);
                const int xrank_i = __builtin_popcountll((shorter >> (8 * pi)) & 0xffull);
                const uint64_t match = __ballot(pi < n_xcd && pj < n_xcd && irank_j == xrank_i);
                const uint32_t mybyte = (uint32_t)((match >> (8 * (x & 7))) & 0xffull);     // lanes x < 8: row x
                const int mine = mybyte ? __builtin_ctz(mybyte) : 0;
                const int wm = __shfl(w, mine, 64);
                if (x < n_xcd && mybyte && wm > 0) {   // (the last group may have fewer super tiles than XCDs)
                    sdeal[x * rounds + cnt] = (uint16_t)(g2 * n_xcd + mine);
                    cnt++;
                    load += wm;
                }
            }
            // super tiles with nothing kept (ranks n_ne ..) fill the XCDs' remaining slots in lane order
            const int room = x < n_xcd ? rounds - cnt : 0;
            int before = room;
#pragma unroll
            for (int off = 1; off < MAX_XCD; off <<= 1) {
                const int o = __shfl_up(before, off, 64);
                if (x >= off) before += o;
            }
            before -= room;
            for (int c = 0; c < room; c++) {
                const int r = n_ne + before + c;
                sdeal[x * rounds + cnt + c] = r < n_super ? (uint16_t)r : (uint16_t)0xffffu;   // 0xffff: no super tile
            }
        }
        __syncthreads();
    }

    // macro tile of XCD x at raw position p (round-major, then slot inside the super tile), or -1
    auto macro_at = [&](int x, int p) -> int {
        const int round = p / (SUPER_M * SUPER_N), slot = p % (SUPER_M * SUPER_N);
        if (p >= P) return -1;
        if (deal == DEAL_FLAT) return (p < flat_chunk && x * flat_chunk + p < nMacM * nMacN) ? x * flat_chunk + p : -1;
        const int sr = deal != DEAL_SNAKE ? (int)sdeal[x * rounds + round] : round * n_xcd + ((round & 1) ? n_xcd - 1 - x : x);
        if (sr >= n_super) return -1;
        const int origin = srank_id[sr];
        const int mi = (origin >> 16) + slot / SUPER_N, mj = (origin & 0xffff) + slot % SUPER_N;
        return (mi < nMacM && mj < nMacN) ? mi * nMacN + mj : -1;
    };
    // one wave per XCD: computing macro tiles to the front in raw order, empty ones from the back
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (wave < n_xcd) {
        const int x = wave;
        int nall = 0;                            // macro tiles in this XCD's sequence (no memory access)
        for (int p0 = 0; p0 < P; p0 += 64) nall += __builtin_popcountll(__ballot(macro_at(x, p0 + lane) >= 0));
        int nc = 0, ne = 0;
        const uint64_t below = (1ull << lane) - 1ull;
        // (loads of UN chunks are issued together: the wave is alone here and each one is an L2 round trip)
        constexpr int UN = 8;
        for (int p0 = 0; p0 < P; p0 += 64 * UN) {
            int mm[UN], ww[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                mm[u] = macro_at(x, p0 + u * 64 + lane);
                ww[u] = mm[u] >= 0 ? g.macro_work[mm[u]] : 0;
            }
#pragma unroll
            for (int u = 0; u < UN; u++) {
                const bool comp = mm[u] >= 0 && ww[u] > 0, empty = mm[u] >= 0 && ww[u] <= 0;
                const uint64_t bc = __ballot(comp), be = __ballot(empty);
                if (comp) g.order[x * P + nc + __builtin_popcountll(bc & below)] = mm[u];
                if (empty) g.order[x * P + nall - 1 - (ne + __builtin_popcountll(be & below))] = mm[u];
                nc += __builtin_popcountll(bc);
                ne += __builtin_popcountll(be);
            }
        }
        if (lane == 0) {
            g.sched[x] = nc;
            g.sched[MAX_XCD + x] = nall;
            g.sched[2 * MAX_XCD + x] = 0;      // ticket counter of the persistent GEMM
        }
    }
    if (threadIdx.x == 0) g.kept_total[0] = (int64_t)total;
}

// Per-tile ascending list of kept k (the reference's offset[], cuSpAMM.cu:315-325)
// from the gate's bitmaps: one wave per output tile, popcount below the lane's
// bit gives every kept k its slot.
__global__ __launch_bounds__(256) void k_klist(const uint64_t *__restrict__ mask, uint16_t *__restrict__ klist,
                                               int64_t n_tiles, int nbK, int words) {
    const int lane = threadIdx.x & 63;
    const int64_t tid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tid >= n_tiles) return;
    int base = 0;
    for (int w = 0; w < words; w++) {
        const uint64_t m = mask[tid * words + w];
        if ((m >> lane) & 1ull)
            klist[tid * nbK + base + __builtin_popcountll(m & ((1ull << lane) - 1ull))] = (uint16_t)(w * 64 + lane);
        base += __builtin_popcountll(m);
    }
}

hipError_t launch_klist(const uint64_t *mask, uint16_t *klist, int64_t n_tiles, int64_t nbK, hipStream_t s) {
    k_klist<<<(unsigned)((n_tiles + 3) / 4), 256, 0, s>>>(mask, klist, n_tiles, (int)nbK, (int)((nbK + 63) / 64));
    return hipGetLastError();
}

// A macro tile's bitmaps take words * NTP * 8 bytes of LDS (tile 32: 512 bytes per 64 k tiles)
// beside 24 bytes of summaries per word; what does not fit a CU's LDS is walked in chunks of
// gate_chunk_words() words; `cap` > 0 (a context's developer knob) forces smaller chunks so that
// ordinary shapes take the chunked path.
static size_t gate_fixed_bytes(size_t words) { return words * 16 + 2 * (words + 1) * 4; }

int gate_chunk_words(int tile, int64_t nbK, int cap) {
    const int MT = macro_dim(tile);
    const size_t ntp = MT * MT < 8 ? 8 : MT * MT;
    const size_t words = (size_t)((nbK + 63) / 64);
    size_t cw = (gate_lds_limit() - gate_fixed_bytes(words)) / (ntp * 8);
    if (cap > 0 && cw > (size_t)cap) cw = (size_t)cap;
    return (int)(cw < words ? cw : words);
}

size_t gate_lds_bytes(int tile, int64_t nbK, int cap) {
    const int MT = macro_dim(tile);
    const size_t ntp = MT * MT < 8 ? 8 : MT * MT;
    const size_t words = (size_t)((nbK + 63) / 64);
    return ntp * (size_t)gate_chunk_words(tile, nbK, cap) * 8 + gate_fixed_bytes(words);
}

// k_gate may use all of a CU's LDS for the macro tile's bitmaps (its workgroups are short)
hipError_t gate_init() {
    hipError_t e;
    const void *gates[6] = {reinterpret_cast<const void *>(&k_gate<8, true>), reinterpret_cast<const void *>(&k_gate<8, false>),
                            reinterpret_cast<const void *>(&k_gate<4, true>), reinterpret_cast<const void *>(&k_gate<4, false>),
                            reinterpret_cast<const void *>(&k_gate<2, true>), reinterpret_cast<const void *>(&k_gate<2, false>)};
    for (const void *f : gates)
        if ((e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)gate_lds_limit())) != hipSuccess) return e;
    // k_order: its tables may take order_lds_limit() on top of a few static bytes
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&k_order), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)order_lds_limit());
}

hipError_t launch_gate(const GateBuffers &g, int64_t nbM, int64_t nbK, int64_t nbN, int tile,
                       float tau, int n_xcd, int chunk_cap, hipStream_t s) {
    const int MT = macro_dim(tile);
    const int nMacM = (int)((nbM + MT - 1) / MT), nMacN = (int)((nbN + MT - 1) / MT);
    const int n_macro = nMacM * nMacN;
    const size_t lds = gate_lds_bytes(tile, nbK, chunk_cap);
    const int cw = gate_chunk_words(tile, nbK, chunk_cap);
    const bool one = cw >= (int)((nbK + 63) / 64);
#define SPAMM_GATE(MTV)                                                                                          \
    if (one) k_gate<MTV, true><<<n_macro, MTV == 2 ? 64 : 256, lds, s>>>(g, (int)nbM, (int)nbK, (int)nbN, nMacN, tau, cw);      \
    else k_gate<MTV, false><<<n_macro, MTV == 2 ? 64 : 256, lds, s>>>(g, (int)nbM, (int)nbK, (int)nbN, nMacN, tau, cw)
    switch (MT) {
        case 8: SPAMM_GATE(8); break;
        case 4: SPAMM_GATE(4); break;
        case 2: SPAMM_GATE(2); break;
        default: return hipErrorInvalidValue;
    }
#undef SPAMM_GATE
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const int nSupM = (nMacM + SUPER_M - 1) / SUPER_M, nSupN = (nMacN + SUPER_N - 1) / SUPER_N;
    const int n_super = nSupM * nSupN;
    const int rounds = (n_super + n_xcd - 1) / n_xcd;
    k_order<<<1, 1024, order_lds_bytes(tile, nbM, nbN), s>>>(g, nMacM, nMacN, nSupN, n_super, rounds, n_xcd);
    return hipGetLastError();
}

}  // namespace spamm
