// Stage 3: gated tile GEMM on MFMA.
//
// Replaces the product loop of get_C_FP16_B32 (cuSpAMM.cu:336-391): for every
// output tile C_ij the sum over kept k of A_ik * B_kj, fp16 operands, fp32
// accumulation, ascending k.  The reference gives each 32x32 output tile its
// own block and re-fetches both operand tiles per product (16 flop/byte).
// Here one workgroup (4 waves, 2 x 2) owns a macro tile of 256 x 256 elements
// of C; each wave owns a quarter of it, 128 x 128 elements (4 x 4 MFMA 32x32x16
// accumulators = 256 fp32 registers per lane): the tiles in tile rows wr, wr + 2,
// ... and tile columns wc, wc + 2, ... of the macro tile (for tiles of 128 that is
// one tile).  Interleaved, because the tiles that keep a k at the edge of a band
// are a corner of the macro tile: with contiguous quarters one wave would multiply
// all of its tile pairs in such a stage and the opposite wave none.
// The workgroup walks the macro tile's union list of k;
// per entry it stages the needed A tiles (256 rows) and B tiles (256 columns)
// of that k in LDS with direct global->LDS loads (a ring of NBUF stages), and every
// wave multiplies only the (tile row, tile column) pairs whose bit is set in
// the entry's mask, so the kept set is exactly the gate's.
//
// Operands come in the packed layout of spamm_internal.h: a tile's bytes are
// already in MFMA operand order, so staging is a straight copy and every
// ds_read_b128 is 512 contiguous bytes per half wave.
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "spamm_internal.h"

namespace spamm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int B>
struct GemmCfg {
    static constexpr int SUB = 128 / B;              // tiles per wave per dimension
    static constexpr int MT = 2 * SUB;               // tiles per macro tile per dimension
    static constexpr int KS = 32;                    // k depth of one stage
    static constexpr int NSPE = B / KS;              // stages per list entry
    static constexpr int SLOT_BYTES = B * KS * 2;    // one tile's share of a stage
    static constexpr int CPS = SLOT_BYTES / 1024;    // 1 KiB wave-loads per slot
    static constexpr int A_BYTES = MT * SLOT_BYTES;  // 256 rows x KS = 16 KiB
    static constexpr int STAGE_BYTES = 2 * A_BYTES;  // 32 KiB
    static constexpr int TILE_BYTES = B * B * 2;
    static constexpr int RB = B / 32;                // MFMA blocks per tile per dimension
    static constexpr int CHW = MT * CPS / 4;          // 1 KiB chunks per wave per operand per stage
    static constexpr int GS = CPS < 4 ? CPS : 4;     // chunks per load group (share a tile)
    static constexpr int NG = CHW / GS;
    static constexpr int LPW = 2 * CHW;              // load instructions per wave per stage
};

// s_waitcnt immediates (gfx9 encoding: vmcnt [3:0]+[15:14], expcnt [6:4], lgkmcnt [11:8])
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | 0x70 | ((lgkm & 15) << 8); }

// One 1 KiB wave-load straight from global memory into LDS: lane l's 16 bytes
// land at lds_addr + IMM + 16*l, read from sbase + IMM + voff (the instruction
// offset applies to the global and to the LDS address alike).  Written as
// inline assembly so that the compiler's wait-count insertion does not see an
// LDS write it cannot disambiguate (it would put a full vmcnt(0) wait before
// every LDS read and serialise the staging ring); completion is awaited
// explicitly with s_waitcnt vmcnt before the workgroup barrier.  M0 carries
// the LDS address and is declared clobbered, so the compiler keeps nothing
// live in it across a load.  Both scalar operands must come from scalar
// instructions (as all callers' do): a VALU-written SGPR (v_readfirstlane)
// read by a vector-memory instruction within five instructions is a hazard
// the compiler does not see inside inline assembly.
template <int IMM>
__device__ __forceinline__ void dma_load(const unsigned char *sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(sbase), "n"(IMM)
                 : "memory", "m0");
}

// One workgroup per macro tile.  The k loop walks stages of 32 k (a list entry
// is B/32 stages); stage t lives in LDS buffer t % NBUF.  Ring protocol, with
// "sync(t)" = every wave waits for its own loads of stage t+1, then a
// workgroup barrier: after sync(t) stage t+1 is readable by all waves and no
// wave reads stage t any more, so the loads of stage t+NBUF go into stage t's
// buffer.  NBUF-1 stages are in flight while one is multiplied.
// PERSIST: the same macro tiles by workgroups that stay -- one per CU -- and take the next item of
// their XCD's sequence from a ticket counter (what the hardware dispatcher does with one workgroup
// per item, without ending and starting workgroups): the ticket after the current one is asked for
// before the current item's first load, so that it has arrived when the k loops end; the next
// item's scalar loads and prologue then run while the stores of C drain.  Nobody waits for another
// workgroup: a ticket beyond the sequence ends the workgroup.  Every workgroup draws exactly one
// ticket beyond the sequence, so the largest ticket (items + workgroups of the XCD - 1) is drawn
// last, and its holder puts the counter back to zero for the next launch.  The ticket is a
// returning atomic issued BEFORE the item's first global->LDS load: it is the oldest outstanding
// vector-memory operation, so the hand-counted vmcnt waits below stay exact.
template <int B, int NBUF, bool PERSIST = false>
__global__ __launch_bounds__(256) void k_gemm(const unsigned char *__restrict__ pA,
                                              const unsigned char *__restrict__ pB,
                                              const MacroEntry *__restrict__ macro_list,
                                              const int32_t *__restrict__ macro_count,
                                              const int32_t *__restrict__ order,
                                              const int32_t *__restrict__ sched, int32_t *__restrict__ ticket, int P,
                                              int n_xcd, int nbM, int nbK, int nbN, int nMacN, int64_t M, int64_t N,
                                              float *__restrict__ C) {
    using G = GemmCfg<B>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef const __attribute__((address_space(4))) u32x4 *entry_ptr;   // scalar (SMEM) loads

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    // Workgroup b runs on XCD b % n_xcd and is that XCD's q-th workgroup,
    // q = b / n_xcd; `order` holds each XCD's sequence: computing macro tiles
    // first, then the ones with nothing kept.  The latter's workgroups only
    // write zeros; they are dispatched when CUs start to fall idle at the end
    // of the XCD's queue, so the zero-fill fills the tail of the kernel
    // instead of competing with the k loops for memory bandwidth.
    const int xcd = blockIdx.x % n_xcd;
    const int ntot = __builtin_amdgcn_readfirstlane(sched[MAX_XCD + xcd]);
    const int32_t *seq = order + (int64_t)xcd * P;
    const uint32_t lds_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    // persistent form: wave 0 draws the tickets and hands them to the other waves through two LDS
    // words behind the ring, used in turn (a wave may still be reading one while the next is written)
    int32_t *tk_word = reinterpret_cast<int32_t *>(smem + NBUF * G::STAGE_BYTES);
    int tk_par = 0;
    auto request = [&]() -> int {
        int v;      // (only lane 0 of wave 0 ever looks at it; left unset elsewhere on purpose)
        asm volatile("" : "=v"(v));
        if (wave == 0 && lane == 0)
            v = __hip_atomic_fetch_add(ticket + xcd, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return v;
    };
    auto publish = [&](int v) -> int {      // (the barrier also says: every wave has left the ring)
        if (wave == 0 && lane == 0) tk_word[tk_par] = v;
        __syncthreads();
        const int r = __builtin_amdgcn_readfirstlane(tk_word[tk_par]);
        tk_par ^= 1;
        return r;
    };
    auto zero_fill = [&](int mz) {
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
        int ln = lane;
        // (workgroups that stay: keeps the lane's part of the address from being computed once for
        // all items and held in registers through the k loops, where there are none to spare)
        if constexpr (PERSIST) asm volatile("" : "+v"(ln));
        const int64_t r0 = (int64_t)(mz / nMacN) * 256, c0 = (int64_t)(mz % nMacN) * 256 + ln * 4;
        if (c0 < N)
            for (int r = wave; r < 256 && r0 + r < M; r += 4)
                __builtin_nontemporal_store(zero, reinterpret_cast<f32x4 *>(C + (r0 + r) * N + c0));
    };
    // (workgroups that stay) the holder of the largest ticket puts the counter back
    auto last_ticket = [&](int qq) {
        if (qq == ntot + (int)(gridDim.x / n_xcd) - 1 && threadIdx.x == 0) ticket[xcd] = 0;
    };
    int q, tk_next = 0;
    if constexpr (PERSIST) q = publish(request());
    else q = blockIdx.x / n_xcd;

  // Workgroups that stay run this loop over the computing items of their XCD's sequence, then the
  // loop at the end of the kernel over the items with nothing kept (the sequence lists them last).
  for (;;) {
    if (q >= ntot) {
        if constexpr (PERSIST) last_ticket(q);
        return;
    }
    const int macro = __builtin_amdgcn_readfirstlane(seq[q]);
    const int mi = macro / nMacN, mj = macro % nMacN;
    const int U = __builtin_amdgcn_readfirstlane(macro_count[2 * macro]);
    const int Ufull = __builtin_amdgcn_readfirstlane(macro_count[2 * macro + 1]);
    entry_ptr ents = (entry_ptr)(uintptr_t)(macro_list + (int64_t)macro * nbK);
    const int S = U * G::NSPE, Sfull = Ufull * G::NSPE;
    if (S == 0) {             // q >= nc: nothing kept in this macro tile
        if constexpr (PERSIST) break;
        zero_fill(macro);
        return;
    }
    if constexpr (PERSIST) tk_next = request();

    f32x16 acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[r][c][i] = 0.0f;

    {
        // ---- staging: each wave copies CHW consecutive 1 KiB chunks of the A
        // part and of the B part of a stage, in groups of GS chunks that share
        // a tile.  Tiles beyond the matrix edge are clamped to the last tile
        // row / column (loaded but never multiplied) and stages beyond the
        // last are clamped to the last (loaded but never read), so staging is
        // branch-free and the number of loads in flight is always the same.
        static_assert(G::LPW == 8, "the issue schedule below assumes 8 loads per wave per stage");
        const unsigned char *rowA[G::NG], *rowB[G::NG];
        uint32_t ldsA[G::NG];
        int slot_of[G::NG];
#pragma unroll
        for (int g = 0; g < G::NG; g++) {
            const int chunk0 = wave * G::CHW + g * G::GS;
            const int slot = chunk0 / G::CPS, within0 = chunk0 % G::CPS;
            int ti = mi * G::MT + slot, tj = mj * G::MT + slot;
            ti = ti < nbM ? ti : nbM - 1;
            tj = tj < nbN ? tj : nbN - 1;
            rowA[g] = pA + (int64_t)ti * nbK * G::TILE_BYTES + within0 * 1024;
            rowB[g] = pB + (int64_t)tj * nbK * G::TILE_BYTES + within0 * 1024;
            ldsA[g] = lds_base + slot * G::SLOT_BYTES + within0 * 1024;
            slot_of[g] = slot;
        }
        const uint32_t voff = lane * 16;

        auto stage_k = [&](int t) -> uint32_t {
            const int tc = t < S ? t : S - 1;
            return ents[tc / G::NSPE].x;
        };
        // k and the needed-rows/columns bits of a stage's entry (one 8-byte scalar load)
        typedef const __attribute__((address_space(4))) uint64_t *entry_kn_ptr;
        auto stage_kn = [&](int t) -> uint64_t {
            const int tc = t < S ? t : S - 1;
            return *(entry_kn_ptr)(uintptr_t)(macro_list + (int64_t)macro * nbK + tc / G::NSPE);
        };
        // Load i (0..LPW-1) of a stage: i < CHW are the wave's A chunks, the
        // rest its B chunks.  A wave is in-order and alone on its SIMD, so a
        // burst of loads that backs up the address FIFO stalls its MFMAs; the
        // loops below therefore issue one load every few MFMAs.
        struct StageAddr {
            int64_t koff;
            uint32_t boff;
        };
        auto stage_addr = [&](int t, uint32_t k) -> StageAddr {
            const int tc = t < S ? t : S - 1;
            StageAddr sa;
            sa.koff = (int64_t)k * G::TILE_BYTES + (tc % G::NSPE) * G::SLOT_BYTES;
            sa.boff = (uint32_t)(t % NBUF) * G::STAGE_BYTES;
            return sa;
        };
        auto issue_one = [&](const StageAddr &sa, auto idx) {
            constexpr int i = decltype(idx)::value;
            constexpr int op = i / G::CHW, ci = i % G::CHW;
            constexpr int g = ci / G::GS, j = ci % G::GS;
            if constexpr (op == 0)
                dma_load<j * 1024>(rowA[g] + sa.koff, voff, ldsA[g] + sa.boff);
            else
                dma_load<j * 1024>(rowB[g] + sa.koff, voff, ldsA[g] + G::A_BYTES + sa.boff);
        };
#define SPAMM_ISSUE(sa, i) issue_one(sa, std::integral_constant<int, i>{})
        // Same load, but when no tile of the macro tile needs this operand slot at this k
        // (need bit clear: the slot is never multiplied) the source is the first chunk of the
        // operand array instead -- always valid and cache resident -- so that the number of
        // loads in flight stays fixed while nothing is fetched for the slot.
        auto issue_needed = [&](const StageAddr &sa, uint32_t need, auto idx) {
            constexpr int i = decltype(idx)::value;
            constexpr int op = i / G::CHW, ci = i % G::CHW;
            constexpr int g = ci / G::GS, j = ci % G::GS;
            if constexpr (op == 0) {
                const unsigned char *src = ((need >> slot_of[g]) & 1u) ? rowA[g] + sa.koff : pA;
                dma_load<j * 1024>(src, voff, ldsA[g] + sa.boff);
            } else {
                const unsigned char *src = ((need >> (8 + slot_of[g])) & 1u) ? rowB[g] + sa.koff : pB;
                dma_load<j * 1024>(src, voff, ldsA[g] + G::A_BYTES + sa.boff);
            }
        };
#define SPAMM_ISSUE_N(sa, nd, i) issue_needed(sa, nd, std::integral_constant<int, i>{})
        auto issue_all = [&](const StageAddr &sa) {
            SPAMM_ISSUE(sa, 0); SPAMM_ISSUE(sa, 1); SPAMM_ISSUE(sa, 2); SPAMM_ISSUE(sa, 3);
            SPAMM_ISSUE(sa, 4); SPAMM_ISSUE(sa, 5); SPAMM_ISSUE(sa, 6); SPAMM_ISSUE(sa, 7);
        };
        auto issue_head = [&](const StageAddr &sa) { SPAMM_ISSUE(sa, 0); SPAMM_ISSUE(sa, 1); };
        // every wave: own loads of the next stage landed and own LDS reads
        // done; then the barrier makes both true for the whole workgroup.
        // INVARIANT behind the hand-counted vmcnt: between the prologue and
        // the end of loop 2 the only vector-memory operations a wave issues
        // are the LPW dma_loads per stage, in stage order (entries and k come
        // through scalar loads, operands through LDS reads, C is stored after
        // the loops).  vmcnt counts completions in issue order, so "at most
        // LPW * (NBUF - 2) outstanding" means every load of the next stage
        // has landed.  Any other global load or store added inside the loops
        // breaks this count: re-derive it (tests/test_isa_contracts.py checks
        // the compiled assembly of every instantiation for it).
        auto sync_next = [&]() {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(G::LPW * (NBUF - 2), 0));
            __syncthreads();
        };

        // LDS byte offset (inside the A or B part of a stage) of this lane's
        // operand vector for MFMA block `blk` (32 of the wave's 128
        // rows/columns: block blk lies in the wave's (blk * 32 / B)-th tile
        // row/column) at k step kk (0 or 1) of the stage.
        auto frag_off = [&](int wsel, int blk, int kk) -> int {
            const int slot = wsel + 2 * ((blk * 32) / B);      // the wave's tile rows / columns: wsel, wsel + 2, ...
            const int ro = (blk * 32) % B;
            return slot * G::SLOT_BYTES + (((2 * kk + (lane >> 5)) * B) + ro + (lane & 31)) * 16;
        };
        auto load_frags = [&](half8 (&af)[4], half8 (&bf)[4], int t, int kk) {
            const unsigned char *bufA = smem + (t % NBUF) * G::STAGE_BYTES;
            const unsigned char *bufB = bufA + G::A_BYTES;
#pragma unroll
            for (int r = 0; r < 4; r++) af[r] = *reinterpret_cast<const half8 *>(bufA + frag_off(wr, r, kk));
#pragma unroll
            for (int c = 0; c < 4; c++) bf[c] = *reinterpret_cast<const half8 *>(bufB + frag_off(wc, c, kk));
        };

        // ---- prologue: stages 0..NBUF-2 and the first two loads of stage
        // NBUF-1 (the "head"; its "tail" of six follows inside the loops, and
        // so on for every later stage); wait for stage 0
#pragma unroll
        for (int t = 0; t < NBUF - 1; t++) issue_all(stage_addr(t, stage_k(t)));
        StageAddr sa_tail = stage_addr(NBUF - 1, stage_k(NBUF - 1));
        issue_head(sa_tail);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(G::LPW * (NBUF - 2) + 2, 0));
        __syncthreads();
        int t = 0;
        // ---- loop 1: entries kept by all tiles of the macro tile; no
        // branches.  Operand vectors are double buffered in registers (a0/b0:
        // k step 0, a1/b1: k step 1) and every LDS read is issued 8+ MFMAs
        // before its first use.  The sync sits in the middle of k step 1 so
        // that the first LDS reads of the next stage overlap its second half.
        // Global->LDS loads are spread out: one after every fourth MFMA.
        // sched_barrier(0) pins the issue order written here.
#define SPAMM_MFMA(A, Bv, r, c) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[r], Bv[c], acc[r][c], 0, 0, 0)
#define SPAMM_FENCE() __builtin_amdgcn_sched_barrier(0)
#define SPAMM_LDA(dst, blk, kk) dst = *reinterpret_cast<const half8 *>(bufA + frag_off(wr, blk, kk))
#define SPAMM_LDB(dst, blk, kk) dst = *reinterpret_cast<const half8 *>(bufB + frag_off(wc, blk, kk))
        half8 a0[4], b0[4], a1[4], b1[4];
        load_frags(a0, b0, 0, 0);
        if (Sfull > 0) {
            uint32_t knext = stage_k(NBUF);
            for (; t < Sfull; t++) {
                // address of the stage issued after this iteration's sync, computed early so that
                // only the scalar load of the next k sits between the barrier and the MFMAs
                const StageAddr sa_new = stage_addr(t + NBUF, knext);
                SPAMM_FENCE();
                {
                    const unsigned char *bufA = smem + (t % NBUF) * G::STAGE_BYTES;
                    const unsigned char *bufB = bufA + G::A_BYTES;
                    // k step 0 (16 MFMA) with the 8 reads of k step 1 in between
                    SPAMM_MFMA(a0, b0, 0, 0); SPAMM_MFMA(a0, b0, 0, 1); SPAMM_LDA(a1[0], 0, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 0, 2); SPAMM_MFMA(a0, b0, 0, 3); SPAMM_LDB(b1[0], 0, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 2); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 1, 0); SPAMM_MFMA(a0, b0, 1, 1); SPAMM_LDB(b1[1], 1, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 1, 2); SPAMM_MFMA(a0, b0, 1, 3); SPAMM_LDB(b1[2], 2, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 3); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 2, 0); SPAMM_MFMA(a0, b0, 2, 1); SPAMM_LDB(b1[3], 3, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 2, 2); SPAMM_MFMA(a0, b0, 2, 3); SPAMM_LDA(a1[1], 1, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 4); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 3, 0); SPAMM_MFMA(a0, b0, 3, 1); SPAMM_LDA(a1[2], 2, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 3, 2); SPAMM_MFMA(a0, b0, 3, 3); SPAMM_LDA(a1[3], 3, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 5); SPAMM_FENCE();
                    // first half of k step 1
                    SPAMM_MFMA(a1, b1, 0, 0); SPAMM_MFMA(a1, b1, 0, 1); SPAMM_MFMA(a1, b1, 0, 2); SPAMM_MFMA(a1, b1, 0, 3);
                    SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 6); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 1, 0); SPAMM_MFMA(a1, b1, 1, 1); SPAMM_MFMA(a1, b1, 1, 2); SPAMM_MFMA(a1, b1, 1, 3);
                    SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 7); SPAMM_FENCE();
                }
                sync_next();
                SPAMM_FENCE();
                // scalar load placed here so that no LDS wait follows it closely
                knext = stage_k(t + 1 + NBUF);
                sa_tail = sa_new;
                SPAMM_FENCE();
                {
                    const unsigned char *bufA = smem + ((t + 1) % NBUF) * G::STAGE_BYTES;
                    const unsigned char *bufB = bufA + G::A_BYTES;
                    // second half of k step 1 with the 8 reads of the next stage's k step 0
                    SPAMM_MFMA(a1, b1, 2, 0); SPAMM_LDA(a0[0], 0, 0); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 2, 1); SPAMM_LDB(b0[0], 0, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 2, 2); SPAMM_LDB(b0[1], 1, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 2, 3); SPAMM_LDB(b0[2], 2, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 3, 0); SPAMM_LDB(b0[3], 3, 0); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 3, 1); SPAMM_LDA(a0[1], 1, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 3, 2); SPAMM_LDA(a0[2], 2, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 3, 3); SPAMM_LDA(a0[3], 3, 0); SPAMM_FENCE();
                }
            }
        }
        // ---- loop 2: entries kept by some tiles only; a wave multiplies
        // exactly the (tile row, tile column) pairs whose bit is set.  Same
        // register double buffering as loop 1: on entry a0/b0 hold k step 0
        // of stage t; k step 1 is read while step 0 multiplies, and the next
        // stage's step 0 (readable after the sync) while step 1 multiplies.
        auto mul_kept = [&](const half8 (&af)[4], const half8 (&bf)[4], uint32_t sb) {
#pragma unroll
            for (int a = 0; a < G::SUB; a++)
#pragma unroll
                for (int b = 0; b < G::SUB; b++) {
                    if ((sb >> (a * G::SUB + b)) & 1u) {
#pragma unroll
                        for (int r = 0; r < G::RB; r++)
#pragma unroll
                            for (int c = 0; c < G::RB; c++)
                                acc[a * G::RB + r][b * G::RB + c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                                    af[a * G::RB + r], bf[b * G::RB + c], acc[a * G::RB + r][b * G::RB + c], 0, 0, 0);
                    }
                }
        };
        uint32_t need_tail = 0xffffu;     // the stage whose head was issued by loop 1 / the prologue: all slots
        for (; t < S; t++) {
            const uint64_t kn = stage_kn(t + NBUF);
            SPAMM_ISSUE_N(sa_tail, need_tail, 2); SPAMM_ISSUE_N(sa_tail, need_tail, 3); SPAMM_ISSUE_N(sa_tail, need_tail, 4);
            SPAMM_ISSUE_N(sa_tail, need_tail, 5); SPAMM_ISSUE_N(sa_tail, need_tail, 6); SPAMM_ISSUE_N(sa_tail, need_tail, 7);
            const u32x4 cur = ents[t / G::NSPE];
            const uint64_t mask = ((uint64_t)cur.w << 32) | cur.z;
            uint32_t sb = 0;
#pragma unroll
            for (int a = 0; a < G::SUB; a++)
#pragma unroll
                for (int b = 0; b < G::SUB; b++) {
                    const int bit = (wr + 2 * a) * G::MT + wc + 2 * b;
                    sb |= (uint32_t)((mask >> bit) & 1ull) << (a * G::SUB + b);
                }
            load_frags(a1, b1, t, 1);
            mul_kept(a0, b0, sb);
            sync_next();
            sa_tail = stage_addr(t + NBUF, (uint32_t)kn);
            // stages past the end repeat the last entry and are never read: nothing to fetch
            need_tail = t + NBUF < S ? (uint32_t)(kn >> 32) : 0u;
            SPAMM_ISSUE_N(sa_tail, need_tail, 0); SPAMM_ISSUE_N(sa_tail, need_tail, 1);
            load_frags(a0, b0, t + 1, 0);
            mul_kept(a1, b1, sb);
        }
#undef SPAMM_MFMA
#undef SPAMM_FENCE
#undef SPAMM_LDA
#undef SPAMM_LDB
#undef SPAMM_ISSUE
#undef SPAMM_ISSUE_N
        // the ring still holds clamped loads: let them land before the
        // workgroup gives its LDS back
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    }
    int q_next = 0;
    if constexpr (PERSIST) q_next = publish(tk_next);

    // ---- epilogue: C[row, col], row-major, ld N (cuSpAMM.cu:391).  MFMA
    // 32x32 result register i of lane l is row 8*(i/4) + 4*(l/32) + i%4,
    // column l%32 of the block: every store instruction writes two full
    // 128-byte row segments.  C is written once and not read again here:
    // non-temporal stores leave the L2 to the operand panels.  (Swapping the
    // MFMA operands would give float4 stores, but each then touches 32 rows
    // with 32 bytes -- measured slower.)
    int lane_e = lane;
    if constexpr (PERSIST) asm volatile("" : "+v"(lane_e));     // (as in zero_fill)
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t row0 = (int64_t)mi * 256 + (wr + 2 * (r / G::RB)) * B + (r % G::RB) * 32;
        if (row0 >= M) continue;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int64_t col0 = (int64_t)mj * 256 + (wc + 2 * (c / G::RB)) * B + (c % G::RB) * 32;
            if (col0 >= N) continue;
            float *out = C + (row0 + 4 * (lane_e >> 5)) * N + col0 + (lane_e & 31);
#pragma unroll
            for (int i = 0; i < 16; i++)
                __builtin_nontemporal_store(acc[r][c][i], &out[(int64_t)(8 * (i / 4) + (i % 4)) * N]);
        }
    }
    if constexpr (!PERSIST) return;
    q = q_next;
  }
  // (workgroups that stay) items with nothing kept: zeros, until the sequence ends
  for (;;) {
    tk_next = request();
    zero_fill(__builtin_amdgcn_readfirstlane(seq[q]));
    q = publish(tk_next);
    if (q >= ntot) {
        last_ticket(q);
        return;
    }
  }
}


// ---------------------------------------------------------------------------
// k_gemm_w64: the same multiply by waves of 64 x 128 (2 x 4 MFMA blocks = 128 accumulator
// registers, two waves per SIMD), NWR wave rows x 2 wave columns per workgroup:
//   NWR = 2  a workgroup per HALF macro tile (128 x 256 of C), two workgroups per CU: one's
//            prologue, epilogue, barriers and LDS reads sit under the other's MFMAs and the work
//            units are half as long (finer tail); the price is the B part of a stage staged once
//            per half, 24 KiB per 2.1 Mflop instead of 32 KiB per 4.2 Mflop.  Workgroups 2 q and
//            2 q + 1 of an XCD's sequence take the upper and lower half of its q-th macro tile.
//   NWR = 4  a whole macro tile by eight waves: k_gemm's 32 KiB per stage, two waves per SIMD.
// Lists, masks and the order of accumulation are the macro tile's, so C is bit-identical to
// k_gemm's.  Measured against k_gemm: halves lose 7-12 % where there is much work per CU and win
// where there is at most one macro tile per CU (chosen there); eight waves are within 1-3 %.
constexpr int HALF_RING = 3;      // stages of the half shape's ring: 3 x 24 KiB, two workgroups per CU
constexpr int W8_RING = 4;        // stages of the eight-wave shape's ring: 4 x 32 KiB, one workgroup per CU
constexpr int PERSIST_RING = 4;   // stages of the persistent form's ring (k_gemm's default)
constexpr int PERSIST_EXTRA_LDS = 16;   // the two ticket words behind the ring

template <int B, int NWR>
struct W64Cfg {
    using G = GemmCfg<B>;
    static constexpr int NW = 2 * NWR;                       // waves per workgroup
    static constexpr int MR = 64 * NWR, WR = 64, NRB = 2;
    static constexpr int MTA = MR / B > 0 ? MR / B : 1;      // A slots (tile rows) of a workgroup
    static constexpr int PARTS = 256 / MR;                   // workgroups per macro tile
    static constexpr int A_BYTES = MR * G::KS * 2;           // 8 or 16 KiB
    static constexpr int B_BYTES = 256 * G::KS * 2;          // 16 KiB
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;    // 24 or 32 KiB
    static constexpr int CHWA = A_BYTES / 1024 / NW;         // 1 KiB chunks per wave per stage: A part (2),
    static constexpr int CHWB = B_BYTES / 1024 / NW;         // B part (4 or 2)
    static constexpr int GSB = G::CPS < CHWB ? G::CPS : CHWB;   // B chunks per load group (share a tile)
    static constexpr int NGB = CHWB / GSB;
    static constexpr int LPW = CHWA + CHWB;                  // loads per wave per stage (6 or 4)
    static constexpr int TRW = WR / B > 0 ? WR / B : 1;      // tile rows a wave touches
    static constexpr int RBR = NRB / TRW;                    // MFMA row blocks per tile row of a wave
    static_assert(G::CPS >= CHWA && CHWA == 2, "a wave's two A chunks lie in one slot");
};

template <int B, int NBUF, int NWR>
__global__ __launch_bounds__(128 * NWR, NWR == 2 ? 2 : 1) void k_gemm_w64(const unsigned char *__restrict__ pA,
                                                      const unsigned char *__restrict__ pB,
                                                      const MacroEntry *__restrict__ macro_list,
                                                      const int32_t *__restrict__ macro_count,
                                                      const int32_t *__restrict__ order,
                                                      const int32_t *__restrict__ sched, int P, int n_xcd, int nbM,
                                                      int nbK, int nbN, int nMacN, int64_t M, int64_t N,
                                                      float *__restrict__ C) {
    using G = GemmCfg<B>;
    using H = W64Cfg<B, NWR>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef const __attribute__((address_space(4))) u32x4 *entry_ptr;   // scalar (SMEM) loads

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    const int xcd = blockIdx.x % n_xcd, q2 = blockIdx.x / n_xcd;
    const int q = q2 / H::PARTS, hf = q2 % H::PARTS;
    const int ntot = __builtin_amdgcn_readfirstlane(sched[MAX_XCD + xcd]);
    if (q >= ntot) return;
    const int32_t *seq = order + (int64_t)xcd * P;
    const int macro = __builtin_amdgcn_readfirstlane(seq[q]);
    const int mi = macro / nMacN, mj = macro % nMacN;
    const int64_t row_half = (int64_t)mi * 256 + hf * H::MR;            // first row of C of this workgroup
    if (row_half >= M) return;                                          // the lower half lies beyond the matrix
    const int U = __builtin_amdgcn_readfirstlane(macro_count[2 * macro]);
    const int Ufull = __builtin_amdgcn_readfirstlane(macro_count[2 * macro + 1]);
    entry_ptr ents = (entry_ptr)(uintptr_t)(macro_list + (int64_t)macro * nbK);
    const int S = U * G::NSPE, Sfull = Ufull * G::NSPE;
    const uint32_t lds_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    if (S == 0) {     // nothing kept in this macro tile: this half's zeros
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
        const int64_t c0 = (int64_t)mj * 256 + lane * 4;
        if (c0 < N)
            for (int r = wave; r < H::MR && row_half + r < M; r += H::NW)
                __builtin_nontemporal_store(zero, reinterpret_cast<f32x4 *>(C + (row_half + r) * N + c0));
        return;
    }

    f32x16 acc[H::NRB][4];
#pragma unroll
    for (int r = 0; r < H::NRB; r++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[r][c][i] = 0.0f;

    {
        // ---- staging: a wave copies 2 consecutive 1 KiB chunks of the A part (one slot) and 4 of
        // the B part (NGB groups of GSB chunks, each group inside one slot).  Clamping as in k_gemm.
        const int chunkA0 = wave * H::CHWA;
        const int slotA = chunkA0 / G::CPS, withinA = chunkA0 % G::CPS;
        int tiA = mi * G::MT + hf * H::MTA + slotA;
        tiA = tiA < nbM ? tiA : nbM - 1;
        const unsigned char *rowA = pA + (int64_t)tiA * nbK * G::TILE_BYTES + withinA * 1024;
        const uint32_t ldsA = lds_base + slotA * G::SLOT_BYTES + withinA * 1024;
        const unsigned char *rowB[H::NGB];
        uint32_t ldsB[H::NGB];
        int slotB[H::NGB];
#pragma unroll
        for (int g = 0; g < H::NGB; g++) {
            const int chunk0 = wave * H::CHWB + g * H::GSB;
            const int slot = chunk0 / G::CPS, within0 = chunk0 % G::CPS;
            int tj = mj * G::MT + slot;
            tj = tj < nbN ? tj : nbN - 1;
            rowB[g] = pB + (int64_t)tj * nbK * G::TILE_BYTES + within0 * 1024;
            ldsB[g] = lds_base + H::A_BYTES + slot * G::SLOT_BYTES + within0 * 1024;
            slotB[g] = slot;
        }
        const uint32_t voff = lane * 16;

        auto stage_k = [&](int t) -> uint32_t {
            const int tc = t < S ? t : S - 1;
            return ents[tc / G::NSPE].x;
        };
        struct StageAddr {
            int64_t koff;
            uint32_t boff;
        };
        auto stage_addr = [&](int t, uint32_t k) -> StageAddr {
            const int tc = t < S ? t : S - 1;
            StageAddr sa;
            sa.koff = (int64_t)k * G::TILE_BYTES + (tc % G::NSPE) * G::SLOT_BYTES;
            sa.boff = (uint32_t)(t % NBUF) * H::STAGE_BYTES;
            return sa;
        };
        // load i of a stage: 0, 1 = the wave's A chunks, 2..5 = its B chunks
        auto issue_one = [&](const StageAddr &sa, auto idx) {
            constexpr int i = decltype(idx)::value;
            if constexpr (i < H::CHWA) {
                dma_load<i * 1024>(rowA + sa.koff, voff, ldsA + sa.boff);
            } else {
                constexpr int g = (i - H::CHWA) / H::GSB, j = (i - H::CHWA) % H::GSB;
                dma_load<j * 1024>(rowB[g] + sa.koff, voff, ldsB[g] + sa.boff);
            }
        };
        // same, but a slot no kept product of this half needs is not fetched (cache-resident placeholder)
        auto issue_needed = [&](const StageAddr &sa, uint32_t needA, uint32_t needB, auto idx) {
            constexpr int i = decltype(idx)::value;
            // (the choice is scalar arithmetic on purpose: the address must stay in scalar registers)
            if constexpr (i < H::CHWA) {
                const int64_t on = -(int64_t)((needA >> slotA) & 1u);
                dma_load<i * 1024>(pA + (((rowA - pA) + sa.koff) & on), voff, ldsA + sa.boff);
            } else {
                constexpr int g = (i - H::CHWA) / H::GSB, j = (i - H::CHWA) % H::GSB;
                const int64_t on = -(int64_t)((needB >> slotB[g]) & 1u);
                dma_load<j * 1024>(pB + (((rowB[g] - pB) + sa.koff) & on), voff, ldsB[g] + sa.boff);
            }
        };
#define SPAMM_ISSUE(sa, i) issue_one(sa, std::integral_constant<int, i>{})
#define SPAMM_ISSUE_N(sa, na, nb_, i) issue_needed(sa, na, nb_, std::integral_constant<int, i>{})
        // (loads 4 and 5 exist in the half shape only)
#define SPAMM_ISSUE_X(sa, i) do { if constexpr (i < H::LPW) issue_one(sa, std::integral_constant<int, (i < H::LPW ? i : 0)>{}); } while (0)
#define SPAMM_ISSUE_NX(sa, na, nb_, i) do { if constexpr (i < H::LPW) issue_needed(sa, na, nb_, std::integral_constant<int, (i < H::LPW ? i : 0)>{}); } while (0)
        auto issue_all = [&](const StageAddr &sa) {
            SPAMM_ISSUE(sa, 0); SPAMM_ISSUE(sa, 1); SPAMM_ISSUE(sa, 2);
            SPAMM_ISSUE(sa, 3); SPAMM_ISSUE_X(sa, 4); SPAMM_ISSUE_X(sa, 5);
        };
        // the ring protocol and its vmcnt invariant are k_gemm's, with LPW = 6 loads per wave per stage
        auto sync_next = [&]() {
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(H::LPW * (NBUF - 2), 0));
            __syncthreads();
        };
        auto frag_off = [&](int first, int blk, int kk) -> int {     // `first`: the wave's first row / column
            const int off = first + blk * 32;
            return (off / B) * G::SLOT_BYTES + (((2 * kk + (lane >> 5)) * B) + off % B + (lane & 31)) * 16;
        };
        auto load_frags = [&](half8 (&af)[H::NRB], half8 (&bf)[4], int t, int kk) {
            const unsigned char *bufA = smem + (t % NBUF) * H::STAGE_BYTES;
            const unsigned char *bufB = bufA + H::A_BYTES;
#pragma unroll
            for (int r = 0; r < H::NRB; r++) af[r] = *reinterpret_cast<const half8 *>(bufA + frag_off(wr * H::WR, r, kk));
#pragma unroll
            for (int c = 0; c < 4; c++) bf[c] = *reinterpret_cast<const half8 *>(bufB + frag_off(wc * 128, c, kk));
        };

        // ---- prologue: stages 0..NBUF-2 and the first two loads of stage NBUF-1
#pragma unroll
        for (int t = 0; t < NBUF - 1; t++) issue_all(stage_addr(t, stage_k(t)));
        StageAddr sa_tail = stage_addr(NBUF - 1, stage_k(NBUF - 1));
        SPAMM_ISSUE(sa_tail, 0); SPAMM_ISSUE(sa_tail, 1);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(H::LPW * (NBUF - 2) + 2, 0));
        __syncthreads();
        int t = 0;
#define SPAMM_MFMA(A, Bv, r, c) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[r], Bv[c], acc[r][c], 0, 0, 0)
#define SPAMM_FENCE() __builtin_amdgcn_sched_barrier(0)
#define SPAMM_LDA(dst, blk, kk) dst = *reinterpret_cast<const half8 *>(bufA + frag_off(wr * H::WR, blk, kk))
#define SPAMM_LDB(dst, blk, kk) dst = *reinterpret_cast<const half8 *>(bufB + frag_off(wc * 128, blk, kk))
        half8 a0[H::NRB], b0[4], a1[H::NRB], b1[4];
        load_frags(a0, b0, 0, 0);
        // ---- loop 1: entries kept by all tiles of the macro tile, branch-free; 8 MFMAs per k step,
        // the 6 LDS reads of the next k step and the stage's 6 global->LDS loads between them
        if (Sfull > 0) {
            uint32_t knext = stage_k(NBUF);
            for (; t < Sfull; t++) {
                const StageAddr sa_new = stage_addr(t + NBUF, knext);
                SPAMM_FENCE();
                {
                    const unsigned char *bufA = smem + (t % NBUF) * H::STAGE_BYTES;
                    const unsigned char *bufB = bufA + H::A_BYTES;
                    SPAMM_MFMA(a0, b0, 0, 0); SPAMM_LDA(a1[0], 0, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 0, 1); SPAMM_LDB(b1[0], 0, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 2); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 0, 2); SPAMM_LDB(b1[1], 1, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 0, 3); SPAMM_LDB(b1[2], 2, 1); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 3); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 1, 0); SPAMM_LDB(b1[3], 3, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 1, 1); SPAMM_LDA(a1[1], 1, 1); SPAMM_FENCE();
                    SPAMM_ISSUE_X(sa_tail, 4); SPAMM_FENCE();
                    SPAMM_MFMA(a0, b0, 1, 2); SPAMM_MFMA(a0, b0, 1, 3); SPAMM_FENCE();
                    SPAMM_ISSUE_X(sa_tail, 5); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 0, 0); SPAMM_MFMA(a1, b1, 0, 1); SPAMM_MFMA(a1, b1, 0, 2); SPAMM_MFMA(a1, b1, 0, 3);
                    SPAMM_FENCE();
                }
                sync_next();
                SPAMM_FENCE();
                knext = stage_k(t + 1 + NBUF);
                sa_tail = sa_new;
                SPAMM_FENCE();
                {
                    const unsigned char *bufA = smem + ((t + 1) % NBUF) * H::STAGE_BYTES;
                    const unsigned char *bufB = bufA + H::A_BYTES;
                    SPAMM_MFMA(a1, b1, 1, 0); SPAMM_LDA(a0[0], 0, 0); SPAMM_LDB(b0[0], 0, 0); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 1, 1); SPAMM_LDB(b0[1], 1, 0); SPAMM_LDB(b0[2], 2, 0); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 1, 2); SPAMM_LDB(b0[3], 3, 0); SPAMM_FENCE();
                    SPAMM_ISSUE(sa_tail, 1); SPAMM_FENCE();
                    SPAMM_MFMA(a1, b1, 1, 3); SPAMM_LDA(a0[1], 1, 0); SPAMM_FENCE();
                }
            }
        }
        // ---- loop 2: entries kept by some tiles only; this half multiplies exactly the pairs of its
        // tile rows whose bit is set, and fetches only the slots those pairs need
        auto mul_kept = [&](const half8 (&af)[H::NRB], const half8 (&bf)[4], uint32_t sb) {
#pragma unroll
            for (int a = 0; a < H::TRW; a++)
#pragma unroll
                for (int b = 0; b < G::SUB; b++) {
                    if ((sb >> (a * G::SUB + b)) & 1u) {
#pragma unroll
                        for (int r = 0; r < H::RBR; r++)
#pragma unroll
                            for (int c = 0; c < G::RB; c++)
                                acc[a * H::RBR + r][b * G::RB + c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                                    af[a * H::RBR + r], bf[b * G::RB + c], acc[a * H::RBR + r][b * G::RB + c], 0, 0, 0);
                    }
                }
        };
        // rows / columns of the macro tile's mask that belong to this half: needA bit a = tile row
        // a of the half holds a kept product, needB bit b = tile column b does
        auto need_of = [&](const u32x4 &e, uint32_t &needA, uint32_t &needB) {
            const uint64_t m = (((uint64_t)e.w << 32) | e.z) >> (hf * H::MTA * G::MT);
            needA = 0; needB = 0;
#pragma unroll
            for (int a = 0; a < H::MTA; a++) {
                const uint32_t rowbits = (uint32_t)(m >> (a * G::MT)) & ((1u << G::MT) - 1u);
                needA |= (rowbits ? 1u : 0u) << a;
                needB |= rowbits;
            }
        };
        uint32_t needA_tail = 0xffu, needB_tail = 0xffu;     // the stage whose head is in flight: all slots
        const int trow0 = (hf * H::MR + wr * H::WR) / B;     // first tile row of the wave inside the macro tile
        for (; t < S; t++) {
            // (stages past the end repeat the last entry and are never read: their mask is cleared,
            // so nothing is fetched for them)
            const int tn = t + NBUF < S ? t + NBUF : S - 1;
            u32x4 nxt = ents[tn / G::NSPE];
            const uint32_t live = (uint32_t)((t + NBUF - S) >> 31);      // all ones while t + NBUF < S
            nxt.z &= live;
            nxt.w &= live;
            SPAMM_ISSUE_N(sa_tail, needA_tail, needB_tail, 2); SPAMM_ISSUE_N(sa_tail, needA_tail, needB_tail, 3);
            SPAMM_ISSUE_NX(sa_tail, needA_tail, needB_tail, 4); SPAMM_ISSUE_NX(sa_tail, needA_tail, needB_tail, 5);
            const u32x4 cur = ents[t / G::NSPE];
            const uint64_t mask = ((uint64_t)cur.w << 32) | cur.z;
            uint32_t sb = 0;
#pragma unroll
            for (int a = 0; a < H::TRW; a++)
#pragma unroll
                for (int b = 0; b < G::SUB; b++) {
                    const int bit = (trow0 + a) * G::MT + wc * G::SUB + b;
                    sb |= (uint32_t)((mask >> bit) & 1ull) << (a * G::SUB + b);
                }
            load_frags(a1, b1, t, 1);
            mul_kept(a0, b0, sb);
            sync_next();
            sa_tail = stage_addr(t + NBUF, nxt.x);
            need_of(nxt, needA_tail, needB_tail);
            needA_tail = __builtin_amdgcn_readfirstlane(needA_tail);
            needB_tail = __builtin_amdgcn_readfirstlane(needB_tail);
            SPAMM_ISSUE_N(sa_tail, needA_tail, needB_tail, 0); SPAMM_ISSUE_N(sa_tail, needA_tail, needB_tail, 1);
            load_frags(a0, b0, t + 1, 0);
            mul_kept(a1, b1, sb);
        }
#undef SPAMM_MFMA
#undef SPAMM_FENCE
#undef SPAMM_LDA
#undef SPAMM_LDB
#undef SPAMM_ISSUE
#undef SPAMM_ISSUE_N
#undef SPAMM_ISSUE_X
#undef SPAMM_ISSUE_NX
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
    }

    // ---- epilogue: as k_gemm's, for the half's 2 x 4 blocks per wave
#pragma unroll
    for (int r = 0; r < H::NRB; r++) {
        const int64_t row0 = row_half + wr * H::WR + r * 32;
        if (row0 >= M) continue;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int64_t col0 = (int64_t)mj * 256 + wc * 128 + c * 32;
            if (col0 >= N) continue;
            float *out = C + (row0 + 4 * (lane >> 5)) * N + col0 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 16; i++)
                __builtin_nontemporal_store(acc[r][c][i], &out[(int64_t)(8 * (i / 4) + (i % 4)) * N]);
        }
    }
}

template <int B, int NBUF>
static hipError_t set_lds_attr() {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm<B, NBUF>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, NBUF * GemmCfg<B>::STAGE_BYTES);
    if (e != hipSuccess || NBUF != HALF_RING) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm_w64<B, HALF_RING, 2>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, HALF_RING * W64Cfg<B, 2>::STAGE_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm_w64<B, W8_RING, 4>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, W8_RING * W64Cfg<B, 4>::STAGE_BYTES);
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm<B, PERSIST_RING, true>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               PERSIST_RING * GemmCfg<B>::STAGE_BYTES + PERSIST_EXTRA_LDS);
}

hipError_t gemm_init() {
    hipError_t e;
    if ((e = set_lds_attr<32, 3>()) != hipSuccess) return e;
    if ((e = set_lds_attr<32, 4>()) != hipSuccess) return e;
    if ((e = set_lds_attr<32, 5>()) != hipSuccess) return e;
    if ((e = set_lds_attr<64, 3>()) != hipSuccess) return e;
    if ((e = set_lds_attr<64, 4>()) != hipSuccess) return e;
    if ((e = set_lds_attr<64, 5>()) != hipSuccess) return e;
    if ((e = set_lds_attr<128, 3>()) != hipSuccess) return e;
    if ((e = set_lds_attr<128, 4>()) != hipSuccess) return e;
    if ((e = set_lds_attr<128, 5>()) != hipSuccess) return e;
    return hipSuccess;
}

template <int B, int NBUF>
static void launch_one(unsigned grid, int n_xcd, const unsigned char *pA, const unsigned char *pB, const GateBuffers &g,
                       int nbM, int nbK, int nbN, int nMacN, int64_t M, int64_t N, float *C, hipStream_t s) {
    k_gemm<B, NBUF><<<grid, 256, NBUF * GemmCfg<B>::STAGE_BYTES, s>>>(pA, pB, g.macro_list, g.macro_count, g.order,
                                                                     g.sched, nullptr, (int)(grid / n_xcd), n_xcd, nbM,
                                                                     nbK, nbN, nMacN, M, N, C);
}

template <int B>
static void launch_tile(int nbuf, int shape, unsigned grid, int n_xcd, int n_cu, const unsigned char *pA,
                        const unsigned char *pB, const GateBuffers &g, int nbM, int nbK, int nbN, int nMacN, int64_t M,
                        int64_t N, float *C, hipStream_t s) {
    if (shape == GEMM_SHAPE_PERSIST) {
        // one workgroup per CU (the ring leaves room for one), an equal number on every XCD; they draw
        // the items of their XCD's sequence from g.sched's ticket words (zero before every launch)
        unsigned stay = (unsigned)(n_cu / n_xcd) * (unsigned)n_xcd;
        if (stay == 0) stay = (unsigned)n_xcd;
        if (stay > grid) stay = grid;
        k_gemm<B, PERSIST_RING, true><<<stay, 256, PERSIST_RING * GemmCfg<B>::STAGE_BYTES + PERSIST_EXTRA_LDS, s>>>(
            pA, pB, g.macro_list, g.macro_count, g.order, g.sched, g.sched + 2 * MAX_XCD, (int)(grid / n_xcd), n_xcd, nbM,
            nbK, nbN, nMacN, M, N, C);
        return;
    }
    if (shape == GEMM_SHAPE_HALF) {
        // two workgroups per macro tile; the ring is HALF_RING stages of 24 KiB so that two workgroups fit a CU
        k_gemm_w64<B, HALF_RING, 2><<<2 * grid, 256, HALF_RING * W64Cfg<B, 2>::STAGE_BYTES, s>>>(
            pA, pB, g.macro_list, g.macro_count, g.order, g.sched, (int)(grid / n_xcd), n_xcd, nbM, nbK, nbN, nMacN, M, N, C);
        return;
    }
    if (shape == GEMM_SHAPE_W8) {
        // a whole macro tile by eight waves of 64 x 128: two waves per SIMD
        k_gemm_w64<B, W8_RING, 4><<<grid, 512, W8_RING * W64Cfg<B, 4>::STAGE_BYTES, s>>>(
            pA, pB, g.macro_list, g.macro_count, g.order, g.sched, (int)(grid / n_xcd), n_xcd, nbM, nbK, nbN, nMacN, M, N, C);
        return;
    }
    if (nbuf == 3) launch_one<B, 3>(grid, n_xcd, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s);
    else if (nbuf == 5) launch_one<B, 5>(grid, n_xcd, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s);
    else launch_one<B, 4>(grid, n_xcd, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s);
}

hipError_t launch_gemm(const void *packedA, const void *packedB, const GateBuffers &g, int64_t M,
                       int64_t K, int64_t N, int tile, float *C, int n_xcd, int n_cu, int ring, int shape, hipStream_t s) {
    const int MT = macro_dim(tile);
    const int nbM = (int)(M / tile), nbK = (int)(K / tile), nbN = (int)(N / tile);
    const int nMacM = (nbM + MT - 1) / MT, nMacN = (nbN + MT - 1) / MT;
    (void)nMacM;
    const int rounds = sched_rounds(tile, nbM, nbN, n_xcd);
    const unsigned grid = (unsigned)(rounds * n_xcd * SUPER_M * SUPER_N);
    const unsigned char *pA = (const unsigned char *)packedA;
    const unsigned char *pB = (const unsigned char *)packedB;
    switch (tile) {
        case 32: launch_tile<32>(ring, shape, grid, n_xcd, n_cu, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s); break;
        case 64: launch_tile<64>(ring, shape, grid, n_xcd, n_cu, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s); break;
        case 128: launch_tile<128>(ring, shape, grid, n_xcd, n_cu, pA, pB, g, nbM, nbK, nbN, nMacN, M, N, C, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace spamm
