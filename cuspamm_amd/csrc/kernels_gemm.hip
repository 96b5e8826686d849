// Stage 3: gated tile GEMM on MFMA.
//
// Replaces the product loop of get_C_FP16_B32 (cuSpAMM.cu:336-391): for every
// output tile C_ij the sum over kept k of A_ik * B_kj, fp16 operands, fp32
// accumulation, ascending k.  The reference gives each 32x32 output tile its
// own block and re-fetches both operand tiles per product (16 flop/byte).
// Here one workgroup (4 waves, 2 x 2) owns a macro tile of 256 x 256 elements
// of C; each wave owns 128 x 128 (4 x 4 MFMA 32x32x16 accumulators = 256 fp32
// registers per lane).  The workgroup walks the macro tile's union list of k;
// per entry it stages the needed A tiles (256 rows) and B tiles (256 columns)
// of that k in LDS with direct global->LDS loads, double buffered, and every
// wave multiplies only the (tile row, tile column) pairs whose bit is set in
// the entry's mask, so the kept set is exactly the gate's.
//
// Operands come in the packed layout of spamm_internal.h: a tile's bytes are
// already in MFMA operand order, so staging is a straight copy and every
// ds_read_b128 is 512 contiguous bytes per half wave.
#include "spamm_internal.h"

namespace spamm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int B>
struct GemmCfg {
    static constexpr int SUB = 128 / B;              // tiles per wave per dimension
    static constexpr int MT = 2 * SUB;               // tiles per macro tile per dimension
    static constexpr int KS = B < 64 ? B : 64;       // k depth of one stage
    static constexpr int NSPE = B / KS;              // stages per list entry
    static constexpr int SLOT_BYTES = B * KS * 2;    // one tile's share of a stage
    static constexpr int CPS = SLOT_BYTES / 1024;    // 1 KiB wave-loads per slot
    static constexpr int A_BYTES = MT * SLOT_BYTES;  // 256 rows x KS
    static constexpr int STAGE_BYTES = 2 * A_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int TILE_BYTES = B * B * 2;
    static constexpr int RB = B / 32;                // MFMA blocks per tile per dimension
};

#define SPAMM_WAIT_VMCNT0() __builtin_amdgcn_s_waitcnt(0x0F70)

// 16 bytes per lane straight from global memory into LDS: lane l's vector
// lands at lds_addr + 16*l.  Written as inline assembly so that the compiler's
// wait-count insertion does not see an LDS write it cannot disambiguate (it
// would put a full vmcnt(0) wait before every LDS read and serialise the
// double buffering); completion is awaited explicitly with
// SPAMM_WAIT_VMCNT0() before the workgroup barrier.  M0 carries the LDS
// address; nothing else in this kernel keeps a value in M0.
__device__ __forceinline__ void dma16(const void *gsrc, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_addr), "v"(gsrc)
                 : "memory");
}

template <int B>
__global__ __launch_bounds__(256) void k_gemm(const unsigned char *__restrict__ pA,
                                              const unsigned char *__restrict__ pB,
                                              const MacroEntry *__restrict__ macro_list,
                                              const int32_t *__restrict__ macro_count,
                                              const int32_t *__restrict__ order, int nbM, int nbK,
                                              int nbN, int nMacN, int64_t M, int64_t N,
                                              float *__restrict__ C) {
    using G = GemmCfg<B>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef const __attribute__((address_space(4))) u32x4 *entry_ptr;   // scalar (SMEM) loads

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    const int macro = __builtin_amdgcn_readfirstlane(order[blockIdx.x]);
    const int mi = macro / nMacN, mj = macro % nMacN;
    const int U = __builtin_amdgcn_readfirstlane(macro_count[macro]);
    entry_ptr ents = (entry_ptr)(uintptr_t)(macro_list + (int64_t)macro * nbK);
    const int S = U * G::NSPE;
    const uint32_t lds_base =
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

    f32x16 acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[r][c][i] = 0.0f;

    // Stage s -> LDS buffer s&1.  Each wave copies CHW consecutive 1 KiB
    // chunks of the A part and of the B part.
    auto issue_loads = [&](int s, u32x4 en) {
        const int h = s % G::NSPE;
        const uint32_t k = en.x, need = en.y;
        const uint32_t buf = lds_base + (s & 1) * G::STAGE_BYTES;
        constexpr int CHW = G::MT * G::CPS / 4;
#pragma unroll
        for (int c = 0; c < CHW; c++) {
            const int chunk = wave * CHW + c;
            const int slot = chunk / G::CPS, within = chunk % G::CPS;
            if ((need >> slot) & 1u) {
                const unsigned char *src = pA + ((int64_t)(mi * G::MT + slot) * nbK + k) * G::TILE_BYTES +
                                           h * G::SLOT_BYTES + within * 1024 + lane * 16;
                dma16(src, buf + slot * G::SLOT_BYTES + within * 1024);
            }
        }
#pragma unroll
        for (int c = 0; c < CHW; c++) {
            const int chunk = wave * CHW + c;
            const int slot = chunk / G::CPS, within = chunk % G::CPS;
            if ((need >> (8 + slot)) & 1u) {
                const unsigned char *src = pB + ((int64_t)(mj * G::MT + slot) * nbK + k) * G::TILE_BYTES +
                                           h * G::SLOT_BYTES + within * 1024 + lane * 16;
                dma16(src, buf + G::A_BYTES + slot * G::SLOT_BYTES + within * 1024);
            }
        }
    };

    // LDS byte offset (inside the A or B part of a stage) of this lane's
    // operand vector for MFMA block `blk` (32 of the wave's 128 rows/columns)
    // at k step kk.
    auto frag_off = [&](int wsel, int blk, int kk) -> int {
        const int slot = wsel * G::SUB + (blk * 32) / B;
        const int ro = (blk * 32) % B;
        return slot * G::SLOT_BYTES + (((2 * kk + (lane >> 5)) * B) + ro + (lane & 31)) * 16;
    };

    u32x4 cur = {0, 0, 0, 0};
    if (S > 0) {
        cur = ents[0];
        issue_loads(0, cur);
    }
    for (int s = 0; s < S; s++) {
        u32x4 nxt = cur;
        if (s + 1 < S) nxt = ents[(s + 1) / G::NSPE];
        SPAMM_WAIT_VMCNT0();
        __syncthreads();
        if (s + 1 < S) issue_loads(s + 1, nxt);

        // bits of this wave's SUB x SUB tiles
        const uint64_t mask = ((uint64_t)cur.w << 32) | cur.z;
        uint32_t sb = 0;
#pragma unroll
        for (int a = 0; a < G::SUB; a++)
#pragma unroll
            for (int b = 0; b < G::SUB; b++) {
                const int bit = (wr * G::SUB + a) * G::MT + wc * G::SUB + b;
                sb |= (uint32_t)((mask >> bit) & 1ull) << (a * G::SUB + b);
            }

        if (sb != 0) {
            const unsigned char *bufA = smem + (s & 1) * G::STAGE_BYTES;
            const unsigned char *bufB = bufA + G::A_BYTES;
            constexpr int NKK = G::KS / 16;
            half8 af[2][4], bf[2][4];
#pragma unroll
            for (int r = 0; r < 4; r++) af[0][r] = *reinterpret_cast<const half8 *>(bufA + frag_off(wr, r, 0));
#pragma unroll
            for (int c = 0; c < 4; c++) bf[0][c] = *reinterpret_cast<const half8 *>(bufB + frag_off(wc, c, 0));
#pragma unroll
            for (int kk = 0; kk < NKK; kk++) {
                if (kk + 1 < NKK) {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        af[(kk + 1) & 1][r] = *reinterpret_cast<const half8 *>(bufA + frag_off(wr, r, kk + 1));
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        bf[(kk + 1) & 1][c] = *reinterpret_cast<const half8 *>(bufB + frag_off(wc, c, kk + 1));
                }
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
                                        af[kk & 1][a * G::RB + r], bf[kk & 1][b * G::RB + c],
                                        acc[a * G::RB + r][b * G::RB + c], 0, 0, 0);
                        }
                    }
            }
        }
        cur = nxt;
    }

    // ---- epilogue: C[row, col], row-major, ld N (cuSpAMM.cu:391).  MFMA
    // 32x32 result register i of lane l is row 8*(i/4) + 4*(l/32) + i%4,
    // column l%32 of the block.
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t row0 = (int64_t)mi * 256 + wr * 128 + r * 32;
        if (row0 >= M) continue;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int64_t col0 = (int64_t)mj * 256 + wc * 128 + c * 32;
            if (col0 >= N) continue;
            float *out = C + (row0 + 4 * (lane >> 5)) * N + col0 + (lane & 31);
#pragma unroll
            for (int i = 0; i < 16; i++) out[(int64_t)(8 * (i / 4) + (i % 4)) * N] = acc[r][c][i];
        }
    }
}

hipError_t gemm_init() {
    hipError_t e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm<32>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, GemmCfg<32>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm<64>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, GemmCfg<64>::LDS_BYTES);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_gemm<128>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, GemmCfg<128>::LDS_BYTES);
    return e;
}

hipError_t launch_gemm(const void *packedA, const void *packedB, const GateBuffers &g, int64_t M,
                       int64_t K, int64_t N, int tile, float *C, hipStream_t s) {
    const int MT = macro_dim(tile);
    const int nbM = (int)(M / tile), nbK = (int)(K / tile), nbN = (int)(N / tile);
    const int nMacM = (nbM + MT - 1) / MT, nMacN = (nbN + MT - 1) / MT;
    const unsigned grid = (unsigned)(nMacM * nMacN);
    const unsigned char *pA = (const unsigned char *)packedA;
    const unsigned char *pB = (const unsigned char *)packedB;
    switch (tile) {
        case 32:
            k_gemm<32><<<grid, 256, GemmCfg<32>::LDS_BYTES, s>>>(pA, pB, g.macro_list, g.macro_count,
                                                               g.order, nbM, nbK, nbN, nMacN, M, N, C);
            break;
        case 64:
            k_gemm<64><<<grid, 256, GemmCfg<64>::LDS_BYTES, s>>>(pA, pB, g.macro_list, g.macro_count,
                                                               g.order, nbM, nbK, nbN, nMacN, M, N, C);
            break;
        case 128:
            k_gemm<128><<<grid, 256, GemmCfg<128>::LDS_BYTES, s>>>(pA, pB, g.macro_list,
                                                                 g.macro_count, g.order, nbM, nbK, nbN, nMacN,
                                                                 M, N, C);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace spamm
