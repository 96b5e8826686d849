// Internal declarations shared by the translation units of libspamm_gfx950.so.
// Host-side launchers only; kernels live in the .hip files.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace spamm {

// ---------------------------------------------------------------------------
// Packed fp16 operand layout (private to the library).
//
// An operand is cut into b x b tiles; every tile is one contiguous block of
// b*b halves.  Inside a tile the element with free index r (row of A / column
// of B) and contraction index k (column of A / row of B) sits at
//     ((k / 8) * b + r) * 8 + (k % 8)          [units: halves]
// i.e. [k-group][r][8]: a 16-byte vector holds 8 consecutive k of one r, which
// is exactly one lane's share of an MFMA 32x32x16 operand, and 32 consecutive
// r are 512 contiguous bytes.  Tile order: A tile (I,Kt) at I*nbK + Kt,
// B tile (Kt,J) at J*nbK + Kt, so that the k tiles of one output tile are
// consecutive in memory for both operands.
// ---------------------------------------------------------------------------

// Output tiles are grouped into macro tiles of (256/b) x (256/b) tiles
// (256 x 256 elements); one workgroup of the gated GEMM owns one macro tile.
inline int macro_dim(int tile) { return 256 / tile; }

// Macro tiles are scheduled in super tiles of SUPER_M x SUPER_N macro tiles:
// 32 workgroups, one per CU of an XCD, that share operand panels in that
// XCD's L2.
constexpr int SUPER_M = 4;
constexpr int SUPER_N = 8;
constexpr int MAX_XCD = 8;      // an unpartitioned MI355X: 8 XCDs of 32 CUs

// Number of XCDs the schedule is built for: workgroup b of a grid runs on XCD b % n.  Derived
// from the CU count of the device (or partition): 32 CUs per XCD; anything that is not 1, 2, 4 or
// 8 whole XCDs gets one flat sequence (n = 1), which is correct on any device and only gives up
// the sharing of operand panels in an XCD's L2.
inline int xcds_for_cu_count(int cus) {
    for (int n = MAX_XCD; n >= 1; n >>= 1)
        if (cus == n * SUPER_M * SUPER_N) return n;
    return 1;
}

// Workgroups per XCD in the GEMM grid: whole super tiles, dealt round-robin over n_xcd XCDs.
// (Buffers are sized for n_xcd = MAX_XCD, which is an upper bound for every smaller power of two.)
inline int sched_rounds(int tile, int64_t nbM, int64_t nbN, int n_xcd = MAX_XCD) {
    const int MT = 256 / tile;
    const int nMacM = (int)((nbM + MT - 1) / MT), nMacN = (int)((nbN + MT - 1) / MT);
    const int n_super = ((nMacM + SUPER_M - 1) / SUPER_M) * ((nMacN + SUPER_N - 1) / SUPER_N);
    return (n_super + n_xcd - 1) / n_xcd;
}

// One entry of a macro tile's union k list: tile column/row k of the
// operands plus the set of output tiles (bit a*MT+b = tile row a, column b of
// the macro tile) that keep the product with this k.  16 bytes so that the
// GEMM fetches an entry with one scalar load.
struct __attribute__((aligned(16))) MacroEntry {
    uint32_t k;
    uint32_t need;      // bits 0..7: tile rows with any kept product, bits 8..15: tile columns
    uint32_t mask_lo;
    uint32_t mask_hi;
};

struct GateBuffers {
    const float *nA;        // [nbM x nbK]
    const float *nBt;       // [nbN x nbK]  (transposed B norm map)
    int32_t *counts;        // [nbM*nbN]
    uint64_t *mask;         // [nbM*nbN*words]
    MacroEntry *macro_list; // [n_macro*nbK]   union list of k per macro tile
    int32_t *macro_count;   // [n_macro][2]    entries in the union list, of which full (listed first)
    int32_t *macro_work;    // [n_macro]       kept products in the macro tile
    int32_t *order;         // [n_xcd * P]     macro tile of XCD x's q-th workgroup (P = rounds * 32), valid for q < sched[8 + x]
    int32_t *sched;         // [24]            per XCD x: [x] computing items, [8 + x] all items, [16 + x] ticket
                            //                 counter of the persistent GEMM (zero between launches)
    int64_t *kept_total;    // [1]  kept products
};

// tau_skip > 0: tau-aware pass, the fp16 copy of tile (i, k) is written only if
// fl(nA[i,k] * rowmax[k]) >= tau_skip (rowmax[k] = max_j nB[k,j], launch_rowmax)
hipError_t launch_normmap_a(const void *X, bool in16, int64_t rows, int64_t cols, int tile, void *packed,
                            float *nm, const float *rowmax, float tau_skip, hipStream_t s);
hipError_t launch_rowmax(const float *nB, int64_t nbK, int64_t nbN, float *rowmax, hipStream_t s);
// tau_skip > 0: the fp16 copy of tiles of norm zero is not written (no product with them reaches tau)
hipError_t launch_normmap_b(const void *X, bool in16, int64_t rows, int64_t cols, int tile, void *packed,
                            float *nm, float *nmT, float tau_skip, hipStream_t s);
// A = B (square): one pass over X for both operand roles
hipError_t launch_normmap_ab(const void *X, bool in16, int64_t n, int tile, void *packedA, float *nmA,
                             void *packedB, float *nmB, float *nmBt, float tau_skip, hipStream_t s);
// error report tooling (kernels_tools.hip)
hipError_t launch_error_vs_dense(const void *packedA, const void *packedB, int64_t M, int64_t K, int64_t N,
                                 int tile, const float *C, int64_t row0, int64_t row1, double *out3,
                                 hipStream_t s);
// out1 += sum over tiles of s_ij^2, s_ij = sum_{k dropped} nA[i,k]*nB[k,j]; per_tile (optional): s_ij
hipError_t launch_dropped_bound(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN,
                                float tau, double *out1, double *per_tile, hipStream_t s);
hipError_t launch_unpack(const void *packed, int64_t rows, int64_t cols, int tile, int role,
                         uint16_t *out, hipStream_t s);
hipError_t launch_transpose_normmap(const float *nB, int64_t nbK, int64_t nbN, float *nBt,
                                    hipStream_t s);
hipError_t launch_fill_decay(float *X, int64_t rows, int64_t cols, const float *table,
                             uint64_t seed, int random, hipStream_t s);

size_t gate_lds_bytes(int tile, int64_t nbK, int chunk_cap = 0);   // chunk_cap > 0: at most that many 64-k words of bitmaps in LDS at a time
inline size_t gate_lds_limit() { return 160 * 1024 - 64; }   // dynamic LDS of k_gate (a few static bytes aside)
// k_order ranks the super tiles of C (4 x 8 macro tiles of 256 x 256) in one workgroup's LDS
constexpr int LPT_MAX_SUPER = 2048;     // the greedy deal's table is laid out for at most this many super tiles,
constexpr int LPT_GREEDY_MAX = 64;      // and it runs while at most this many of them hold any work
constexpr int BAND_DEAL_MAX = 256;      // the grouped row-major deal runs up to this many super tiles with work
inline size_t order_lds_bytes(int tile, int64_t nbM, int64_t nbN) {
    const int MT = 256 / tile;
    const int64_t nMacM = (nbM + MT - 1) / MT, nMacN = (nbN + MT - 1) / MT;
    const size_t n_super = (size_t)(((nMacM + SUPER_M - 1) / SUPER_M) * ((nMacN + SUPER_N - 1) / SUPER_N));
    // length + origin by rank, and for the greedy deal a table of at most MAX_XCD x rounds (or
    // n_super parked ranks) 16-bit entries; beyond 512 super tiles the ranking sorts indices
    // padded to a power of two in the second array's place
    size_t np2 = 1024;
    while (np2 < n_super) np2 *= 2;
    const size_t tables = n_super * 2 * sizeof(int) + (n_super <= (size_t)LPT_MAX_SUPER ? (n_super + 2 * MAX_XCD) * sizeof(uint16_t) * 2 : 0);
    const size_t sorting = n_super > 512 ? (n_super + np2) * sizeof(int) : 0;
    return tables > sorting ? tables : sorting;
}
inline size_t order_lds_limit() { return 64 * 1024; }
hipError_t gate_init();   // one-time kernel attribute set-up
hipError_t launch_gate(const GateBuffers &g, int64_t nbM, int64_t nbK, int64_t nbN, int tile,
                       float tau, int n_xcd, int chunk_cap, hipStream_t s);
// per-tile ascending k lists [n_tiles x nbK] from the gate's bitmaps (read-back only)
hipError_t launch_klist(const uint64_t *mask, uint16_t *klist, int64_t n_tiles, int64_t nbK, hipStream_t s);

// tau selection (kernels_tau.hip)
struct TauState {
    unsigned long long want;      // rank (1-based, from the top) still to find inside the prefix
    unsigned long long greater;   // products strictly above the current prefix range
    unsigned long long kept;      // products >= tau (valid after the last pass)
    uint32_t prefix;              // decided high bits, right-aligned
    uint32_t tau_bits;
};
struct TauCounts {
    unsigned long long count;     // products with (double)p >= threshold
    unsigned long long positive;  // products > 0
    double sum;                   // sum of all products
};
size_t tau_workspace_bytes();
inline size_t tau_counts_offset() { return 64 + 2048 * 8; }
hipError_t launch_tau_select(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN,
                             unsigned long long want, void *workspace, hipStream_t s);
hipError_t launch_tau_count(const float *nA, const float *nBt, int64_t nbM, int64_t nbK, int64_t nbN,
                            double thr, void *workspace, hipStream_t s);

hipError_t gemm_init();   // one-time kernel attribute set-up
hipError_t launch_gemm(const void *packedA, const void *packedB, const GateBuffers &g, int64_t M,
                       int64_t K, int64_t N, int tile, float *C, int n_xcd, int n_cu, int ring, int shape, hipStream_t s);
// work unit of the gated GEMM: a whole macro tile (256 x 256 of C, one workgroup per CU), half of
// one (128 x 256, two workgroups per CU), a whole one by eight waves, or whole ones by workgroups
// that stay on their CU and draw items from a ticket counter per XCD
constexpr int GEMM_SHAPE_FULL = 1, GEMM_SHAPE_HALF = 2, GEMM_SHAPE_W8 = 3, GEMM_SHAPE_PERSIST = 4;
constexpr int SCHED_WORDS = 3 * MAX_XCD;     // GateBuffers::sched

}  // namespace spamm
