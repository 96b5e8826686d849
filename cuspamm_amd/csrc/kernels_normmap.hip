// Stage 1: fused fp32 -> fp16 conversion + tile Frobenius norm map.
//
// Replaces the reference's norm kernels (cuSpAMM.cu:21-71 fp32, :74-123 fp16)
// and its host-side element-wise __float2half (tool.cu:418,432).  HBM-bound:
// per element 4 bytes read, 2 bytes written.  The fp16 copy is written in the
// packed tile layout described in spamm_internal.h so that the gated GEMM can
// stream MFMA operands without any transposition.
//
// Norm accumulation order (fp32, bit-identical to the host checker):
//   chunk(r,q) = ((((0 + x0^2) + x1^2) + ... ) + x7^2) over 8 consecutive
//   elements along the contraction axis (x = fp16-rounded value; squares are
//   exact in fp32); chunk index c = r*(b/8)+q; lane L = c%64 accumulates
//   chunks c = L, 64+L, 128+L, ... in ascending order; then a 6-step xor
//   butterfly (1,2,4,8,16,32) across the 64 lanes; norm = sqrtf(sum).
#include "spamm_internal.h"

namespace spamm {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Convert two floats to fp16 (round-to-nearest-even), add their squares to s
// in order (a then b) and return the packed pair.
__device__ __forceinline__ uint32_t cvt_pack2(float a, float b, float &s) {
    _Float16 ha = (_Float16)a;
    _Float16 hb = (_Float16)b;
    float fa = (float)ha;
    float fb = (float)hb;
    s = s + fa * fa;
    s = s + fb * fb;
    half2v v = {ha, hb};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float butterfly64(float v) {
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) v = v + __shfl_xor(v, s, 64);
    return v;
}

// ------------------------------------------------------------------ role A
// One wave per tile.  Lane L covers chunk column q = L % (B/8) of rows
// rl + it*RPI, rl = L / (B/8): every wave-wide load reads RPI full tile rows
// (B*4 contiguous bytes each) and the chunk index of lane L at step `it` is
// exactly it*64 + L, so the canonical order needs no data exchange.
template <int B>
__global__ __launch_bounds__(256) void k_normmap_a(const float *__restrict__ X, int64_t ld,
                                                   int64_t nbc, int64_t ntiles,
                                                   uint4 *__restrict__ packed,
                                                   float *__restrict__ nm) {
    constexpr int QN = B / 8;
    constexpr int RPI = 64 / QN;
    constexpr int IT = B / RPI;
    constexpr int UN = IT < 8 ? IT : 8;
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= ntiles) return;
    const int64_t I = t / nbc, J = t % nbc;
    const int q = lane % QN, rl = lane / QN;
    const float *src = X + (I * B + rl) * ld + J * B + 8 * q;
    uint4 *dst = packed + t * (B * B / 8) + q * B + rl;
    float partial = 0.0f;
    for (int it0 = 0; it0 < IT; it0 += UN) {
        f32x4 v0[UN], v1[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const f32x4 *p = reinterpret_cast<const f32x4 *>(src + (int64_t)(it0 + u) * RPI * ld);
            v0[u] = __builtin_nontemporal_load(p);
            v1[u] = __builtin_nontemporal_load(p + 1);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            float s = 0.0f;
            uint4 o;
            o.x = cvt_pack2(v0[u].x, v0[u].y, s);
            o.y = cvt_pack2(v0[u].z, v0[u].w, s);
            o.z = cvt_pack2(v1[u].x, v1[u].y, s);
            o.w = cvt_pack2(v1[u].z, v1[u].w, s);
            partial = partial + s;
            dst[(it0 + u) * RPI] = o;
        }
    }
    partial = butterfly64(partial);
    if (lane == 0) nm[t] = sqrtf(partial);
}

// ------------------------------------------------------------------ role B
// The contraction axis is the row axis, so a lane needs 8 consecutive rows of
// one column.  Lane L reads a float4 (4 columns) from 8 consecutive rows and
// transposes in registers: 4 output vectors of 8 halves, 64 contiguous bytes
// of the packed tile.  A wave covers CW = max(B,64) columns (two tiles when
// B = 32) and KGPI k-groups per step.  Chunk sums go through a wave-private
// LDS strip so that the canonical order can be applied afterwards.
template <int B>
__global__ __launch_bounds__(256) void k_normmap_b(const float *__restrict__ X, int64_t ld,
                                                   int64_t nbK, int64_t nbN, int64_t nJw,
                                                   uint4 *__restrict__ packed,
                                                   float *__restrict__ nm,
                                                   float *__restrict__ nmT) {
    constexpr int CW = B < 64 ? 64 : B;
    constexpr int TPW = CW / B;           // tiles per wave
    constexpr int L4 = CW / 4;            // lanes across one row
    constexpr int KGPI = 64 / L4;         // k-groups per step
    constexpr int QN = B / 8;             // k-groups per tile
    constexpr int IT = QN / KGPI;
    constexpr int PITCH = QN + 1;         // padded LDS row: conflict-free dump
    constexpr int STEPS = B * B / 8 / 64;
    __shared__ float lds[4][TPW * B * PITCH];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t w = (int64_t)blockIdx.x * 4 + wave;
    const bool active = w < nbK * nJw;
    const int64_t Kt = active ? w / nJw : 0;
    const int64_t Jw = active ? w % nJw : 0;
    const int n4 = lane % L4, kgl = lane / L4;
    const int64_t col0 = Jw * CW + 4 * n4;
    const bool valid = active && col0 < nbN * B;
    const int ts = (4 * n4) / B;                 // which tile of the wave
    const int nl = (4 * n4) % B;                 // first column inside that tile
    const int64_t J = Jw * TPW + ts;
    float *strip = lds[wave];

    if (valid) {
        uint4 *dtile = packed + (J * nbK + Kt) * (int64_t)(B * B / 8);
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const int kg = it * KGPI + kgl;
            const float *src = X + (Kt * B + kg * 8) * ld + col0;
            f32x4 v[8];
#pragma unroll
            for (int j = 0; j < 8; j++)
                v[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + j * ld));
            uint4 o[4];
            float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            o[0].x = cvt_pack2(v[0].x, v[1].x, s[0]);
            o[0].y = cvt_pack2(v[2].x, v[3].x, s[0]);
            o[0].z = cvt_pack2(v[4].x, v[5].x, s[0]);
            o[0].w = cvt_pack2(v[6].x, v[7].x, s[0]);
            o[1].x = cvt_pack2(v[0].y, v[1].y, s[1]);
            o[1].y = cvt_pack2(v[2].y, v[3].y, s[1]);
            o[1].z = cvt_pack2(v[4].y, v[5].y, s[1]);
            o[1].w = cvt_pack2(v[6].y, v[7].y, s[1]);
            o[2].x = cvt_pack2(v[0].z, v[1].z, s[2]);
            o[2].y = cvt_pack2(v[2].z, v[3].z, s[2]);
            o[2].z = cvt_pack2(v[4].z, v[5].z, s[2]);
            o[2].w = cvt_pack2(v[6].z, v[7].z, s[2]);
            o[3].x = cvt_pack2(v[0].w, v[1].w, s[3]);
            o[3].y = cvt_pack2(v[2].w, v[3].w, s[3]);
            o[3].z = cvt_pack2(v[4].w, v[5].w, s[3]);
            o[3].w = cvt_pack2(v[6].w, v[7].w, s[3]);
            uint4 *d = dtile + kg * B + nl;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                d[c] = o[c];
                strip[(ts * B + nl + c) * PITCH + kg] = s[c];
            }
        }
    }
    __syncthreads();
    if (!active) return;
#pragma unroll
    for (int tsel = 0; tsel < TPW; tsel++) {
        const int64_t Jt = Jw * TPW + tsel;
        if (Jt >= nbN) break;
        float partial = 0.0f;
        for (int it = 0; it < STEPS; it++) {
            const int c = it * 64 + lane;
            const int r = c / QN, q = c % QN;
            partial = partial + strip[(tsel * B + r) * PITCH + q];
        }
        partial = butterfly64(partial);
        if (lane == 0) {
            const float nv = sqrtf(partial);
            nm[Kt * nbN + Jt] = nv;
            nmT[Jt * nbK + Kt] = nv;
        }
    }
}

// ------------------------------------------------------------- utilities
// Packed fp16 -> row-major fp16 bit patterns (read-back helper, not on the
// hot path).  One thread per 16-byte vector.
__global__ void k_unpack(const uint4 *__restrict__ packed, int64_t rows, int64_t cols, int B,
                         int role, uint16_t *__restrict__ out) {
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t nvec = rows * cols / 8;
    if (v >= nvec) return;
    const int64_t vpt = (int64_t)B * B / 8;
    const int64_t tile = v / vpt;
    const int iv = (int)(v % vpt);
    const int kg = iv / B, r = iv % B;
    const uint4 d = packed[v];
    const uint32_t wds[4] = {d.x, d.y, d.z, d.w};
    if (role == 0) {
        const int64_t nbK = cols / B;
        const int64_t I = tile / nbK, Kt = tile % nbK;
        uint16_t *o = out + (I * B + r) * cols + Kt * B + kg * 8;
        for (int e = 0; e < 8; e++) o[e] = (uint16_t)(wds[e >> 1] >> ((e & 1) * 16));
    } else {
        const int64_t nbK = rows / B;
        const int64_t J = tile / nbK, Kt = tile % nbK;
        for (int e = 0; e < 8; e++)
            out[(Kt * B + kg * 8 + e) * cols + J * B + r] =
                (uint16_t)(wds[e >> 1] >> ((e & 1) * 16));
    }
}

__global__ void k_transpose_nm(const float *__restrict__ nB, int64_t nbK, int64_t nbN,
                               float *__restrict__ nBt) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nbK * nbN) return;
    const int64_t k = i / nbN, j = i % nbN;
    nBt[j * nbK + k] = nB[i];
}

// Synthetic inputs (tool.cu:370-436 plus a seeded uniform factor): the hash
// and the single fp32 multiply are the same integer / IEEE operations as in
// the host checker, so device and host inputs are bit-identical.
__device__ __forceinline__ float hash_uniform(uint64_t seed, uint64_t idx) {
    uint64_t z = idx + seed * 0x9E3779B97F4A7C15ull + 0x632BE59BD9B4E019ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const uint32_t k = (uint32_t)(z >> 40);
    return (float)k * 1.1920928955078125e-07f - 1.0f;
}

__global__ __launch_bounds__(256) void k_fill_decay(float *__restrict__ X, int64_t rows,
                                                    int64_t cols, const float *__restrict__ table,
                                                    uint64_t seed, int random) {
    const int64_t n4 = rows * cols / 4;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < n4;
         v += (int64_t)gridDim.x * blockDim.x) {
        const int64_t e0 = v * 4;
        const int64_t i = e0 / cols, j0 = e0 % cols;
        float o[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int64_t j = j0 + c;
            const int64_t d = i > j ? i - j : j - i;
            const float u = random ? hash_uniform(seed, (uint64_t)(e0 + c)) : 1.0f;
            o[c] = u * table[d];
        }
        reinterpret_cast<float4 *>(X)[v] = make_float4(o[0], o[1], o[2], o[3]);
    }
}

// ---------------------------------------------------------------- launchers
hipError_t launch_normmap_a(const float *X, int64_t rows, int64_t cols, int tile, void *packed,
                            float *nm, hipStream_t s) {
    const int64_t nbr = rows / tile, nbc = cols / tile;
    const int64_t ntiles = nbr * nbc;
    const unsigned grid = (unsigned)((ntiles + 3) / 4);
    switch (tile) {
        case 32: k_normmap_a<32><<<grid, 256, 0, s>>>(X, cols, nbc, ntiles, (uint4 *)packed, nm); break;
        case 64: k_normmap_a<64><<<grid, 256, 0, s>>>(X, cols, nbc, ntiles, (uint4 *)packed, nm); break;
        case 128: k_normmap_a<128><<<grid, 256, 0, s>>>(X, cols, nbc, ntiles, (uint4 *)packed, nm); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_normmap_b(const float *X, int64_t rows, int64_t cols, int tile, void *packed,
                            float *nm, float *nmT, hipStream_t s) {
    const int64_t nbK = rows / tile, nbN = cols / tile;
    const int cw = tile < 64 ? 64 : tile;
    const int64_t nJw = (cols + cw - 1) / cw;
    const unsigned grid = (unsigned)((nbK * nJw + 3) / 4);
    switch (tile) {
        case 32: k_normmap_b<32><<<grid, 256, 0, s>>>(X, cols, nbK, nbN, nJw, (uint4 *)packed, nm, nmT); break;
        case 64: k_normmap_b<64><<<grid, 256, 0, s>>>(X, cols, nbK, nbN, nJw, (uint4 *)packed, nm, nmT); break;
        case 128: k_normmap_b<128><<<grid, 256, 0, s>>>(X, cols, nbK, nbN, nJw, (uint4 *)packed, nm, nmT); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_unpack(const void *packed, int64_t rows, int64_t cols, int tile, int role,
                         uint16_t *out, hipStream_t s) {
    const int64_t nvec = rows * cols / 8;
    k_unpack<<<(unsigned)((nvec + 255) / 256), 256, 0, s>>>((const uint4 *)packed, rows, cols, tile,
                                                            role, out);
    return hipGetLastError();
}

hipError_t launch_transpose_normmap(const float *nB, int64_t nbK, int64_t nbN, float *nBt,
                                    hipStream_t s) {
    const int64_t n = nbK * nbN;
    k_transpose_nm<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(nB, nbK, nbN, nBt);
    return hipGetLastError();
}

hipError_t launch_fill_decay(float *X, int64_t rows, int64_t cols, const float *table,
                             uint64_t seed, int random, hipStream_t s) {
    const int64_t n4 = rows * cols / 4;
    int64_t blocks = (n4 + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    k_fill_decay<<<(unsigned)blocks, 256, 0, s>>>(X, rows, cols, table, seed, random);
    return hipGetLastError();
}

}  // namespace spamm
