// libspamm_dev_gfx950.so: measurement aids kept apart from the engine (include/spamm_dev.h).
#include "../../include/spamm_dev.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

namespace {

// ---- matrix-pipeline ceiling: a grid of one workgroup per CU (4 waves, one per SIMD) that issues
// nothing but independent 32x32x16 fp16 MFMAs on 16 accumulator blocks per wave.  On this part the
// sustained clock under MFMA load depends on the operand values (power management), so the rate
// measured here with operands like the workload's is the ceiling a GEMM can reach, below the
// datasheet peak.  trace[2 b] = 100 MHz wall ticks, trace[2 b + 1] = shader clocks of workgroup b.
typedef _Float16 ceil_half8 __attribute__((ext_vector_type(8)));
typedef float ceil_f32x16 __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256) void k_mfma_ceiling(const ceil_half8 *__restrict__ in, float *__restrict__ out,
                                                      unsigned long long *__restrict__ trace, int iters) {
    ceil_half8 a[4], b[4];
    for (int i = 0; i < 4; i++) {
        a[i] = in[(i * 256 + threadIdx.x) % 2048];
        b[i] = in[((i + 4) * 256 + threadIdx.x) % 2048];
    }
    ceil_f32x16 acc[4][4];
    for (int r = 0; r < 4; r++)
        for (int c = 0; c < 4; c++)
            for (int i = 0; i < 16; i++) acc[r][c][i] = 0.0f;
    const unsigned long long w0 = wall_clock64(), c0 = clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int c = 0; c < 4; c++)
                acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[r], b[c], acc[r][c], 0, 0, 0);
    }
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    float s = 0.0f;
    for (int r = 0; r < 4; r++)
        for (int c = 0; c < 4; c++)
            for (int i = 0; i < 16; i++) s += acc[r][c][i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (threadIdx.x == 0) {
        trace[blockIdx.x * 2] = w1 - w0;
        trace[blockIdx.x * 2 + 1] = c1 - c0;
    }
}



// ---- read-only reference kernel: every thread walks the buffer with a grid stride, one 16-byte load
// in flight per thread and trip; CASE only gives the four uses distinct kernel names in a profile
// (0: large buffer, full grid = HBM under load; 1: small buffer re-read, full grid = memory-side cache
// under load; 2 / 3: the same two with a few workgroups = latency with idle queues).
template <int CASE>
__global__ __launch_bounds__(256) void k_dev_read(const uint4 *__restrict__ p, size_t n16, int passes,
                                                  unsigned *__restrict__ out) {
    unsigned acc = 0;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (int r = 0; r < passes; r++)
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
            const uint4 v = p[i];
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
        }
    if (acc == 0x9e3779b9u) out[0] = acc;       // keeps the loads alive; practically never taken
}

struct Cleanup {
    void *buf = nullptr;
    hipStream_t stream = nullptr;
    ~Cleanup() {
        if (buf) (void)hipFree(buf);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

}  // namespace

#define DEVCHK(call)                                  \
    do {                                              \
        hipError_t e__ = (call);                      \
        if (e__ != hipSuccess) {                      \
            (void)hipGetLastError();                  \
            return -(int)e__;                         \
        }                                             \
    } while (0)

extern "C" int spamm_dev_read_reference(int device, int which, double *gbps) {
    if (!gbps || which < 0 || which > 3 || device < 0) return -1;
    DEVCHK(hipSetDevice(device));
    const size_t bytes = (which & 1) ? ((size_t)96 << 20) : ((size_t)4 << 30);
    const int passes = (which & 1) ? 40 : 1;
    const int n_wg = (which & 2) ? 32 : 4096;
    Cleanup cl;
    DEVCHK(hipStreamCreate(&cl.stream));
    DEVCHK(hipMalloc(&cl.buf, bytes + 256));
    DEVCHK(hipMemsetAsync(cl.buf, 1, bytes + 256, cl.stream));
    hipEvent_t e0, e1;
    DEVCHK(hipEventCreate(&e0));
    DEVCHK(hipEventCreate(&e1));
    const uint4 *p = (const uint4 *)cl.buf;
    unsigned *out = (unsigned *)((char *)cl.buf + bytes);
    float best = 0.0f;
    for (int rep = 0; rep < 3; rep++) {
        DEVCHK(hipEventRecord(e0, cl.stream));
        switch (which) {
            case 0: k_dev_read<0><<<n_wg, 256, 0, cl.stream>>>(p, bytes / 16, passes, out); break;
            case 1: k_dev_read<1><<<n_wg, 256, 0, cl.stream>>>(p, bytes / 16, passes, out); break;
            case 2: k_dev_read<2><<<n_wg, 256, 0, cl.stream>>>(p, bytes / 16, passes, out); break;
            default: k_dev_read<3><<<n_wg, 256, 0, cl.stream>>>(p, bytes / 16, passes, out); break;
        }
        DEVCHK(hipGetLastError());
        DEVCHK(hipEventRecord(e1, cl.stream));
        DEVCHK(hipEventSynchronize(e1));
        float ms = 0.0f;
        DEVCHK(hipEventElapsedTime(&ms, e0, e1));
        if (rep == 0 || ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *gbps = (double)bytes * passes / (best * 1e-3) / 1e9;
    return 0;
}

extern "C" int spamm_dev_mfma_ceiling(int device, int random_operands, int iters, double *tflops, double *clock_ghz) {
    if (!tflops || !clock_ghz || iters <= 0 || iters > (1 << 20) || device < 0) return -1;
    DEVCHK(hipSetDevice(device));
    int n_wg = 0;
    DEVCHK(hipDeviceGetAttribute(&n_wg, hipDeviceAttributeMultiprocessorCount, device));
    if (n_wg <= 0 || n_wg > 4096) return -1;
    // operands: 2048 vectors of 8 halves, zeros or uniform in [-1, 1) (a fixed LCG sequence)
    std::vector<_Float16> h(2048 * 8);
    uint32_t x = 12345u;
    for (size_t i = 0; i < h.size(); i++) {
        x = x * 1664525u + 1013904223u;
        h[i] = random_operands ? (_Float16)(((float)(x >> 8) / 8388608.0f) - 1.0f) : (_Float16)0.0f;
    }
    const size_t in_bytes = h.size() * 2, out_bytes = (size_t)n_wg * 256 * 4, tr_bytes = (size_t)n_wg * 16;
    Cleanup cl;
    DEVCHK(hipStreamCreate(&cl.stream));
    DEVCHK(hipMalloc(&cl.buf, in_bytes + out_bytes + tr_bytes));
    char *base = (char *)cl.buf;
    DEVCHK(hipMemcpyAsync(base, h.data(), in_bytes, hipMemcpyHostToDevice, cl.stream));
    DEVCHK(hipStreamSynchronize(cl.stream));
    double best_ns = 0.0, best_clk = 0.0;
    std::vector<unsigned long long> tr((size_t)n_wg * 2);
    for (int rep = 0; rep < 3; rep++) {   // the clock settles over the first launches; keep the last
        k_mfma_ceiling<<<n_wg, 256, 0, cl.stream>>>((const ceil_half8 *)base, (float *)(base + in_bytes),
                                                    (unsigned long long *)(base + in_bytes + out_bytes), iters);
        DEVCHK(hipGetLastError());
        DEVCHK(hipMemcpyAsync(tr.data(), base + in_bytes + out_bytes, tr_bytes, hipMemcpyDeviceToHost, cl.stream));
        DEVCHK(hipStreamSynchronize(cl.stream));
        double w = 0.0, k = 0.0;
        for (int i = 0; i < n_wg; i++) { w += (double)tr[2 * i]; k += (double)tr[2 * i + 1]; }
        best_ns = w / n_wg * 10.0;        // wall ticks are 10 ns
        best_clk = k / n_wg;
    }
    if (best_ns <= 0.0) return -1;
    const double flops = (double)iters * 16.0 * 32768.0 * 4.0 * n_wg;   // per MFMA 2*32*32*16, 4 waves per workgroup
    *tflops = flops / best_ns * 1e-3;
    *clock_ghz = best_clk / best_ns;
    return 0;
}
