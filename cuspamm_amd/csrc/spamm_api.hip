// C ABI of libspamm_gfx950.so: the host driver that replaces the timed body of
// the reference's main() (cuSpAMM.cu:458-546) and its per-device plan
// (TGPUplan, cuSpAMM.cu:6-12, 433-451).  See include/spamm.h for the contract.
#include "../../include/spamm.h"

#include <math.h>
#include <atomic>
#include <new>
#include <utility>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

#include "spamm_internal.h"

using namespace spamm;

// Workspace of spamm_multiply_noalloc: one fixed array per GPU, part of the code object, held from
// the moment the library is loaded until the process ends.  In host code this name is only a
// handle for hipGetSymbolAddress: the device address is looked up once per context (= per device)
// in spamm_create and everything below uses that pointer.
static __device__ __align__(256) unsigned char scratch[SPAMM_NOALLOC_WORKSPACE_BYTES];

// Every spamm_multiply_noalloc on a device overwrites that device's array, whichever context makes
// the call: a per-device generation number, bumped by each such call, tells a context whether what
// it left there is still its own (see static_stale).
static constexpr int MAX_DEVICES = 64;
static std::atomic<uint64_t> g_static_gen[MAX_DEVICES];

namespace {

struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    bool borrowed = false;    // p points into the fixed device array: never freed
};

}  // namespace

// Everything a multiply leaves behind: the shape it ran at, what is valid, and
// the device buffers.  A context holds two of these: its own (hipMalloc'd, grown
// on demand) and one carved out of the library's fixed device array for
// spamm_multiply_noalloc; `static_cast<Workspace &>(*ctx)` is the live one.
struct Workspace {
    // problem shape of the current workspace contents
    int64_t M = 0, K = 0, N = 0;
    int tile = 0;
    bool have_a = false, have_b = false, have_gate = false;
    // nA / nB+nBt hold norm maps of the current M x K / K x N at the current tile
    bool nm_a = false, nm_b = false;
    float tau = 0.0f;
    // A's fp16 copy was written by a tau-aware pass: tiles that no product can keep at
    // a_pruned_tau are missing, so the copy serves a GEMM only for tau >= a_pruned_tau
    bool a_pruned = false;
    float a_pruned_tau = 0.0f;
    // B's fp16 copy lacks its tiles of norm zero: it serves any tau > 0
    bool b_pruned = false;

    DevBuf packedA, packedB, nA, nB, nBt, rowmaxB;
    DevBuf counts, klist, mask, macro_list, macro_count, macro_work, order, sched, kept_total;
};

struct spamm_ctx : Workspace {
    int device = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    int last_hip = 0;
    int n_xcd = MAX_XCD;        // XCDs the GEMM schedule is built for (from the device's CU count)
    int n_cu = MAX_XCD * SUPER_M * SUPER_N;     // CUs of the device
    int gate_chunk_cap = 0;     // SPAMM_OPT_GATE_CHUNK_WORDS: the gate's k chunk, 0 = what LDS holds
    int gemm_ring = 4;          // SPAMM_OPT_GEMM_RING: LDS stages of the GEMM's staging ring
    int gemm_shape = 0;         // SPAMM_OPT_GEMM_SHAPE: 0 = chosen per call, else one of GEMM_SHAPE_*
    uint64_t static_gen = 0;    // generation of the fixed array this context's noalloc results belong to

    Workspace parked;           // the workspace that is not live (see in_static)
    bool in_static = false;     // live workspace = carve-outs of the fixed device array
    bool no_alloc = false;      // inside spamm_multiply_noalloc: ensure() must not allocate
    unsigned char *static_ptr = nullptr;   // device address of the fixed array on this context's device

    DevBuf staging;   // read-back staging / decay table
    DevBuf tauws;     // tau selection workspace

    hipEvent_t ev[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    bool timing = false;        // events of the last multiply are valid
    bool ev_a = false, ev_b = false, ev_gate = false, ev_gemm = false;
};

namespace {

#define HIPCHK(ctx, call)                         \
    do {                                          \
        hipError_t e__ = (call);                  \
        if (e__ != hipSuccess) {                  \
            (ctx)->last_hip = (int)e__;           \
            (void)hipGetLastError();              \
            return e__ == hipErrorOutOfMemory ? SPAMM_ENOMEM : SPAMM_EHIP; \
        }                                         \
    } while (0)

int ensure(spamm_ctx *c, DevBuf &b, size_t bytes) {
    if (bytes == 0) bytes = 16;
    if (b.cap >= bytes) return SPAMM_OK;
    if (c->no_alloc) return SPAMM_ELIMIT;       // the carve-out was sized by the same formulas: not reached
    if (b.p && !b.borrowed) {
        HIPCHK(c, hipStreamSynchronize(c->stream));
        HIPCHK(c, hipFree(b.p));
    }
    b.p = nullptr;
    b.cap = 0;
    b.borrowed = false;
    HIPCHK(c, hipMalloc(&b.p, bytes));
    b.cap = bytes;
    return SPAMM_OK;
}

bool tile_ok(int t) { return t == 32 || t == 64 || t == 128; }

struct Shape {
    int64_t nbM, nbK, nbN, words, n_macro;
};

Shape shape_of(const spamm_ctx *c) {
    Shape s;
    s.nbM = c->M / c->tile;
    s.nbK = c->K / c->tile;
    s.nbN = c->N / c->tile;
    s.words = (s.nbK + 63) / 64;
    const int MT = macro_dim(c->tile);
    s.n_macro = ((s.nbM + MT - 1) / MT) * ((s.nbN + MT - 1) / MT);
    return s;
}

GateBuffers gate_buffers(spamm_ctx *c) {
    GateBuffers g;
    g.nA = (const float *)c->nA.p;
    g.nBt = (const float *)c->nBt.p;
    g.counts = (int32_t *)c->counts.p;
    g.mask = (uint64_t *)c->mask.p;
    g.macro_list = (MacroEntry *)c->macro_list.p;
    g.macro_count = (int32_t *)c->macro_count.p;
    g.macro_work = (int32_t *)c->macro_work.p;
    g.order = (int32_t *)c->order.p;
    g.sched = (int32_t *)c->sched.p;
    g.kept_total = (int64_t *)c->kept_total.p;
    return g;
}

// Work unit of the gated GEMM when the caller has not fixed it: with at most half a macro tile per CU
// halves double the workgroups that run at once (2048^3 at tile 32, 64 macro tiles: -6 %); from one
// macro tile per CU on, whole macro tiles by four waves are as fast or faster (4096^3 dense, 256 macro
// tiles: halves +7 %; 128 flop per staged byte against 85).  Between one and three COMPUTING macro
// tiles per CU halves can win up to 10 % by finer rounds (270 on 256 CUs), but that count is known
// only on the device after the gate, and the host chooses the launch.
int gemm_shape_for(const spamm_ctx *c) {
    if (c->gemm_shape) return c->gemm_shape;
    const Shape s = shape_of(c);
    return 2 * s.n_macro <= (int64_t)c->n_xcd * SUPER_M * SUPER_N ? GEMM_SHAPE_HALF : GEMM_SHAPE_FULL;
}

int set_device(spamm_ctx *c) {
    HIPCHK(c, hipSetDevice(c->device));
    return SPAMM_OK;
}

// Called when an operand with a different shape/tile arrives: everything
// derived from the old shape is stale.
void reset_shape(spamm_ctx *c, int tile) {
    c->tile = tile;
    c->M = c->K = c->N = 0;
    c->have_a = c->have_b = c->have_gate = false;
    c->nm_a = c->nm_b = false;
    c->a_pruned = c->b_pruned = false;
}

// The buffers of a workspace that the library allocated (carve-outs of the fixed array are not freed).
void free_workspace(Workspace &w) {
    DevBuf *bufs[] = {&w.packedA, &w.packedB, &w.nA, &w.nB, &w.nBt, &w.rowmaxB, &w.counts, &w.klist,
                      &w.mask, &w.macro_list, &w.macro_count, &w.macro_work, &w.order, &w.sched, &w.kept_total};
    for (DevBuf *b : bufs) {
        if (b->p && !b->borrowed) (void)hipFree(b->p);
        *b = DevBuf();
    }
}

// An ordinary producing call (multiply, norm-map stage, uploaded norm maps) works in the context's
// own workspace: if the last call was spamm_multiply_noalloc, bring it back.  Its contents and
// validity flags are as the last ordinary call left them.
void leave_static(spamm_ctx *c) {
    if (!c->in_static || c->no_alloc) return;
    std::swap(static_cast<Workspace &>(*c), c->parked);
    c->in_static = false;
}

// The live workspace is the fixed array and another spamm_multiply_noalloc on this device (from
// any context) has overwritten it since: nothing this context left there can be read or consumed.
bool static_stale(const spamm_ctx *c) {
    return c->in_static && c->static_gen != g_static_gen[c->device].load(std::memory_order_acquire);
}

int copy_out(spamm_ctx *c, const void *dev, void *host, size_t bytes) {
    HIPCHK(c, hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return SPAMM_OK;
}

}  // namespace

extern "C" {

int spamm_version(void) { return 100; }

const char *spamm_strerror(int code) {
    switch (code) {
        case SPAMM_OK: return "ok";
        case SPAMM_EINVAL: return "invalid argument (dimension not a multiple of tile, tile not in {32,64,128}, null pointer, or size limit)";
        case SPAMM_ENOMEM: return "out of memory";
        case SPAMM_EHIP: return "HIP runtime error (see spamm_last_hip_error)";
        case SPAMM_ESTATE: return "stage called before the stage it depends on";
        case SPAMM_ENODEV: return "no usable gfx950 device";
        case SPAMM_ELIMIT: return "problem needs more than the fixed workspace of spamm_multiply_noalloc";
        default: return "unknown error";
    }
}

int spamm_create(spamm_ctx **out, int device) {
    if (!out) return SPAMM_EINVAL;
    *out = nullptr;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0) {
        (void)hipGetLastError();
        return SPAMM_ENODEV;
    }
    if (device < 0 || device >= ndev || device >= MAX_DEVICES) return SPAMM_EINVAL;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return SPAMM_ENODEV;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return SPAMM_ENODEV;
    spamm_ctx *c = new (std::nothrow) spamm_ctx();
    if (!c) return SPAMM_ENOMEM;
    c->device = device;
    // the schedule groups workgroups by XCD (32 CUs sharing an L2): 256 CUs = 8 XCDs; a partitioned
    // device shows 128 / 64 / 32 CUs; any other CU count gets one flat sequence
    c->n_xcd = xcds_for_cu_count(prop.multiProcessorCount);
    c->n_cu = prop.multiProcessorCount;
    int rc = set_device(c);
    if (rc == SPAMM_OK && hipStreamCreate(&c->own_stream) != hipSuccess) rc = SPAMM_EHIP;
    c->stream = c->own_stream;
    for (int i = 0; i < 5 && rc == SPAMM_OK; i++)
        if (hipEventCreate(&c->ev[i]) != hipSuccess) rc = SPAMM_EHIP;
    if (rc == SPAMM_OK && (gemm_init() != hipSuccess || gate_init() != hipSuccess)) rc = SPAMM_EHIP;
    if (rc == SPAMM_OK) {
        // this device's copy of the fixed workspace array (each GPU has its own, at its own address)
        void *sp = nullptr;
        if (hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)) != hipSuccess || !sp) rc = SPAMM_EHIP;
        c->static_ptr = (unsigned char *)sp;
    }
    if (rc != SPAMM_OK) {
        (void)hipGetLastError();
        spamm_destroy(c);          // releases whatever was created
        return rc;
    }
    *out = c;
    return SPAMM_OK;
}

int spamm_destroy(spamm_ctx *c) {
    if (!c) return SPAMM_EINVAL;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    free_workspace(*c);
    free_workspace(c->parked);
    if (c->staging.p) (void)hipFree(c->staging.p);
    if (c->tauws.p) (void)hipFree(c->tauws.p);
    for (int i = 0; i < 5; i++)
        if (c->ev[i]) (void)hipEventDestroy(c->ev[i]);
    if (c->own_stream) (void)hipStreamDestroy(c->own_stream);
    delete c;
    return SPAMM_OK;
}

int spamm_set_stream(spamm_ctx *c, void *hip_stream) {
    if (!c) return SPAMM_EINVAL;
    c->stream = hip_stream ? (hipStream_t)hip_stream : c->own_stream;
    return SPAMM_OK;
}

int spamm_set_option(spamm_ctx *c, int option, int value) {
    if (!c) return SPAMM_EINVAL;
    switch (option) {
        case SPAMM_OPT_NUM_XCD:
            if (value == 0) {
                hipDeviceProp_t prop;
                if (hipGetDeviceProperties(&prop, c->device) != hipSuccess) return SPAMM_EHIP;
                value = xcds_for_cu_count(prop.multiProcessorCount);
            }
            if (value != 1 && value != 2 && value != 4 && value != 8) return SPAMM_EINVAL;
            c->n_xcd = value;
            c->have_gate = false;          // the schedule was built for the old count
            return SPAMM_OK;
        case SPAMM_OPT_GATE_CHUNK_WORDS:
            if (value < 0) return SPAMM_EINVAL;
            c->gate_chunk_cap = value;
            return SPAMM_OK;
        case SPAMM_OPT_GEMM_RING:
            if (value == 0) value = 4;
            if (value < 3 || value > 5) return SPAMM_EINVAL;
            c->gemm_ring = value;
            return SPAMM_OK;
        case SPAMM_OPT_GEMM_SHAPE:
            if (value < 0 || value > GEMM_SHAPE_PERSIST) return SPAMM_EINVAL;
            c->gemm_shape = value;
            return SPAMM_OK;
        default:
            return SPAMM_EINVAL;
    }
}

int spamm_last_hip_error(spamm_ctx *c) { return c ? c->last_hip : 0; }

int spamm_synchronize(spamm_ctx *c) {
    if (!c) return SPAMM_EINVAL;
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return SPAMM_OK;
}

static int normmap_any(spamm_ctx *c, int role, const void *dX, bool in16, int64_t rows, int64_t cols,
                       int32_t tile, const float *prune_tau = nullptr) {
    if (!c || !dX || !tile_ok(tile)) return SPAMM_EINVAL;
    if (role != SPAMM_ROLE_A && role != SPAMM_ROLE_B) return SPAMM_EINVAL;
    if (rows <= 0 || cols <= 0 || rows % tile || cols % tile) return SPAMM_EINVAL;
    if (rows / tile > 65535 || cols / tile > 65535) return SPAMM_EINVAL;
    int rc = set_device(c);
    if (rc) return rc;
    leave_static(c);
    if (c->tile != tile) reset_shape(c, tile);
    const size_t nt = (size_t)(rows / tile) * (size_t)(cols / tile);
    c->have_gate = false;
    if (role == SPAMM_ROLE_A) {
        // a new A invalidates B (fp16 copy and norm map alike) only if the shared dimension K
        // changes; A itself is invalid until its pass has been launched
        if (c->K != cols) c->have_b = c->nm_b = false;
        c->have_a = c->nm_a = false;
        c->a_pruned = false;
        c->M = rows;
        c->K = cols;
        if ((rc = ensure(c, c->packedA, (size_t)rows * cols * 2))) return rc;
        if ((rc = ensure(c, c->nA, nt * 4))) return rc;
        // tau-aware pass: needs B's norm map of the same K (the caller checked have_b)
        const bool prune = prune_tau != nullptr && *prune_tau > 0.0f && c->have_b && c->nB.p;
        if (prune) {
            if ((rc = ensure(c, c->rowmaxB, (size_t)(cols / tile) * 4))) return rc;
            HIPCHK(c, launch_rowmax((const float *)c->nB.p, cols / tile, c->N / tile, (float *)c->rowmaxB.p, c->stream));
        }
        if (c->timing) HIPCHK(c, hipEventRecord(c->ev[1], c->stream));
        HIPCHK(c, launch_normmap_a(dX, in16, rows, cols, tile, c->packedA.p, (float *)c->nA.p,
                                   prune ? (const float *)c->rowmaxB.p : nullptr, prune ? *prune_tau : 0.0f, c->stream));
        if (c->timing) { HIPCHK(c, hipEventRecord(c->ev[2], c->stream)); c->ev_a = true; }
        c->have_a = c->nm_a = true;
        c->a_pruned = prune;
        c->a_pruned_tau = prune ? *prune_tau : 0.0f;
    } else {
        if (c->K != rows) c->have_a = c->nm_a = false;
        if (c->a_pruned) c->have_a = false;     // pruned against the previous B's norms
        c->have_b = c->nm_b = false;
        c->b_pruned = false;
        c->K = rows;
        c->N = cols;
        if ((rc = ensure(c, c->packedB, (size_t)rows * cols * 2))) return rc;
        if ((rc = ensure(c, c->nB, nt * 4))) return rc;
        if ((rc = ensure(c, c->nBt, nt * 4))) return rc;
        if (c->timing) HIPCHK(c, hipEventRecord(c->ev[0], c->stream));
        const bool prune = prune_tau != nullptr && *prune_tau > 0.0f;
        HIPCHK(c, launch_normmap_b(dX, in16, rows, cols, tile, c->packedB.p, (float *)c->nB.p,
                                   (float *)c->nBt.p, prune ? *prune_tau : 0.0f, c->stream));
        if (c->timing) { HIPCHK(c, hipEventRecord(c->ev[1], c->stream)); c->ev_b = true; }
        c->have_b = c->nm_b = true;
        c->b_pruned = prune;
    }
    return SPAMM_OK;
}

int spamm_normmap_f32(spamm_ctx *c, int role, const float *dX, int64_t rows, int64_t cols,
                      int32_t tile) {
    return normmap_any(c, role, dX, false, rows, cols, tile);
}

int spamm_normmap_f16(spamm_ctx *c, int role, const void *dXh, int64_t rows, int64_t cols,
                      int32_t tile) {
    return normmap_any(c, role, dXh, true, rows, cols, tile);
}

int spamm_set_normmaps(spamm_ctx *c, const float *nA, const float *nB, int64_t nbM, int64_t nbK,
                       int64_t nbN, int32_t tile) {
    if (!c || !nA || !nB || !tile_ok(tile)) return SPAMM_EINVAL;
    if (nbM <= 0 || nbK <= 0 || nbN <= 0 || nbM > 65535 || nbK > 65535 || nbN > 65535)
        return SPAMM_EINVAL;
    int rc = set_device(c);
    if (rc) return rc;
    leave_static(c);
    reset_shape(c, tile);
    c->M = nbM * tile;
    c->K = nbK * tile;
    c->N = nbN * tile;
    if ((rc = ensure(c, c->nA, (size_t)nbM * nbK * 4))) return rc;
    if ((rc = ensure(c, c->nB, (size_t)nbK * nbN * 4))) return rc;
    if ((rc = ensure(c, c->nBt, (size_t)nbK * nbN * 4))) return rc;
    HIPCHK(c, hipMemcpyAsync(c->nA.p, nA, (size_t)nbM * nbK * 4, hipMemcpyHostToDevice, c->stream));
    HIPCHK(c, hipMemcpyAsync(c->nB.p, nB, (size_t)nbK * nbN * 4, hipMemcpyHostToDevice, c->stream));
    HIPCHK(c, launch_transpose_normmap((const float *)c->nB.p, nbK, nbN, (float *)c->nBt.p, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    // norm maps only: the gate may run, the GEMM may not (no operands)
    c->have_a = c->have_b = false;
    c->nm_a = c->nm_b = true;
    c->have_gate = false;
    return SPAMM_OK;
}

int spamm_gate(spamm_ctx *c, float tau) {
    if (!c) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->tile || !c->M || !c->K || !c->N || !c->nm_a || !c->nm_b) return SPAMM_ESTATE;   // both norm maps, same K and tile
    if (tau != tau) return SPAMM_EINVAL;   // NaN
    int rc = set_device(c);
    if (rc) return rc;
    const Shape s = shape_of(c);
    if (gate_lds_bytes(c->tile, s.nbK) > gate_lds_limit()) return SPAMM_EINVAL;   // (defensive: the gate walks long K in chunks that fit)
    if (order_lds_bytes(c->tile, s.nbM, s.nbN) > order_lds_limit()) return SPAMM_EINVAL;   // more than 8192 super tiles of C
    const size_t nt = (size_t)s.nbM * s.nbN;
    if ((rc = ensure(c, c->counts, nt * 4))) return rc;
    if ((rc = ensure(c, c->mask, nt * s.words * 8))) return rc;
    if ((rc = ensure(c, c->macro_list, (size_t)s.n_macro * s.nbK * sizeof(MacroEntry)))) return rc;
    if ((rc = ensure(c, c->macro_count, (size_t)s.n_macro * 8))) return rc;
    if ((rc = ensure(c, c->macro_work, (size_t)s.n_macro * 4))) return rc;
    if ((rc = ensure(c, c->order, (size_t)sched_rounds(c->tile, s.nbM, s.nbN) * MAX_XCD * SUPER_M * SUPER_N * 4))) return rc;
    if ((rc = ensure(c, c->sched, SCHED_WORDS * 4))) return rc;
    if ((rc = ensure(c, c->kept_total, 16))) return rc;
    if (c->timing && !c->ev_a) HIPCHK(c, hipEventRecord(c->ev[2], c->stream));
    HIPCHK(c, launch_gate(gate_buffers(c), s.nbM, s.nbK, s.nbN, c->tile, tau, c->n_xcd, c->gate_chunk_cap, c->stream));
    if (c->timing) { HIPCHK(c, hipEventRecord(c->ev[3], c->stream)); c->ev_gate = true; }
    c->tau = tau;
    c->have_gate = true;
    return SPAMM_OK;
}

int spamm_gemm_gated(spamm_ctx *c, float *dC) {
    if (!c || !dC) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_a || !c->have_b || !c->have_gate) return SPAMM_ESTATE;
    if (c->a_pruned && !(c->tau >= c->a_pruned_tau)) return SPAMM_ESTATE;   // A's copy lacks tiles this tau keeps
    if (c->b_pruned && !(c->tau > 0.0f)) return SPAMM_ESTATE;               // B's copy lacks its zero tiles
    int rc = set_device(c);
    if (rc) return rc;
    if (c->timing && !c->ev_gate) HIPCHK(c, hipEventRecord(c->ev[3], c->stream));
    HIPCHK(c, launch_gemm(c->packedA.p, c->packedB.p, gate_buffers(c), c->M, c->K, c->N, c->tile, dC,
                          c->n_xcd, c->n_cu, c->gemm_ring, gemm_shape_for(c), c->stream));
    if (c->timing) { HIPCHK(c, hipEventRecord(c->ev[4], c->stream)); c->ev_gemm = true; }
    return SPAMM_OK;
}

static int multiply_any(spamm_ctx *c, const spamm_params *p, const void *dA, const void *dB, bool in16,
                        float *dC) {
    if (!c || !p || !dC) return SPAMM_EINVAL;
    const bool reuse_a = (p->flags & SPAMM_FLAG_REUSE_A) != 0, reuse_b = (p->flags & SPAMM_FLAG_REUSE_B) != 0;
    if ((!dA && !reuse_a) || (!dB && !reuse_b)) return SPAMM_EINVAL;
    if (!tile_ok(p->tile)) return SPAMM_EINVAL;
    if (p->M <= 0 || p->K <= 0 || p->N <= 0) return SPAMM_EINVAL;
    if (p->M % p->tile || p->K % p->tile || p->N % p->tile) return SPAMM_EINVAL;
    if (p->tau != p->tau) return SPAMM_EINVAL;
    leave_static(c);
    c->timing = (p->flags & SPAMM_FLAG_TIMING) != 0;
    c->ev_a = c->ev_b = c->ev_gate = c->ev_gemm = false;
    int rc;
    // same order as the reference: B's norm map first, then A's (cuSpAMM.cu:478-503)
    // an operand flagged for reuse must be resident with the same shape and tile
    if (reuse_a && !(c->have_a && c->tile == p->tile && c->M == p->M && c->K == p->K)) return SPAMM_ESTATE;
    // a copy of A written by a tau-aware pass serves the same B and thresholds not below that tau only
    if (reuse_a && c->a_pruned && !(reuse_b && p->tau >= c->a_pruned_tau)) return SPAMM_ESTATE;
    if (reuse_b && c->b_pruned && !(p->tau > 0.0f)) return SPAMM_ESTATE;
    if (reuse_b && !(c->have_b && c->tile == p->tile && c->K == p->K && c->N == p->N)) return SPAMM_ESTATE;
    bool a_eq_b = (p->flags & SPAMM_FLAG_A_EQ_B) != 0;
    if (a_eq_b && (reuse_a || reuse_b || dA != dB || p->M != p->K || p->K != p->N)) return SPAMM_EINVAL;
    // tile 128: the single pass for both roles needs every register of a SIMD for one wave and is slower
    // than the two passes (1.44 against 1.34 ms per multiply at N = 16384): the flag then only asserts
    // dA == dB, and the two ordinary passes (with their full tau-aware pruning) run
    if (a_eq_b && p->tile == 128) a_eq_b = false;
    if (a_eq_b) {
        // one read of the matrix feeds both operand roles (the reference's A = B runs convert and
        // norm the same data twice)
        if (reuse_a || reuse_b || dA != dB || p->M != p->K || p->K != p->N) return SPAMM_EINVAL;
        if (c->tile != p->tile) reset_shape(c, p->tile);
        const int64_t n = p->M;
        if (n / p->tile > 65535) return SPAMM_EINVAL;
        if ((rc = set_device(c))) return rc;
        const size_t nt = (size_t)(n / p->tile) * (size_t)(n / p->tile);
        // nothing of the old contents is valid until the pass has been launched
        c->have_a = c->have_b = c->have_gate = false;
        c->nm_a = c->nm_b = false;
        c->a_pruned = c->b_pruned = false;
        if ((rc = ensure(c, c->packedA, (size_t)n * n * 2))) return rc;
        if ((rc = ensure(c, c->packedB, (size_t)n * n * 2))) return rc;
        if ((rc = ensure(c, c->nA, nt * 4))) return rc;
        if ((rc = ensure(c, c->nB, nt * 4))) return rc;
        if ((rc = ensure(c, c->nBt, nt * 4))) return rc;
        c->M = c->K = c->N = n;
        if (c->timing) HIPCHK(c, hipEventRecord(c->ev[0], c->stream));
        const bool prune = (p->flags & SPAMM_FLAG_PRUNE) != 0 && p->tau > 0.0f;
        HIPCHK(c, launch_normmap_ab(dA, in16, n, p->tile, c->packedA.p, (float *)c->nA.p, c->packedB.p,
                                    (float *)c->nB.p, (float *)c->nBt.p, prune ? p->tau : 0.0f, c->stream));
        if (c->timing) {
            HIPCHK(c, hipEventRecord(c->ev[1], c->stream));
            HIPCHK(c, hipEventRecord(c->ev[2], c->stream));
            c->ev_a = c->ev_b = true;
        }
        c->have_a = c->have_b = true;
        c->nm_a = c->nm_b = true;
        c->a_pruned = c->b_pruned = prune;       // both copies lack their tiles of norm zero:
        c->a_pruned_tau = 1.0e-45f;              // they serve any tau > 0 (smallest positive float)
        c->have_gate = false;
    } else if (!reuse_b) {
        const bool prune = (p->flags & SPAMM_FLAG_PRUNE) != 0;
        if ((rc = normmap_any(c, SPAMM_ROLE_B, dB, in16, p->K, p->N, p->tile, prune ? &p->tau : nullptr))) return rc;
    } else if (c->timing) {
        HIPCHK(c, hipEventRecord(c->ev[0], c->stream));
        HIPCHK(c, hipEventRecord(c->ev[1], c->stream));
        c->ev_b = true;
    }
    if (a_eq_b) {
        // done above
    } else if (!reuse_a) {
        const bool prune = (p->flags & SPAMM_FLAG_PRUNE) != 0;
        if ((rc = normmap_any(c, SPAMM_ROLE_A, dA, in16, p->M, p->K, p->tile, prune ? &p->tau : nullptr))) return rc;
    } else if (c->timing) {
        HIPCHK(c, hipEventRecord(c->ev[2], c->stream));
        c->ev_a = true;
    }
    if ((rc = spamm_gate(c, p->tau))) return rc;
    if ((rc = spamm_gemm_gated(c, dC))) return rc;
    return SPAMM_OK;
}

// Gives every buffer a multiply of this shape needs its place in the fixed array (base != null) and
// returns the bytes used; with base == null only the size is computed.  Same sizes as the ensure()
// calls of the stages.
static size_t carve_static(Workspace &w, const spamm_params *p, unsigned char *base) {
    const size_t t = (size_t)p->tile;
    const size_t M = (size_t)p->M, K = (size_t)p->K, N = (size_t)p->N;
    const size_t nbM = M / t, nbK = K / t, nbN = N / t, nt = nbM * nbN, words = (nbK + 63) / 64;
    const size_t MT = (size_t)macro_dim(p->tile);
    const size_t n_macro = ((nbM + MT - 1) / MT) * ((nbN + MT - 1) / MT);
    size_t off = 0;
    auto take = [&](DevBuf &b, size_t bytes) {
        if (bytes == 0) bytes = 16;
        if (base) {
            if (b.p && !b.borrowed) (void)hipFree(b.p);    // not reached: the static workspace owns nothing here
            b.p = base + off;
            b.cap = bytes;
            b.borrowed = true;
        }
        off += (bytes + 255) & ~(size_t)255;
    };
    take(w.packedA, M * K * 2);
    take(w.packedB, K * N * 2);
    take(w.nA, nbM * nbK * 4);
    take(w.nB, nbK * nbN * 4);
    take(w.nBt, nbK * nbN * 4);
    take(w.rowmaxB, nbK * 4);
    take(w.counts, nt * 4);
    take(w.mask, nt * words * 8);
    take(w.macro_list, n_macro * nbK * sizeof(MacroEntry));
    take(w.macro_count, n_macro * 8);
    take(w.macro_work, n_macro * 4);
    take(w.order, (size_t)sched_rounds(p->tile, (int64_t)nbM, (int64_t)nbN) * MAX_XCD * SUPER_M * SUPER_N * 4);
    take(w.sched, SCHED_WORDS * 4);
    take(w.kept_total, 16);
    return off;
}

int spamm_multiply_noalloc(spamm_ctx *c, const spamm_params *p, const float *dA, const float *dB, float *dC) {
    if (!c || !p || !dA || !dB || !dC) return SPAMM_EINVAL;
    if (p->flags & (SPAMM_FLAG_REUSE_A | SPAMM_FLAG_REUSE_B)) return SPAMM_EINVAL;   // the array is shared: nothing persists
    if (!tile_ok(p->tile)) return SPAMM_EINVAL;
    if (p->M <= 0 || p->K <= 0 || p->N <= 0) return SPAMM_EINVAL;
    if (p->M % p->tile || p->K % p->tile || p->N % p->tile) return SPAMM_EINVAL;
    if (p->M / p->tile > 65535 || p->K / p->tile > 65535 || p->N / p->tile > 65535) return SPAMM_ELIMIT;
    if (p->tau != p->tau) return SPAMM_EINVAL;
    if (!c->static_ptr) return SPAMM_ESTATE;
    if (carve_static(*c, p, nullptr) > (size_t)SPAMM_NOALLOC_WORKSPACE_BYTES) return SPAMM_ELIMIT;
    if (!c->in_static) {
        std::swap(static_cast<Workspace &>(*c), c->parked);
        c->in_static = true;
    }
    reset_shape(c, p->tile);           // the carve-outs move with the shape, and other contexts share the array
    c->static_gen = g_static_gen[c->device].fetch_add(1, std::memory_order_acq_rel) + 1;
    (void)carve_static(*c, p, c->static_ptr);
    c->no_alloc = true;
    const int rc = multiply_any(c, p, dA, dB, false, dC);
    c->no_alloc = false;
    return rc;
}

int spamm_multiply(spamm_ctx *c, const spamm_params *p, const float *dA, const float *dB, float *dC) {
    return multiply_any(c, p, dA, dB, false, dC);
}

int spamm_multiply_f16(spamm_ctx *c, const spamm_params *p, const void *dAh, const void *dBh, float *dC) {
    return multiply_any(c, p, dAh, dBh, true, dC);
}

int spamm_error_vs_dense_f64(spamm_ctx *c, const float *dC, int64_t row0, int64_t row1, double *out3) {
    if (!c || !dC || !out3) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_a || !c->have_b || c->a_pruned || c->b_pruned) return SPAMM_ESTATE;   // needs complete fp16 copies
    if (row0 < 0 || row1 > c->M || row0 >= row1 || row0 % 64 || row1 % 64 || c->N % 64 || c->K % 16)
        return SPAMM_EINVAL;
    int rc = set_device(c);
    if (rc) return rc;
    if ((rc = ensure(c, c->tauws, tau_workspace_bytes()))) return rc;
    double *d = (double *)c->tauws.p;
    HIPCHK(c, launch_error_vs_dense(c->packedA.p, c->packedB.p, c->M, c->K, c->N, c->tile, dC, row0, row1, d,
                                    c->stream));
    double sq[3];
    if ((rc = copy_out(c, d, sq, sizeof(sq)))) return rc;
    for (int i = 0; i < 3; i++) out3[i] = sqrt(sq[i]);
    return SPAMM_OK;
}

int spamm_dropped_bound(spamm_ctx *c, float tau, double *out) {
    if (!c || !out || tau != tau) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    Shape s;
    if (!c->tile || !c->M || !c->K || !c->N || !c->nm_a || !c->nm_b) return SPAMM_ESTATE;   // both norm maps, same K and tile
    int rc = set_device(c);
    if (rc) return rc;
    s = shape_of(c);
    if ((rc = ensure(c, c->tauws, tau_workspace_bytes()))) return rc;
    double *d = (double *)c->tauws.p;
    HIPCHK(c, launch_dropped_bound((const float *)c->nA.p, (const float *)c->nBt.p, s.nbM, s.nbK, s.nbN, tau, d,
                                   nullptr, c->stream));
    double sq;
    if ((rc = copy_out(c, d, &sq, sizeof(sq)))) return rc;
    *out = sqrt(sq);
    return SPAMM_OK;
}

int spamm_dropped_bound_tiles(spamm_ctx *c, float tau, double *host_out) {
    if (!c || !host_out || tau != tau) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->tile || !c->M || !c->K || !c->N || !c->nm_a || !c->nm_b) return SPAMM_ESTATE;   // both norm maps, same K and tile
    int rc = set_device(c);
    if (rc) return rc;
    const Shape s = shape_of(c);
    const size_t nt = (size_t)s.nbM * s.nbN;
    if ((rc = ensure(c, c->tauws, tau_workspace_bytes()))) return rc;
    if ((rc = ensure(c, c->staging, nt * 8))) return rc;
    HIPCHK(c, launch_dropped_bound((const float *)c->nA.p, (const float *)c->nBt.p, s.nbM, s.nbK, s.nbN, tau,
                                   (double *)c->tauws.p, (double *)c->staging.p, c->stream));
    return copy_out(c, c->staging.p, host_out, nt * 8);
}

// ---- input adapters (host side; getMatrixFromCSV / getMatrixFromMTX, tool.cu:282-366)
static int load_text(const char *path, std::vector<char> &buf) {
    FILE *f = fopen(path, "rb");
    if (!f) return SPAMM_EINVAL;
    fseek(f, 0, SEEK_END);
    long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    if (n < 0) { fclose(f); return SPAMM_EINVAL; }
    buf.resize((size_t)n + 1);
    size_t got = fread(buf.data(), 1, (size_t)n, f);
    fclose(f);
    buf[got] = 0;
    return SPAMM_OK;
}

int spamm_load_csv_f32(const char *path, int64_t rows, int64_t cols, int64_t ld, float *host_out) {
    if (!path || !host_out || rows <= 0 || cols <= 0 || ld < cols) return SPAMM_EINVAL;
    std::vector<char> buf;
    int rc = load_text(path, buf);
    if (rc) return rc;
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < ld; j++) host_out[i * ld + j] = 0.0f;
    char *p = buf.data();
    for (int64_t i = 0; i < rows && *p; i++) {            // one line per matrix row, at most `rows` lines
        char *eol = strchr(p, '\n');
        if (eol) *eol = 0;
        int64_t j = 0;
        char *q = p;
        while (*q && j < cols) {
            char *end;
            float x = strtof(q, &end);
            if (end == q) x = 0.0f;                       // empty / unparsable field reads as 0
            host_out[i * ld + j++] = x;
            char *comma = strchr(q, ',');
            if (!comma) break;
            q = comma + 1;
        }
        if (!eol) break;
        p = eol + 1;
    }
    return SPAMM_OK;
}

int spamm_load_mtx_f32(const char *path, int64_t rows, int64_t cols, int64_t ld, float *host_out) {
    if (!path || !host_out || rows <= 0 || cols <= 0 || ld < cols) return SPAMM_EINVAL;
    std::vector<char> buf;
    int rc = load_text(path, buf);
    if (rc) return rc;
    for (int64_t i = 0; i < rows; i++)
        for (int64_t j = 0; j < ld; j++) host_out[i * ld + j] = 0.0f;
    char *p = buf.data();
    bool first = true;
    while (*p) {
        char *eol = strchr(p, '\n');
        if (eol) *eol = 0;
        if (first) {
            first = false;                                // the first line (header / sizes) is skipped
        } else {
            long long r, cidx;
            double v;
            if (sscanf(p, "%lld %lld %lf", &r, &cidx, &v) == 3) {   // 1-based "row col val"
                if (r < 1 || r > rows || cidx < 1 || cidx > cols) return SPAMM_EINVAL;
                host_out[(r - 1) * ld + (cidx - 1)] = (float)v;
            }
        }
        if (!eol) break;
        p = eol + 1;
    }
    return SPAMM_OK;
}

static int tau_prepare(spamm_ctx *c, Shape *s) {
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->tile || !c->M || !c->K || !c->N || !c->nm_a || !c->nm_b) return SPAMM_ESTATE;   // both norm maps, same K and tile
    int rc = set_device(c);
    if (rc) return rc;
    *s = shape_of(c);
    return ensure(c, c->tauws, tau_workspace_bytes());
}

static int tau_count(spamm_ctx *c, const Shape &s, double thr, TauCounts *out) {
    HIPCHK(c, launch_tau_count((const float *)c->nA.p, (const float *)c->nBt.p, s.nbM, s.nbK, s.nbN, thr,
                               c->tauws.p, c->stream));
    return copy_out(c, (char *)c->tauws.p + tau_counts_offset(), out, sizeof(*out));
}

int spamm_count_kept(spamm_ctx *c, double threshold, int64_t *count_out, double *sum_out) {
    if (!c || threshold != threshold) return SPAMM_EINVAL;
    Shape s;
    int rc = tau_prepare(c, &s);
    if (rc) return rc;
    TauCounts tc;
    if ((rc = tau_count(c, s, threshold, &tc))) return rc;
    if (count_out) *count_out = (int64_t)tc.count;
    if (sum_out) *sum_out = tc.sum;
    return SPAMM_OK;
}

int spamm_tau_for_ratio(spamm_ctx *c, double ratio, float *tau_out, double *achieved_out) {
    if (!c || !tau_out || !(ratio >= 0.0) || ratio > 1.0) return SPAMM_EINVAL;
    Shape s;
    int rc = tau_prepare(c, &s);
    if (rc) return rc;
    const unsigned long long total = (unsigned long long)s.nbM * s.nbK * s.nbN;
    TauCounts tc;
    if ((rc = tau_count(c, s, 0.0, &tc))) return rc;
    double w = ceil(ratio * (double)total);
    unsigned long long want = w < 1.0 ? 1ull : (unsigned long long)w;
    if (want > total) want = total;
    if (tc.positive == 0) {                 // nothing but zeros: only tau = 0 keeps anything
        *tau_out = 0.0f;
        if (achieved_out) *achieved_out = 1.0;
        return SPAMM_OK;
    }
    if (want > tc.positive) want = tc.positive;     // zero tail: settle for the smallest positive product
    HIPCHK(c, launch_tau_select((const float *)c->nA.p, (const float *)c->nBt.p, s.nbM, s.nbK, s.nbN, want,
                                c->tauws.p, c->stream));
    TauState st;
    if ((rc = copy_out(c, c->tauws.p, &st, sizeof(st)))) return rc;
    memcpy(tau_out, &st.tau_bits, 4);
    if (achieved_out) *achieved_out = (double)st.kept / (double)total;
    return SPAMM_OK;
}

int spamm_tune_bisect(spamm_ctx *c, double expected, double tol, int max_rounds, float *tau_out,
                      double *achieved_out) {
    if (!c || !tau_out || max_rounds < 1 || !(tol > 0.0)) return SPAMM_EINVAL;
    Shape s;
    int rc = tau_prepare(c, &s);
    if (rc) return rc;
    const long long total = (long long)(s.nbM * s.nbK * s.nbN);
    double Norm = 0, up = 0, down = 0, rate = 0;
    for (int Ti = 0; Ti < max_rounds; Ti++) {       // tool.cu:445-486
        TauCounts tc;
        if ((rc = tau_count(c, s, Norm, &tc))) return rc;
        rate = (double)((float)tc.count / (float)total);
        if (fabs(rate - expected) < tol) break;
        if (Ti == 0) {
            Norm = tc.sum / (double)total;
            up = Norm;
            continue;
        }
        if (rate > expected) {
            if (up == Norm) up *= 2;
            down = Norm;
            Norm = (Norm + up) / 2;
        } else {
            up = Norm;
            Norm = (Norm + down) / 2;
        }
    }
    *tau_out = (float)Norm;
    if (achieved_out) *achieved_out = rate;
    return SPAMM_OK;
}

int spamm_get_stats(spamm_ctx *c, spamm_stats *out) {
    if (!c || !out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    memset(out, 0, sizeof(*out));
    if (!c->have_gate) return SPAMM_ESTATE;
    int rc = set_device(c);
    if (rc) return rc;
    const Shape s = shape_of(c);
    out->total_products = s.nbM * s.nbK * s.nbN;
    int64_t kept = 0;
    if ((rc = copy_out(c, c->kept_total.p, &kept, 8))) return rc;
    out->kept_products = kept;
    if (c->timing && c->ev_a && c->ev_b && c->ev_gate && c->ev_gemm) {
        HIPCHK(c, hipEventElapsedTime(&out->ms_normmap_b, c->ev[0], c->ev[1]));
        HIPCHK(c, hipEventElapsedTime(&out->ms_normmap_a, c->ev[1], c->ev[2]));
        HIPCHK(c, hipEventElapsedTime(&out->ms_gate, c->ev[2], c->ev[3]));
        HIPCHK(c, hipEventElapsedTime(&out->ms_gemm, c->ev[3], c->ev[4]));
        HIPCHK(c, hipEventElapsedTime(&out->ms_total, c->ev[0], c->ev[4]));
        out->timing_valid = 1;
    }
    return SPAMM_OK;
}

int spamm_get_normmap(spamm_ctx *c, int role, float *host_out) {
    if (!c || !host_out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->tile) return SPAMM_ESTATE;
    const Shape s = shape_of(c);
    if (role == SPAMM_ROLE_A) {
        if (!c->nm_a) return SPAMM_ESTATE;
        return copy_out(c, c->nA.p, host_out, (size_t)s.nbM * s.nbK * 4);
    }
    if (role == SPAMM_ROLE_B) {
        if (!c->nm_b) return SPAMM_ESTATE;
        return copy_out(c, c->nB.p, host_out, (size_t)s.nbK * s.nbN * 4);
    }
    return SPAMM_EINVAL;
}

int spamm_get_counts(spamm_ctx *c, int32_t *host_out) {
    if (!c || !host_out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_gate) return SPAMM_ESTATE;
    const Shape s = shape_of(c);
    return copy_out(c, c->counts.p, host_out, (size_t)s.nbM * s.nbN * 4);
}

int spamm_get_klist(spamm_ctx *c, uint16_t *host_out) {
    if (!c || !host_out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_gate) return SPAMM_ESTATE;
    const Shape s = shape_of(c);
    // built from the bitmaps on demand: the multiply itself never reads per-tile lists
    int rc = set_device(c);
    if (rc) return rc;
    const size_t bytes = (size_t)s.nbM * s.nbN * s.nbK * 2;
    if ((rc = ensure(c, c->klist, bytes))) return rc;
    HIPCHK(c, launch_klist((const uint64_t *)c->mask.p, (uint16_t *)c->klist.p, s.nbM * s.nbN, s.nbK, c->stream));
    return copy_out(c, c->klist.p, host_out, bytes);
}

int spamm_get_mask(spamm_ctx *c, uint64_t *host_out) {
    if (!c || !host_out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_gate) return SPAMM_ESTATE;
    const Shape s = shape_of(c);
    return copy_out(c, c->mask.p, host_out, (size_t)s.nbM * s.nbN * s.words * 8);
}

int spamm_get_macro_counts(spamm_ctx *c, int32_t *host_counts, int32_t *host_sched) {
    if (!c || !host_counts) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    if (!c->have_gate) return SPAMM_ESTATE;
    const Shape s = shape_of(c);
    int rc = copy_out(c, c->macro_count.p, host_counts, (size_t)s.n_macro * 8);
    if (rc == SPAMM_OK && host_sched) rc = copy_out(c, c->sched.p, host_sched, 2 * MAX_XCD * 4);
    return rc;
}

int spamm_get_fp16(spamm_ctx *c, int role, uint16_t *host_out) {
    if (!c || !host_out) return SPAMM_EINVAL;
    if (static_stale(c)) return SPAMM_ESTATE;
    int rc = set_device(c);
    if (rc) return rc;
    int64_t rows, cols;
    const void *packed;
    if (role == SPAMM_ROLE_A) {
        if (!c->have_a || c->a_pruned) return SPAMM_ESTATE;
        rows = c->M; cols = c->K; packed = c->packedA.p;
    } else if (role == SPAMM_ROLE_B) {
        if (!c->have_b || c->b_pruned) return SPAMM_ESTATE;
        rows = c->K; cols = c->N; packed = c->packedB.p;
    } else {
        return SPAMM_EINVAL;
    }
    const size_t bytes = (size_t)rows * cols * 2;
    if ((rc = ensure(c, c->staging, bytes))) return rc;
    HIPCHK(c, launch_unpack(packed, rows, cols, c->tile, role, (uint16_t *)c->staging.p, c->stream));
    return copy_out(c, c->staging.p, host_out, bytes);
}

int spamm_fill_decay_f32(spamm_ctx *c, float *dX, int64_t rows, int64_t cols,
                         const float *host_table, uint64_t seed, int random) {
    if (!c || !dX || !host_table || rows <= 0 || cols <= 0 || cols % 4) return SPAMM_EINVAL;
    int rc = set_device(c);
    if (rc) return rc;
    const int64_t n = rows > cols ? rows : cols;
    if ((rc = ensure(c, c->staging, (size_t)n * 4))) return rc;
    HIPCHK(c, hipMemcpyAsync(c->staging.p, host_table, (size_t)n * 4, hipMemcpyHostToDevice, c->stream));
    HIPCHK(c, launch_fill_decay(dX, rows, cols, (const float *)c->staging.p, seed, random, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return SPAMM_OK;
}

}  // extern "C"
