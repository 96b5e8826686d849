"""spamm_multiply_noalloc: the multiply in the library's fixed device workspace, for callers that
cannot allocate (graph capture, serving loops).  Checked through the C ABI against spamm_multiply
and against the host checker: kept mask, counts and norm maps bit-exact, C within 1e-3 relative
Frobenius error (the same kernels run, so C is in fact identical); two calls in a row, the second
with a smaller problem."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

C_TOL = 1e-3          # relative Frobenius error allowed for C


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _case(orc, M, K, N, lam, seeds):
    tab = orc.decay_table("exp", max(M, K, N), lam)
    return orc.fill_decay(M, K, tab, seeds[0]), orc.fill_decay(K, N, tab, seeds[1])


def _check_against(ctx, orc, C, ref, what):
    assert np.array_equal(ctx.get_mask(), ref["mask"]), what + ": kept mask"
    assert np.array_equal(ctx.get_counts(), ref["counts"]), what + ": counts"
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), ref["nA"].view(np.uint32)), what + ": norm map A"
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), ref["nB"].view(np.uint32)), what + ": norm map B"
    assert ctx.get_stats().kept_products == ref["kept"], what + ": kept products"
    err, nrm, _ = orc.frob_diff(C.cpu().numpy(), ref["C"])
    assert err <= C_TOL * nrm, "%s: C off by %g" % (what, err / nrm)


def test_noalloc_equals_multiply_two_calls_second_smaller(orc, ctx):
    import torch
    cases = [((768, 512, 1024), 64, 0.4, 0.02, False), ((256, 384, 128), 32, 0.05, 0.03, True)]
    ctx.multiply(*map(_dev, _case(orc, 256, 256, 256, 0.02, (5, 6))), 64, 0.1)    # kernels loaded, own workspace in use
    ctx.multiply(*map(_dev, _case(orc, 256, 256, 256, 0.02, (5, 6))), 32, 0.1, prune=True)
    for (M, K, N), tile, tau, lam, prune in cases:
        A, B = _case(orc, M, K, N, lam, (1, 2))
        dA, dB = _dev(A), _dev(B)
        ref = orc.spamm(A, B, tile, tau)
        assert 0 < ref["kept"] < (M // tile) * (K // tile) * (N // tile)
        want = ctx.multiply(dA, dB, tile, tau, prune=prune).clone()
        want_mask = ctx.get_mask()
        got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        ctx.multiply_noalloc(dA, dB, tile, tau, got, prune=prune)
        ctx.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed inside the call"
        assert np.array_equal(ctx.get_mask(), want_mask)
        assert torch.equal(got, want)
        _check_against(ctx, orc, got, ref, "noalloc %dx%dx%d tile %d" % (M, K, N, tile))


def test_noalloc_leaves_the_contexts_own_workspace_alone(orc, ctx):
    import torch
    A1, B = _case(orc, 512, 512, 512, 0.01, (1, 2))
    A2, B2 = _case(orc, 256, 256, 256, 0.01, (3, 4))
    dA1, dB = _dev(A1), _dev(B)
    ref = ctx.multiply(dA1, dB, 64, 0.5).clone()
    got2 = torch.empty((256, 256), dtype=torch.float32, device="cuda")
    ctx.multiply_noalloc(_dev(A2), _dev(B2), 64, 0.5, got2)          # runs in the fixed array
    r2 = orc.spamm(A2, B2, 64, 0.5)
    _check_against(ctx, orc, got2, r2, "noalloc 256")
    again = ctx.multiply(dA1, dB, 64, 0.5, reuse_a=True, reuse_b=True)   # own fp16 copies and norm maps still valid
    assert torch.equal(again, ref)
    assert np.array_equal(ctx.get_mask(), orc.spamm(A1, B, 64, 0.5)["mask"])


def test_noalloc_results_go_stale_when_another_context_uses_the_array(orc, ctx):
    """All contexts on a GPU share the one fixed array: after another context's noalloc call this
    context's read-backs and stage calls must refuse (SPAMM_ESTATE) instead of handing out the other
    call's bytes; an ordinary multiply brings the context back to its own workspace."""
    import torch
    import cuspamm_amd as sp
    A, B = _case(orc, 256, 256, 256, 0.02, (1, 2))
    A2, B2 = _case(orc, 384, 128, 256, 0.02, (3, 4))
    dA, dB = _dev(A), _dev(B)
    got = torch.empty((256, 256), dtype=torch.float32, device="cuda")
    other = sp.SpammContext(0)
    try:
        ctx.multiply_noalloc(dA, dB, 64, 0.1, got)
        ref = orc.spamm(A, B, 64, 0.1)
        _check_against(ctx, orc, got, ref, "first context")
        got2 = torch.empty((384, 256), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        other.multiply_noalloc(_dev(A2), _dev(B2), 64, 0.1, got2)
        _check_against(other, orc, got2, orc.spamm(A2, B2, 64, 0.1), "second context")
        for call in (ctx.get_mask, ctx.get_counts, ctx.get_stats, lambda: ctx.get_normmap(0), lambda: ctx.gate(0.1),
                     lambda: ctx.gemm_gated(got), lambda: ctx.dropped_bound(0.1), lambda: ctx.tau_for_ratio(0.5)):
            with pytest.raises(sp.SpammError) as ei:
                call()
            assert ei.value.code == sp.api.ESTATE
        # the other context's results are still its own
        assert np.array_equal(other.get_mask(), orc.spamm(A2, B2, 64, 0.1)["mask"])
        # an ordinary call returns to the own workspace; a new noalloc call makes the results current again
        C = ctx.multiply(dA, dB, 64, 0.1)
        assert torch.equal(C, got) and np.array_equal(ctx.get_mask(), ref["mask"])
        ctx.multiply_noalloc(dA, dB, 64, 0.1, got)
        assert np.array_equal(ctx.get_mask(), ref["mask"])
        with pytest.raises(sp.SpammError):
            other.get_mask()
    finally:
        other.close()


def test_noalloc_a_equals_b(orc, ctx):
    import torch
    n = 512
    A = orc.fill_decay(n, n, orc.decay_table("exp", n, 0.02), 7)
    dA = _dev(A)
    got = torch.empty((n, n), dtype=torch.float32, device="cuda")
    ctx.multiply_noalloc(dA, dA, 32, 1e-2, got, a_eq_b=True)
    _check_against(ctx, orc, got, orc.spamm(A, A, 32, 1e-2), "noalloc A = B")


def test_noalloc_at_the_workspace_limit(orc, ctx):
    # 3072^3 needs 36 MiB of fp16 copies plus lists: the largest cube that fits the 40 MiB array
    import torch
    n = 3072
    tab = orc.decay_table("exp", n, 0.004)
    dA = torch.empty((n, n), dtype=torch.float32, device="cuda")
    dB = torch.empty((n, n), dtype=torch.float32, device="cuda")
    ctx.fill_decay(dA, tab, 1)
    ctx.fill_decay(dB, tab, 2)
    for tile in (32, 128):
        ctx.normmap_f32(1, dB, tile)
        ctx.normmap_f32(0, dA, tile)
        tau, ach = ctx.tau_for_ratio(0.15)
        want = ctx.multiply(dA, dB, tile, tau, prune=True).clone()
        want_mask, want_counts = ctx.get_mask(), ctx.get_counts()
        got = torch.full((n, n), float("nan"), dtype=torch.float32, device="cuda")
        ctx.multiply_noalloc(dA, dB, tile, tau, got, prune=True)
        assert np.array_equal(ctx.get_mask(), want_mask) and np.array_equal(ctx.get_counts(), want_counts)
        assert torch.equal(got, want)
        assert abs(ctx.get_stats().kept_products / (n // tile) ** 3 - ach) < 1e-9


def test_noalloc_limits_and_flags(ctx):
    import ctypes
    import torch
    import cuspamm_amd as sp
    x = torch.zeros((64, 64), dtype=torch.float32, device="cuda")
    ptr = x.data_ptr()
    L = sp.load_library()

    def call(M, K, N, tile, flags=0, tau=0.0):
        p = sp.SpammParams(M, K, N, tile, tau, flags, 0)
        return L.spamm_multiply_noalloc(ctx._h, ctypes.byref(p), ctypes.c_void_p(ptr), ctypes.c_void_p(ptr),
                                        ctypes.c_void_p(ptr))
    # refused before any kernel runs (the pointers are never dereferenced)
    assert call(4096, 4096, 4096, 64) == sp.api.ELIMIT            # 64 MiB of fp16 copies > 40 MiB
    assert call(64 * 70000, 64, 64, 64) == sp.api.ELIMIT
    assert call(64, 64, 64, 64, sp.FLAG_REUSE_A) == sp.api.EINVAL
    assert call(64, 64, 64, 64, sp.FLAG_REUSE_B) == sp.api.EINVAL
    assert call(64, 60, 64, 64) == sp.api.EINVAL
    assert call(64, 64, 64, 48) == sp.api.EINVAL
    assert call(64, 64, 64, 64, 0, float("nan")) == sp.api.EINVAL
    assert "fixed workspace" in L.spamm_strerror(sp.api.ELIMIT).decode()
    assert call(64, 64, 64, 64) == 0                               # x * x with tau 0: zeros
    ctx.synchronize()
    assert float(x.abs().max()) == 0.0


# The callers this entry point is for: a HIP graph captures the multiply once and replays it on
# changing inputs (mask and schedule are rebuilt on the device at every replay); eager multiplies
# run between the replays and every replay is compared with one.
def test_noalloc_multiply_replays_in_a_hip_graph(orc, ctx):
    import torch
    import cuspamm_amd as sp
    M, K, N, tile, tau = 1024, 768, 1280, 64, 0.3
    tab = orc.decay_table("exp", max(M, K, N), 0.01)
    A0, B0 = orc.fill_decay(M, K, tab, 1), orc.fill_decay(K, N, tab, 2)
    dA = torch.from_numpy(A0).cuda()
    dB = torch.from_numpy(B0).cuda()
    C = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        gctx = sp.SpammContext(0)                     # bound to the side stream
        gctx.multiply_noalloc(dA, dB, tile, tau, C)   # warm-up: kernels loaded before the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            gctx.multiply_noalloc(dA, dB, tile, tau, C, prune=True)
    torch.cuda.synchronize()
    for rep, scale in enumerate((1.0, 0.5, 3.0, 1.0)):
        dA.copy_(torch.from_numpy(A0).cuda() * scale)                 # new inputs in the captured buffers
        want = ctx.multiply(dA, dB, tile, tau).clone()                # eager work between the replays
        want_mask = ctx.get_mask()
        C.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, want), "replay %d" % rep
        ref = orc.spamm((A0 * np.float32(scale)).astype(np.float32), B0, tile, tau)
        assert np.array_equal(want_mask, ref["mask"])
        err, nrm, _ = orc.frob_diff(C.cpu().numpy(), ref["C"])
        assert err <= 1e-3 * nrm
    gctx.close()
