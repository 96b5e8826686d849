"""fp16-input entry point, operand reuse and the error-report tooling."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _vs_checker(orc, ctx, C, A32, B32, tile, tau, what):
    """The library's last multiply against the host checker run on the same fp32 values: kept mask,
    counts and norm maps bit-exact, C within 1e-3 relative Frobenius error."""
    ref = orc.spamm(np.ascontiguousarray(A32, dtype=np.float32), np.ascontiguousarray(B32, dtype=np.float32), tile, tau)
    assert np.array_equal(ctx.get_mask(), ref["mask"]), what
    assert np.array_equal(ctx.get_counts(), ref["counts"]), what
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), ref["nA"].view(np.uint32)), what
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), ref["nB"].view(np.uint32)), what
    assert ctx.get_stats().kept_products == ref["kept"], what
    err, nrm, _ = orc.frob_diff(C.cpu().numpy(), ref["C"])
    assert err <= 1e-3 * nrm, "%s: C off by %g" % (what, err / max(nrm, 1e-300))
    return ref


@pytest.mark.parametrize("tile", [32, 64, 128])
def test_fp16_inputs_equal_fp32_inputs_of_the_same_values(orc, ctx, tile):
    import torch
    M, K, N = 3 * 128, 2 * 128, 4 * 128
    tab = orc.decay_table("exp", max(M, K, N), 0.01)
    A = _dev(orc.fill_decay(M, K, tab, 1)).half()
    B = _dev(orc.fill_decay(K, N, tab, 2)).half()
    ctx.normmap_f16(1, B, tile)
    ctx.normmap_f16(0, A, tile)
    tau, ach = ctx.tau_for_ratio(0.5)
    assert 0.45 < ach < 0.6
    C16 = ctx.multiply(A, B, tile, tau).clone()
    # fp16 is the reference's real input type (para.h:1, cuSpAMM.cu:486): the checker, fed the same
    # values as fp32 (its fp16 rounding is then the identity), must agree
    _vs_checker(orc, ctx, C16, A.float().cpu().numpy(), B.float().cpu().numpy(), tile, tau, "fp16 inputs")
    m16, nA16, nB16 = ctx.get_mask(), ctx.get_normmap(0), ctx.get_normmap(1)
    assert np.array_equal(ctx.get_fp16(0), A.cpu().numpy().view(np.uint16))
    assert np.array_equal(ctx.get_fp16(1), B.cpu().numpy().view(np.uint16))
    C32 = ctx.multiply(A.float(), B.float(), tile, tau)
    assert np.array_equal(ctx.get_mask(), m16)
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), nA16.view(np.uint32))
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), nB16.view(np.uint32))
    assert torch.equal(C16, C32)
    Cp = ctx.multiply(A, B, tile, tau, prune=True)      # tau-aware passes on fp16 inputs
    assert torch.equal(C16, Cp)
    _vs_checker(orc, ctx, Cp, A.float().cpu().numpy(), B.float().cpu().numpy(), tile, tau, "fp16 inputs, tau-aware")
    kept = ctx.get_stats().kept_products
    assert 0 < kept < (M // tile) * (K // tile) * (N // tile)


def test_operand_reuse(orc, ctx):
    import torch
    import cuspamm_amd as sp
    n = 512
    tab = orc.decay_table("exp", n, 0.01)
    A1, A2, B = (_dev(orc.fill_decay(n, n, tab, s)) for s in (1, 3, 2))
    ref1 = ctx.multiply(A1, B, 64, 0.5).clone()
    ref2 = ctx.multiply(A2, B, 64, 0.5).clone()
    ctx.multiply(A1, B, 64, 0.5)
    hA1, hA2, hB = A1.cpu().numpy(), A2.cpu().numpy(), B.cpu().numpy()
    got2 = ctx.multiply(A2, B, 64, 0.5, reuse_b=True)          # B's fp16 copy and norm map are kept
    assert torch.equal(got2, ref2)
    _vs_checker(orc, ctx, got2, hA2, hB, 64, 0.5, "new A against the resident B")
    got1 = ctx.multiply(A1, B, 64, 0.5, reuse_b=True)
    assert torch.equal(got1, ref1)
    _vs_checker(orc, ctx, got1, hA1, hB, 64, 0.5, "first A again against the resident B")
    got1 = ctx.multiply(A1, B, 64, 0.1, reuse_a=True, reuse_b=True)   # only tau changes
    _vs_checker(orc, ctx, got1, hA1, hB, 64, 0.1, "both operands resident, new tau")
    assert torch.equal(got1.clone(), ctx.multiply(A1, B, 64, 0.1))
    # a new B against the resident A (matrix powers: X, then X * B2)
    B2 = _dev(orc.fill_decay(n, n, tab, 9))
    ctx.multiply(A1, B, 64, 0.5)
    gotb = ctx.multiply(A1, B2, 64, 0.5, reuse_a=True)
    _vs_checker(orc, ctx, gotb, hA1, B2.cpu().numpy(), 64, 0.5, "new B against the resident A")
    with pytest.raises(sp.SpammError) as ei:                    # shape changed: nothing to reuse
        ctx.multiply(A1[:256].contiguous(), B, 64, 0.5, reuse_a=True)
    assert ei.value.code == -4


def test_error_report_matches_checker(orc, ctx):
    n, tile = 512, 64
    tab = orc.decay_table("exp", n, 0.01)
    A, B = orc.fill_decay(n, n, tab, 1), orc.fill_decay(n, n, tab, 2)
    for tau in (0.0, 0.5, 3.0):
        C = ctx.multiply(_dev(A), _dev(B), tile, tau)
        Af = orc.f16_bits_to_f32(ctx.get_fp16(0))
        Bf = orc.f16_bits_to_f32(ctx.get_fp16(1))
        dense = orc.gemm_dense_f64(Af, Bf)
        e, d, c = orc.frob_diff(C.cpu().numpy(), dense)
        ge, gd, gc = ctx.error_vs_dense(C)
        assert abs(gd - d) <= 1e-10 * d and abs(gc - c) <= 1e-10 * c
        assert abs(ge - e) <= 1e-6 * e + 1e-12 * d
        bound = orc.dropped_bound(ctx.get_normmap(0), ctx.get_normmap(1), tau)
        gb = ctx.dropped_bound(tau)
        assert abs(gb - bound) <= 1e-9 * max(bound, 1e-30)
        assert ge <= gb * (1 + 1e-4) + 1e-5 * gd
        # per output tile: the dropped sums themselves, against the checker's, and consistent with
        # the scalar (root of the sum of squares, whole matrix and a row range)
        gt = ctx.dropped_bound_tiles(tau)
        ot = orc.dropped_bound_tiles(ctx.get_normmap(0), ctx.get_normmap(1), tau)
        assert gt.shape == ot.shape == (n // tile, n // tile)
        assert np.all(np.abs(gt - ot) <= 1e-12 * np.maximum(ot, 1e-300)), np.abs(gt - ot).max()
        assert np.array_equal(gt == 0, ot == 0)
        assert abs(np.sqrt((gt ** 2).sum()) - gb) <= 1e-9 * max(gb, 1e-30)
        part = orc.dropped_bound(ctx.get_normmap(0), ctx.get_normmap(1), tau, 2, 5)
        assert abs(np.sqrt((gt[2:5] ** 2).sum()) - part) <= 1e-9 * max(part, 1e-30)
        # row range
        ge2, gd2, _ = ctx.error_vs_dense(C, 128, 256)
        e2, d2, _ = orc.frob_diff(C.cpu().numpy()[128:256], dense[128:256])
        assert abs(gd2 - d2) <= 1e-10 * d2 and abs(ge2 - e2) <= 1e-6 * e2 + 1e-12 * d2


@pytest.mark.parametrize("tile", [32, 64, 128])
def test_a_equals_b_single_pass(orc, ctx, tile):
    # BASELINE config 1 shape (A = B): one read of the matrix must give the same fp16 copies, norm
    # maps, mask and C as the two-pass run
    import torch
    import cuspamm_amd as sp
    n = 1024
    tab = orc.decay_table("exp", n, 0.5 if tile == 32 else 0.05)
    X = _dev(orc.fill_decay(n, n, tab, 1))
    tau = 1e-4 if tile == 32 else 2.0
    C2 = ctx.multiply(X, X, tile, tau).clone()
    ref = (ctx.get_mask(), ctx.get_normmap(0), ctx.get_normmap(1), ctx.get_fp16(0), ctx.get_fp16(1))
    C1 = ctx.multiply(X, X, tile, tau, a_eq_b=True)
    hX = X.cpu().numpy()
    chk = _vs_checker(orc, ctx, C1, hX, hX, tile, tau, "A = B single pass")
    assert np.array_equal(ctx.get_fp16(0), chk["hA"]) and np.array_equal(ctx.get_fp16(1), chk["hB"])
    got = (ctx.get_mask(), ctx.get_normmap(0), ctx.get_normmap(1), ctx.get_fp16(0), ctx.get_fp16(1))
    for r, g in zip(ref, got):
        assert np.array_equal(r.view(np.uint8), g.view(np.uint8))
    assert torch.equal(C1, C2)
    kept = ctx.get_stats().kept_products
    assert 0 < kept < (n // tile) ** 3
    with pytest.raises(sp.SpammError):                       # the flag needs the same pointer and a square problem
        ctx.multiply(X, X.clone(), tile, tau, a_eq_b=True)
    # the single pass with the tau-aware flag: tiles of norm zero are left out of both copies
    # (exp(-0.5 d) is exactly zero in fp16 beyond d = 33, exp(-0.05 d) beyond d = 333)
    assert np.count_nonzero(ref[1] == 0) > 0
    ctx.multiply(torch.full_like(X, 1000.0), X, tile, 0.0)   # loud workspace
    Cp = ctx.multiply(X, X, tile, tau, a_eq_b=True, prune=True)
    assert torch.equal(Cp, C2)
    assert np.array_equal(ctx.get_mask(), ref[0])
    _vs_checker(orc, ctx, Cp, hX, hX, tile, tau, "A = B single pass, tau-aware")
    with pytest.raises(sp.SpammError):
        ctx.get_fp16(0)
    with pytest.raises(sp.SpammError):
        ctx.get_fp16(1)
    assert torch.equal(ctx.multiply(X, X, tile, tau * 3, reuse_a=True, reuse_b=True), ctx.multiply(X, X, tile, tau * 3))


@pytest.mark.parametrize("tile", [32, 64, 128])
def test_tau_aware_passes_give_the_same_product(orc, ctx, tile):
    """SPAMM_FLAG_PRUNE: A tiles that no product can keep and B tiles of norm zero are not copied;
    C, mask, counts and norm maps must not change.  The workspace is first filled with loud
    operands so that a GEMM reading a skipped tile would show."""
    import torch
    import cuspamm_amd as sp
    M, K, N = 4 * 256, 3 * 256, 2 * 256 + tile
    tab = orc.decay_table("exp", max(M, K, N), 0.05)      # exactly zero in fp16 beyond |i - j| ~ 333
    A = _dev(orc.fill_decay(M, K, tab, 1))
    B = _dev(orc.fill_decay(K, N, tab, 2))
    ctx.normmap_f32(1, B, tile)
    ctx.normmap_f32(0, A, tile)
    tau, ach = ctx.tau_for_ratio(0.05)
    assert tau > 0 and 0.01 < ach < 0.2
    Cref = ctx.multiply(A, B, tile, tau).clone()
    mask, counts, nA, nB = ctx.get_mask(), ctx.get_counts(), ctx.get_normmap(0), ctx.get_normmap(1)
    kept = ctx.get_stats().kept_products
    # the checker's kept set says which A tiles are needed at all: some must be skippable here,
    # and some B tiles must be exactly zero
    needed = np.unpackbits(mask.view(np.uint8), axis=-1, bitorder="little")[..., :K // tile].any(axis=1)
    assert 0 < needed.sum() < needed.size
    assert 0 < np.count_nonzero(nB == 0) < nB.size
    loud = ctx.multiply(torch.full_like(A, 1000.0), torch.full_like(B, 1000.0), tile, 0.0)   # both workspace copies are now loud
    assert float(loud.min()) > 0
    C = ctx.multiply(A, B, tile, tau, prune=True)
    assert torch.equal(C, Cref)
    assert np.array_equal(ctx.get_mask(), mask) and np.array_equal(ctx.get_counts(), counts)
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), nA.view(np.uint32))
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), nB.view(np.uint32))
    assert ctx.get_stats().kept_products == kept
    # the incomplete copies are fenced off
    for call in (lambda: ctx.get_fp16(0), lambda: ctx.get_fp16(1), lambda: ctx.error_vs_dense(C),
                 lambda: ctx.multiply(A, B, tile, tau * 0.5, reuse_a=True, reuse_b=True),
                 lambda: ctx.multiply(A, B, tile, tau, reuse_a=True),
                 lambda: ctx.multiply(A, B, tile, 0.0, reuse_b=True)):
        with pytest.raises(sp.SpammError) as ei:
            call()
        assert ei.value.code == -4
    # ... but serve the same operands at the same or a larger threshold
    ctx.multiply(A, B, tile, tau, prune=True)
    C2 = ctx.multiply(A, B, tile, tau * 2, reuse_a=True, reuse_b=True).clone()
    C3 = ctx.multiply(A, B, tile, tau * 0.5, reuse_b=True).clone()        # B's copy serves any tau > 0
    assert torch.equal(C2, ctx.multiply(A, B, tile, tau * 2))
    assert torch.equal(C3, ctx.multiply(A, B, tile, tau * 0.5))
    # and a plain call makes them whole again
    assert np.array_equal(ctx.get_fp16(0), orc.f32_to_f16_bits(A.cpu().numpy()))
    assert np.array_equal(ctx.get_fp16(1), orc.f32_to_f16_bits(B.cpu().numpy()))
    # tau = 0 (nothing may be left out) and tau = inf through the flag
    assert torch.equal(ctx.multiply(A, B, tile, 0.0, prune=True), ctx.multiply(A, B, tile, 0.0))
    assert np.array_equal(ctx.get_fp16(1), orc.f32_to_f16_bits(B.cpu().numpy()))
    assert float(ctx.multiply(A, B, tile, float("inf"), prune=True).abs().max()) == 0.0
