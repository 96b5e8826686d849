"""GPU parity: the HIP path (through the C ABI) against the host checker.

Bars: generator, fp16 copy, norm maps, kept mask, counts and k lists are
bit-exact; C is within 1e-3 relative Frobenius error of the checker (the bar
the task states; observed ~5e-7); the error against an exact fp64 dense product
is reported next to the dropped-norm bound.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

C_REL_TOL = 1e-3
HERE = os.path.dirname(os.path.abspath(__file__))


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _run_case(orc, ctx, A, B, tile, tau):
    """Runs the multiply on the GPU and the checker on the host; asserts every bar."""
    import torch
    dA, dB = _dev(A), _dev(B)
    M, K = A.shape
    N = B.shape[1]
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ctx.multiply(dA, dB, tile, tau, C=C)
    ref = orc.spamm(A, B, tile, tau)
    assert np.array_equal(ctx.get_fp16(0), ref["hA"])
    assert np.array_equal(ctx.get_fp16(1), ref["hB"])
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), ref["nA"].view(np.uint32))
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), ref["nB"].view(np.uint32))
    assert np.array_equal(ctx.get_mask(), ref["mask"])
    counts = ctx.get_counts()
    assert np.array_equal(counts, ref["counts"])
    klist = ctx.get_klist()
    valid = np.arange(klist.shape[2])[None, None, :] < counts[:, :, None]
    assert np.array_equal(klist[valid], ref["klist"][valid])
    st = ctx.get_stats()
    assert st.kept_products == ref["kept"]
    assert st.total_products == (M // tile) * (K // tile) * (N // tile)
    Cg = C.cpu().numpy()
    assert not np.isnan(Cg).any()                            # C fully overwritten
    err, nrm, _ = orc.frob_diff(Cg, ref["C"])
    if nrm > 0:
        assert err / nrm <= C_REL_TOL
    else:
        assert err == 0
    empty = ref["counts"] == 0
    if empty.any():
        blocks = Cg.reshape(M // tile, tile, N // tile, tile).transpose(0, 2, 1, 3)
        assert np.all(blocks[empty] == 0)
    return ref, Cg


CASES = [
    # M, K, N, tile, kind, lam, tau
    (256, 256, 256, 64, "exp", 0.05, 1e-3),
    (512, 512, 512, 32, "exp", 0.02, 1e-2),
    (512, 512, 512, 128, "exp", 0.01, 300.0),
    (1024, 1024, 1024, 64, "exp", 0.01, 0.5),
    (320, 448, 768, 64, "exp", 0.01, 30.0),                  # rectangular, partial macro tiles
    (96, 160, 224, 32, "alg", 0.0, 1e-3),                    # odd tile counts
    (1024, 1024, 1024, 32, "exp", 0.5, 1e-4),                # BASELINE config 1 (A != B here)
    (1536, 1536, 1536, 64, "alg", 0.0, 1e-5),                # subnormal-heavy inputs
    (64, 64, 64, 64, "none", 0.0, 0.0),                      # one tile
    (128, 128, 128, 128, "none", 0.0, 0.0),
    (2048, 2048, 2048, 128, "exp", 0.003, 50.0),
]


@pytest.mark.parametrize("M,K,N,tile,kind,lam,tau", CASES)
def test_multiply_matches_checker(orc, ctx, M, K, N, tile, kind, lam, tau):
    tab = orc.decay_table(kind, max(M, K, N), lam)
    A = orc.fill_decay(M, K, tab, 1)
    B = orc.fill_decay(K, N, tab, 2)
    ref, _ = _run_case(orc, ctx, A, B, tile, tau)
    if tau > 0 and kind != "none":
        total = (M // tile) * (K // tile) * (N // tile)
        assert 0 < ref["kept"] < total, "case does not exercise the gate"


@pytest.mark.parametrize("M,K,N,tile,lam,tau", [(1024, 2048, 768, 64, 0.004, 0.3), (640, 1024, 896, 32, 0.01, 0.05),
                                                 (512, 4096, 1280, 128, 0.002, 5.0)])
def test_macro_tile_work_lists_match_the_mask(orc, ctx, M, K, N, tile, lam, tau):
    """spamm_get_macro_counts against the checker's mask: per 256 x 256 macro tile of C the number of
    k tiles kept by any of its output tiles and by all of them, and the per-XCD totals."""
    tab = orc.decay_table("exp", max(M, K, N), lam)
    A, B = orc.fill_decay(M, K, tab, 1), orc.fill_decay(K, N, tab, 2)
    ctx.multiply(_dev(A), _dev(B), tile, tau)
    ref = orc.spamm(A, B, tile, tau)
    counts, sched = ctx.get_macro_counts()
    nbM, nbK, nbN, mt = M // tile, K // tile, N // tile, 256 // tile
    bits = np.unpackbits(ref["mask"].view(np.uint8), axis=2, bitorder="little")[:, :, :nbK].astype(bool)   # [i, j, k]
    want = np.zeros_like(counts)
    for mi in range(counts.shape[0]):
        for mj in range(counts.shape[1]):
            blk = bits[mi * mt:(mi + 1) * mt, mj * mt:(mj + 1) * mt].reshape(-1, nbK)
            want[mi, mj, 0] = np.count_nonzero(blk.any(axis=0))
            # "kept by all" counts the tiles inside the matrix only when the macro tile is whole
            want[mi, mj, 1] = np.count_nonzero(blk.all(axis=0)) if blk.shape[0] == mt * mt else 0
    assert np.array_equal(counts[..., 0], want[..., 0])
    whole = np.zeros(counts.shape[:2], dtype=bool)
    whole[:nbM // mt, :nbN // mt] = True
    assert np.array_equal(counts[..., 1][whole], want[..., 1][whole])
    assert np.all(counts[..., 1] <= counts[..., 0])
    assert 0 < np.count_nonzero(counts[..., 0]) and sched[:8].sum() == np.count_nonzero(counts[..., 0])
    assert sched[8:].sum() == counts.shape[0] * counts.shape[1]


def test_small_products_are_dealt_to_every_xcd(orc, ctx):
    """C of fewer super tiles (4 x 8 macro tiles) than the chip has XCDs: the macro tiles themselves are
    dealt, in equal chunks of consecutive ones, so that no XCD stays empty (2048^3 at tile 32 -- the
    reference's default experiment -- is two super tiles); a larger C goes by whole super tiles."""
    import torch
    for n, tile, want in ((2048, 32, [8] * 8), (1536, 64, [5, 5, 5, 5, 5, 5, 5, 1]), (1024, 128, [2] * 8)):
        A = torch.rand((n, n), dtype=torch.float32, device="cuda")
        ctx.multiply(A, A, tile, 0.0)
        counts, sched = ctx.get_macro_counts()
        assert list(sched[8:16]) == want and list(sched[:8]) == want, (n, tile, sched)
    A = torch.rand((4096, 4096), dtype=torch.float32, device="cuda")       # 16 x 16 macro tiles = 8 super tiles
    ctx.multiply(A, A, 64, 0.0)
    counts, sched = ctx.get_macro_counts()
    assert list(sched[8:16]) == [32] * 8


def test_baseline_config1_a_equals_b(orc, ctx):
    # N=1024, A=B, exp(-0.5|i-j|), tile 32, tau=1e-4
    tab = orc.decay_table("exp", 1024, 0.5)
    A = orc.fill_decay(1024, 1024, tab, 1)
    ref, _ = _run_case(orc, ctx, A, A.copy(), 32, 1e-4)
    assert 0.005 < ref["kept"] / 32 ** 3 < 0.03


def test_reference_default_experiment(orc, ctx):
    """The reference as checked out (para.h:1-14, cuSpAMM.cu:428-431): 2048^3, tile 32 (main.h:32),
    both operands getDecayMatrixAlg(0.1, 0.1) (tool.cu:426-436), Norm = 1.548969, fp16 inputs
    (USINGHALF 1) resident before the multiply."""
    import torch
    n, b, tau = 2048, 32, 1.548969
    tab = orc.decay_table("ref_alg", n, c=0.1, v=0.1)
    A = orc.fill_decay(n, n, tab, 0, random=False)
    dA32 = torch.empty((n, n), dtype=torch.float32, device="cuda")
    ctx.fill_decay(dA32, tab, 0, random=False)                     # the device generator gives the same matrix
    assert np.array_equal(dA32.cpu().numpy(), A)
    hA = dA32.half()
    hB = hA.clone()
    C = torch.full((n, n), float("nan"), dtype=torch.float32, device="cuda")
    ctx.multiply(hA, hB, b, tau, C=C)
    ref = orc.spamm(A, A.copy(), b, tau)
    assert np.array_equal(ctx.get_fp16(0), ref["hA"]) and np.array_equal(ctx.get_fp16(1), ref["hB"])
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), ref["nA"].view(np.uint32))
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), ref["nB"].view(np.uint32))
    assert np.array_equal(ctx.get_mask(), ref["mask"])
    assert np.array_equal(ctx.get_counts(), ref["counts"])
    st = ctx.get_stats()
    assert st.kept_products == ref["kept"] and 0.04 < st.kept_products / st.total_products < 0.06
    Cg = C.cpu().numpy()
    assert not np.isnan(Cg).any()
    err, nrm, _ = orc.frob_diff(Cg, ref["C"])
    assert err <= C_REL_TOL * nrm
    # the tuner the reference runs on this matrix (tuneValidRate, tool.cu:438-490; main.h:35-38)
    assert ctx.tune_bisect(0.75, 0.01, 20) == pytest.approx(orc.tune_bisect(ref["nA"], ref["nB"], 0.75, 0.01, 20))
    # the pruned call and the A = B single pass give the same C bit for bit
    C2 = ctx.multiply(hA, hB, b, tau, prune=True)
    assert torch.equal(C2, C)
    C3 = ctx.multiply(hA, hA, b, tau, a_eq_b=True)
    assert torch.equal(C3, C)


@pytest.mark.parametrize("name", ["exp_b32", "exp_b64_rect", "alg_b32", "exp_b128"])
def test_against_committed_golden_vectors(ctx, name):
    import torch
    g = np.load(os.path.join(HERE, "golden", "spamm_small.npz"))
    M, K, N, tile = (int(v) for v in g[name + "_cfg"])
    tau = float(g[name + "_tau"][0])
    dA = torch.empty((M, K), dtype=torch.float32, device="cuda")
    dB = torch.empty((K, N), dtype=torch.float32, device="cuda")
    ctx.fill_decay(dA, g[name + "_table"], 1)
    ctx.fill_decay(dB, g[name + "_table"], 2)
    assert np.array_equal(dA[:4, :8].cpu().numpy(), g[name + "_A_sample"])
    assert np.array_equal(dB[-4:, -8:].cpu().numpy(), g[name + "_B_sample"])
    C = ctx.multiply(dA, dB, tile, tau)
    assert np.array_equal(ctx.get_normmap(0).view(np.uint32), g[name + "_nA"].view(np.uint32))
    assert np.array_equal(ctx.get_normmap(1).view(np.uint32), g[name + "_nB"].view(np.uint32))
    assert np.array_equal(ctx.get_counts(), g[name + "_counts"])
    assert np.array_equal(ctx.get_mask(), g[name + "_mask"])
    Cg = C.cpu().numpy().astype(np.float64)
    ref = g[name + "_C"].astype(np.float64)
    assert np.linalg.norm(Cg - ref) <= C_REL_TOL * np.linalg.norm(ref)


def test_device_generator_is_bit_identical(orc, ctx):
    import torch
    for rows, cols, kind, lam, rnd in [(256, 512, "exp", 0.1, True), (384, 128, "alg", 0, True),
                                       (128, 128, "ref_alg", 0, False), (128, 256, "ref_exp", 0, False)]:
        tab = orc.decay_table(kind, max(rows, cols), lam, c=0.1, v=0.1)
        X = torch.empty((rows, cols), dtype=torch.float32, device="cuda")
        ctx.fill_decay(X, tab, 42, random=rnd)
        ref = orc.fill_decay(rows, cols, tab, 42, random=rnd)
        assert np.array_equal(X.cpu().numpy().view(np.uint32), ref.view(np.uint32))


def test_conversion_edge_values(orc, ctx):
    # ties, subnormals, overflow, signed zeros: the device conversion must be IEEE RNE
    rng = np.random.default_rng(0)
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0
    mid = ((lo + hi) / 2).astype(np.float32)
    vals = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)),
                           np.array([0.0, -0.0, 65504.0, 65519.0, 2.0 ** -24, 2.0 ** -25, 3e-8, 1e-10], dtype=np.float32)])
    vals = np.concatenate([vals, -vals, rng.normal(size=4096).astype(np.float32) * 1e-6])
    n = 512 * 256
    X = np.resize(vals, n).reshape(512, 256).astype(np.float32)
    import torch
    for role in (0, 1):
        ctx.normmap_f32(role, _dev(X), 64)
        got = ctx.get_fp16(role)
        assert np.array_equal(got, orc.f32_to_f16_bits(X))
        nm = ctx.get_normmap(role)
        assert np.array_equal(nm.view(np.uint32), orc.normmap(got, 64, role).view(np.uint32))


def test_closed_forms_on_device(ctx):
    import torch
    for tile in (32, 64, 128):
        n = 2 * tile
        ones = torch.ones((n, 3 * tile), dtype=torch.float32, device="cuda")
        onesB = torch.ones((3 * tile, n), dtype=torch.float32, device="cuda")
        C = ctx.multiply(ones, onesB, tile, 0.0)
        assert torch.all(C == 3 * tile)                       # every entry = K exactly
        assert np.all(ctx.get_normmap(0) == tile) and np.all(ctx.get_normmap(1) == tile)
        # identity: C = fp16(B) on the kept tiles, diagonal tile norms sqrt(b)
        eye = torch.eye(n, dtype=torch.float32, device="cuda")
        B = torch.rand((n, n), dtype=torch.float32, device="cuda") - 0.5
        C = ctx.multiply(eye, B, tile, 1e-6)
        assert torch.equal(C, B.half().float())
        nmA = ctx.get_normmap(0)
        assert np.array_equal(nmA, np.sqrt(np.float32(tile)) * np.eye(2, dtype=np.float32))


def test_tau_extremes(orc, ctx):
    import torch
    tab = orc.decay_table("exp", 512, 0.02)
    A = orc.fill_decay(512, 512, tab, 1)
    B = orc.fill_decay(512, 512, tab, 2)
    ref, Cg = _run_case(orc, ctx, A, B, 64, 0.0)
    assert ref["kept"] == 8 ** 3
    dense = orc.gemm_dense_f64(ref["Af"], ref["Bf"])
    err, nrm, _ = orc.frob_diff(Cg, dense)
    assert err / nrm < 1e-5                                   # tau=0 is a plain fp16 GEMM
    ref, Cg = _run_case(orc, ctx, A, B, 64, float("inf"))
    assert ref["kept"] == 0 and np.all(Cg == 0)


def test_hand_built_normmaps_straddling_tau(orc, ctx):
    # exact equality must be kept ('>=', cuSpAMM.cu:306)
    nA = np.array([[2.0, 1.0], [0.5, 4.0]], dtype=np.float32)
    nB = np.array([[3.0, 1.0], [6.0, 1.5]], dtype=np.float32)
    for tile in (32, 64, 128):
        for tau in (6.0, float(np.nextafter(np.float32(6.0), np.float32(7.0))), 0.0, 1.5, 24.0, 25.0):
            ctx.set_normmaps(nA, nB, tile)
            ctx.gate(tau)
            total, counts, klist, mask = orc.gate(nA, nB, tau)
            assert np.array_equal(ctx.get_counts(), counts)
            assert np.array_equal(ctx.get_mask(), mask)
            assert ctx.get_stats().kept_products == total
    ctx.set_normmaps(nA, nB, 64)
    ctx.gate(6.0)
    assert ctx.get_counts().tolist() == [[2, 0], [1, 1]]


def test_gate_on_random_maps_with_ragged_k(orc, ctx):
    rng = np.random.default_rng(4)
    for nbM, nbK, nbN, tile in [(5, 70, 3, 64), (9, 130, 11, 32), (3, 513, 2, 128), (1, 1, 1, 64), (17, 64, 9, 32)]:
        nA = np.abs(rng.normal(size=(nbM, nbK))).astype(np.float32)
        nB = np.abs(rng.normal(size=(nbK, nbN))).astype(np.float32)
        nA[rng.random(nA.shape) < 0.1] = 0
        for tau in (0.0, 0.3, 1.0, 4.0):
            ctx.set_normmaps(nA, nB, tile)
            ctx.gate(tau)
            total, counts, klist, mask = orc.gate(nA, nB, tau)
            assert np.array_equal(ctx.get_counts(), counts)
            assert np.array_equal(ctx.get_mask(), mask)
            got = ctx.get_klist()
            valid = np.arange(nbK)[None, None, :] < counts[:, :, None]
            assert np.array_equal(got[valid], klist[valid])
            assert ctx.get_stats().kept_products == total


def test_gate_at_the_most_super_tiles_of_c(orc, ctx):
    # 64 x 128 = 8192 super tiles of C (tile 128: 512 x 2048 tiles) fill the schedule kernel's
    # tables to their limit; one tile more in either direction is refused, not mis-scheduled
    import cuspamm_amd as sp
    rng = np.random.default_rng(11)
    nbM, nbK, nbN, tile = 512, 2, 2048, 128
    nA = np.abs(rng.normal(size=(nbM, nbK))).astype(np.float32)
    nB = np.abs(rng.normal(size=(nbK, nbN))).astype(np.float32)
    ctx.set_normmaps(nA, nB, tile)
    ctx.gate(1.0)
    total, counts, _, mask = orc.gate(nA, nB, 1.0, want_klist=False)
    assert np.array_equal(ctx.get_counts(), counts)
    assert np.array_equal(ctx.get_mask(), mask)
    assert ctx.get_stats().kept_products == total
    for shape in ((nbM + 1, nbN), (nbM, nbN + 1)):
        ctx.set_normmaps(np.ones((shape[0], nbK), np.float32), np.ones((nbK, shape[1]), np.float32), tile)
        with pytest.raises(sp.SpammError) as e:
            ctx.gate(1.0)
        assert e.value.code == -1                             # invalid argument: size limit


def test_error_vs_fp64_dense_and_bound(orc, ctx):
    tab = orc.decay_table("exp", 1024, 0.01)
    A = orc.fill_decay(1024, 1024, tab, 1)
    B = orc.fill_decay(1024, 1024, tab, 2)
    import torch
    dA, dB = _dev(A), _dev(B)
    ctx.normmap_f32(1, dB, 64)
    ctx.normmap_f32(0, dA, 64)
    nA, nB = ctx.get_normmap(0), ctx.get_normmap(1)
    Af = orc.f16_bits_to_f32(ctx.get_fp16(0))
    Bf = orc.f16_bits_to_f32(ctx.get_fp16(1))
    dense = orc.gemm_dense_f64(Af, Bf)
    last = -1.0
    for ratio in (0.9, 0.5, 0.2, 0.05):
        tau, _ = orc.tau_for_ratio(nA, nB, ratio)
        C = ctx.multiply(dA, dB, 64, tau).cpu().numpy()
        err, nrm, _ = orc.frob_diff(C, dense)
        bound = orc.dropped_bound(nA, nB, tau)
        assert err <= bound * (1 + 1e-4) + 1e-5 * nrm         # measured error within the tau-derived bound
        assert bound <= tau * 16 * 16 * (1 + 1e-6)            # tau * nbK * sqrt(nbM*nbN)
        assert err >= last                                    # dropping more cannot reduce the error here
        last = err


def test_argument_errors(ctx):
    import torch
    import cuspamm_amd as sp
    A = torch.zeros((128, 128), dtype=torch.float32, device="cuda")
    C = torch.zeros((128, 128), dtype=torch.float32, device="cuda")
    pa, pc = A.data_ptr(), C.data_ptr()
    bad = [
        sp.SpammParams(128, 128, 128, 48, 0.0, 0, 0),         # tile not in {32,64,128}
        sp.SpammParams(100, 128, 128, 32, 0.0, 0, 0),         # M not a tile multiple
        sp.SpammParams(128, 128, 96, 64, 0.0, 0, 0),
        sp.SpammParams(0, 128, 128, 32, 0.0, 0, 0),
        sp.SpammParams(128, 128, 128, 32, float("nan"), 0, 0),
    ]
    for p in bad:
        assert ctx.multiply_raw(p, pa, pa, pc) == -1
    ok = sp.SpammParams(128, 128, 128, 32, 0.0, 0, 0)
    assert ctx.multiply_raw(ok, 0, pa, pc) == -1              # null pointers
    assert ctx.multiply_raw(ok, pa, pa, 0) == -1
    assert ctx.multiply_raw(ok, pa, pa, pc) == 0
    fresh = sp.SpammContext(0)
    with pytest.raises(sp.SpammError) as ei:
        fresh.gate(0.0)
    assert ei.value.code == -4                                # nothing to gate yet
    fresh.normmap_f32(0, A, 32)
    with pytest.raises(sp.SpammError) as ei:
        fresh.gemm_gated(C)
    assert ei.value.code == -4
    fresh.close()


def test_stages_refuse_norm_maps_of_mismatched_shape(ctx):
    """A norm map of B taken at one K and one of A taken at another must not be gated together:
    every stage that reads both returns SPAMM_ESTATE (and launches nothing)."""
    import torch
    import cuspamm_amd as sp
    fresh = sp.SpammContext(0)
    B = torch.ones((128, 128), dtype=torch.float32, device="cuda")
    A = torch.ones((128, 256), dtype=torch.float32, device="cuda")
    fresh.normmap_f32(sp.ROLE_B, B, 32)                       # K = 128
    fresh.normmap_f32(sp.ROLE_A, A, 32)                       # K = 256: B's map no longer fits
    for call in (lambda: fresh.gate(0.0), lambda: fresh.tau_for_ratio(0.5), lambda: fresh.count_kept(0.0),
                 lambda: fresh.dropped_bound(0.0), lambda: fresh.tune_bisect(), lambda: fresh.get_normmap(sp.ROLE_B)):
        with pytest.raises(sp.SpammError) as ei:
            call()
        assert ei.value.code == -4
    assert fresh.get_normmap(sp.ROLE_A).shape == (4, 8)       # A's own map is fine
    fresh.normmap_f32(sp.ROLE_B, torch.ones((256, 64), dtype=torch.float32, device="cuda"), 32)
    fresh.gate(0.0)                                           # matching K again
    assert int(fresh.get_counts().sum()) == 4 * 8 * 2
    # the other way round, and a tile change
    fresh.normmap_f32(sp.ROLE_B, B, 32)
    with pytest.raises(sp.SpammError) as ei:
        fresh.gate(0.0)
    assert ei.value.code == -4
    fresh.normmap_f32(sp.ROLE_A, torch.ones((64, 128), dtype=torch.float32, device="cuda"), 64)
    with pytest.raises(sp.SpammError) as ei:
        fresh.gate(0.0)
    assert ei.value.code == -4
    fresh.close()


def test_workspace_reuse_across_shapes(orc, ctx):
    # same context, shrinking and growing problems, different tiles: no stale state
    for M, K, N, tile, tau in [(512, 256, 384, 64, 5.0), (128, 128, 128, 32, 0.1), (768, 512, 256, 128, 100.0),
                               (128, 128, 128, 32, 0.1)]:
        tab = orc.decay_table("exp", max(M, K, N), 0.01)
        _run_case(orc, ctx, orc.fill_decay(M, K, tab, 3), orc.fill_decay(K, N, tab, 4), tile, tau)


def test_stage_api_equals_multiply(orc, ctx):
    import torch
    tab = orc.decay_table("exp", 512, 0.02)
    dA, dB = _dev(orc.fill_decay(512, 512, tab, 1)), _dev(orc.fill_decay(512, 512, tab, 2))
    C1 = ctx.multiply(dA, dB, 64, 0.7).clone()
    ctx.normmap_f32(1, dB, 64)
    ctx.normmap_f32(0, dA, 64)
    ctx.gate(0.7)
    C2 = torch.empty_like(C1)
    ctx.gemm_gated(C2)
    assert torch.equal(C1, C2)
    # re-gating with another tau reuses the norm maps and operands
    ctx.gate(0.0)
    ctx.gemm_gated(C2)
    C3 = ctx.multiply(dA, dB, 64, 0.0)
    assert torch.equal(C2, C3)


def test_two_contexts_on_two_streams_do_not_interfere(orc, ctx):
    """Distinct contexts are independent (no globals): two of them, each on its own stream (default
    priority), run different problems alternately; each must reproduce what the session context
    computes alone."""
    import torch
    import cuspamm_amd as sp
    cases = []
    for M, K, N, tile, lam, ratio, seed in [(768, 512, 640, 64, 0.01, 0.3, 5), (512, 1024, 384, 32, 0.02, 0.1, 7)]:
        tab = orc.decay_table("exp", max(M, K, N), lam)
        dA, dB = _dev(orc.fill_decay(M, K, tab, seed)), _dev(orc.fill_decay(K, N, tab, seed + 1))
        ctx.normmap_f32(1, dB, tile)
        ctx.normmap_f32(0, dA, tile)
        tau = ctx.tau_for_ratio(ratio)[0]
        cases.append((dA, dB, tile, tau, ctx.multiply(dA, dB, tile, tau).clone(), ctx.get_mask()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    others = [sp.SpammContext(0), sp.SpammContext(0)]
    outs = [torch.empty_like(c[4]) for c in cases]
    try:
        for c2, s in zip(others, streams):
            c2.set_stream(s.cuda_stream)
        for rep in range(4):
            for i in (0, 1):
                dA, dB, tile, tau = cases[i][:4]
                others[i].multiply(dA, dB, tile, tau, C=outs[i], prune=bool(rep & 1))
        for i in (0, 1):
            others[i].synchronize()
            assert torch.equal(outs[i], cases[i][4])
            assert np.array_equal(others[i].get_mask(), cases[i][5])
    finally:
        for c2 in others:
            c2.close()
