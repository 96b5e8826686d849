"""Pins the checker's tile Frobenius norm map (cuSpAMM.cu:21-71, 74-123:
normmap[I,J] = sqrt(sum of squares of tile (I,J)), row-major map) with closed
forms, invariants and fp64 brute force."""
import numpy as np
import pytest

TILES = [32, 64, 128]


def _bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def _brute(hbits, b):
    x = hbits.view(np.float16).astype(np.float64)
    r, c = x.shape
    return np.sqrt((x.reshape(r // b, b, c // b, b) ** 2).sum(axis=(1, 3)))


@pytest.mark.parametrize("b", TILES)
@pytest.mark.parametrize("role", [0, 1])
def test_all_ones_is_exactly_b(orc, b, role):
    # getNormMatrix input (tool.cu:370-403): every tile norm = sqrt(b*b) = b, exactly
    H = _bits(np.ones((2 * b, 3 * b)))
    nm = orc.normmap(H, b, role)
    assert nm.shape == (2, 3)
    assert np.all(nm == np.float32(b))


@pytest.mark.parametrize("b", TILES)
@pytest.mark.parametrize("role", [0, 1])
def test_identity(orc, b, role):
    H = _bits(np.eye(3 * b))
    nm = orc.normmap(H, b, role)
    expect = np.sqrt(np.float32(b)) * np.eye(3, dtype=np.float32)
    assert np.array_equal(nm, expect)


@pytest.mark.parametrize("b", TILES)
def test_single_element_position(orc, b):
    # one non-zero entry: only its tile has a norm; catches swapped tile indices / layouts
    X = np.zeros((2 * b, 4 * b), dtype=np.float32)
    X[b + 3, 2 * b + 5] = 3.0
    for role in (0, 1):
        nm = orc.normmap(_bits(X), b, role)
        expect = np.zeros((2, 4), dtype=np.float32)
        expect[1, 2] = 3.0
        assert np.array_equal(nm, expect)


@pytest.mark.parametrize("b", TILES)
def test_geometric_decay_closed_form(orc, b):
    # tool.cu:409-422: a_ij = c * v^|i-j|.  For an off-diagonal tile at tile distance D >= 1 the
    # sum of squares is v^(2bD) * (sum_{s=-(b-1)}^{b-1} (b-|s|) v^(2s)); diagonal tile similar.
    c, v, n = 1.0, 0.99, 4 * b   # entries stay normal fp16 numbers
    i, j = np.indices((n, n))
    X = (c * v ** np.abs(i - j)).astype(np.float32)
    nm = orc.normmap(_bits(X), b, 0)
    s = np.arange(-(b - 1), b)
    w = (b - np.abs(s)).astype(np.float64)
    for D in (1, 2, 3):
        closed = c * np.sqrt(np.sum(w * v ** (2.0 * (b * D + s))))
        assert abs(nm[0, D] - closed) / closed < 2e-3       # fp16 rounding of the entries
        assert nm[0, D] == nm[D, 0] or abs(nm[0, D] - nm[D, 0]) / closed < 1e-6
    closed0 = c * np.sqrt(np.sum(w * v ** (2.0 * np.abs(s))))
    assert abs(nm[1, 1] - closed0) / closed0 < 2e-3


@pytest.mark.parametrize("b", TILES)
@pytest.mark.parametrize("role", [0, 1])
def test_brute_force_fp64_and_invariant(orc, b, role):
    rng = np.random.default_rng(b + role)
    X = (rng.uniform(-1, 1, size=(3 * b, 2 * b)) * np.exp(-0.05 * rng.integers(0, 200, size=(3 * b, 2 * b))))
    H = _bits(X)
    nm = orc.normmap(H, b, role)
    ref = _brute(H, b)
    assert np.all(np.abs(nm - ref) <= 4e-7 * ref + 1e-30)    # fp32 accumulation of exact squares
    total = (H.view(np.float16).astype(np.float64) ** 2).sum()
    assert abs((nm.astype(np.float64) ** 2).sum() - total) <= 1e-6 * total


@pytest.mark.parametrize("b", TILES)
def test_role_b_is_role_a_of_the_transpose(orc, b):
    # the accumulation order runs along the contraction axis: columns for A, rows for B
    rng = np.random.default_rng(11)
    H = _bits(rng.normal(size=(2 * b, 3 * b)))
    nb = orc.normmap(H, b, 1)
    na_t = orc.normmap(np.ascontiguousarray(H.T), b, 0)
    assert np.array_equal(nb.view(np.uint32), na_t.T.view(np.uint32))


def test_order_is_the_documented_one(orc):
    # explicit pure-numpy statement of the documented fp32 order on one 32x32 tile
    b = 32
    rng = np.random.default_rng(3)
    H = _bits(rng.normal(size=(b, b)) * 10 ** rng.uniform(-4, 2, size=(b, b)))
    x = H.view(np.float16).astype(np.float32)
    sq = x * x                                              # exact in fp32
    chunk = np.zeros((b, b // 8), dtype=np.float32)
    for e in range(8):
        chunk = chunk + sq.reshape(b, b // 8, 8)[:, :, e]
    flat = chunk.reshape(-1)                                # index c = r*(b/8)+q
    partial = flat[:64].copy()
    for it in range(1, flat.size // 64):
        partial = partial + flat[it * 64:(it + 1) * 64]
    s = 1
    while s < 64:
        partial = partial + partial[np.arange(64) ^ s]
        s <<= 1
    assert orc.normmap(H, b, 0)[0, 0] == np.sqrt(partial[0])


def test_subnormal_and_zero_tiles(orc):
    b = 32
    X = np.zeros((b, 2 * b), dtype=np.float32)
    X[:, b:] = 2.0 ** -24                                   # smallest fp16 subnormal
    nm = orc.normmap(_bits(X), b, 0)
    assert nm[0, 0] == 0.0
    assert nm[0, 1] == np.float32(b * 2.0 ** -24)           # sqrt(1024 * 2^-48)


def test_rejects_bad_shapes(orc):
    with pytest.raises(ValueError):
        orc.normmap(np.zeros((48, 64), dtype=np.uint16), 32, 0)
    with pytest.raises(ValueError):
        orc.normmap(np.zeros((64, 64), dtype=np.uint16), 16, 0)


def test_reference_fp16_norm_model_and_the_gate_decisions_it_would_change(orc):
    """The reference's fp16 norm kernel (cuSpAMM.cu:74-123) rounds every square to fp16 and sums
    columns in an fp16 accumulator; the checker (and the GPU) use the clean fp32 norm.  A model of
    that arithmetic shows how far apart the two are on BASELINE's first configuration (N = 1024,
    A = B, exp(-0.5 d), tile 32, tau = 1e-4): the norms agree to ~1e-3 relative, and only products
    within that distance of tau can be gated differently.  This is a report, not a parity pin."""
    n, b, tau = 1024, 32, np.float32(1e-4)
    X = orc.fill_decay(n, n, orc.decay_table("exp", n, 0.5), 1)
    h = orc.f32_to_f16_bits(X)
    clean_a, clean_b = orc.normmap(h, b, 0), orc.normmap(h, b, 1)
    model = orc.normmap_ref16_model(h)
    # closed forms hold for the model too: all-ones tile -> exactly 32, zeros -> 0
    ones = orc.f32_to_f16_bits(np.ones((64, 64), dtype=np.float32))
    assert np.all(orc.normmap_ref16_model(ones) == 32.0)
    assert np.all(orc.normmap_ref16_model(np.zeros((32, 32), dtype=np.uint16)) == 0.0)
    nz = clean_a > 1e-3                      # tiles whose squares are not lost to fp16 underflow
    rel = np.abs(model[nz] - clean_a[nz]) / clean_a[nz]
    assert rel.max() < 5e-3
    # squares below 2^-24 vanish in fp16: far-off-diagonal tiles read as zero in the model
    assert np.count_nonzero(model == 0) >= np.count_nonzero(clean_a == 0)
    keep_clean = (clean_a[:, None, :] * clean_b.T[None, :, :]) >= tau       # [i, j, k]
    keep_model = (model[:, None, :] * model.T[None, :, :]) >= tau
    differ = int(np.count_nonzero(keep_clean != keep_model))
    total = keep_clean.size
    print("gate decisions that differ: %d of %d (%.4f %%), kept clean %d, kept model %d"
          % (differ, total, 100.0 * differ / total, keep_clean.sum(), keep_model.sum()))
    assert differ <= 0.005 * total
