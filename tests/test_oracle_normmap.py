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
