"""Pins the checker's fp32->fp16 conversion (tool.cu:418 __float2half, RNE)
against numpy's IEEE float16 cast, which is an independent implementation."""
import numpy as np


def _np_bits(x):
    with np.errstate(over="ignore"):
        return x.astype(np.float16).view(np.uint16)


def test_all_fp16_values_round_trip(orc):
    h = np.arange(65536, dtype=np.uint16)
    x = orc.f16_bits_to_f32(h)
    ref = h.view(np.float16).astype(np.float32)
    assert np.array_equal(x.view(np.uint32), ref.view(np.uint32))
    finite = np.isfinite(ref)
    back = orc.f32_to_f16_bits(x)
    assert np.array_equal(back[finite], h[finite])
    nan = np.isnan(ref)
    assert np.all(np.isnan(back[nan].view(np.float16)))


def test_strided_sweep_of_all_fp32_patterns(orc):
    # every 2^11-th bit pattern plus an odd offset: 2M values across all exponents
    u = (np.arange(0, 1 << 32, 1 << 11, dtype=np.uint64) + 1237).astype(np.uint32)
    x = u.view(np.float32)
    ok = ~np.isnan(x)
    assert np.array_equal(orc.f32_to_f16_bits(x)[ok], _np_bits(x)[ok])


def test_ties_and_neighbours(orc):
    # midpoints between consecutive fp16 values (normal and subnormal) and their fp32 neighbours
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0   # the overflow threshold midpoint 65520
    mid = ((lo + hi) / 2).astype(np.float32)
    pats = []
    for d in (-1, 0, 1):
        pats.append((mid.view(np.uint32).astype(np.int64) + d).astype(np.uint32).view(np.float32))
    x = np.concatenate(pats)
    x = np.concatenate([x, -x])
    assert np.array_equal(orc.f32_to_f16_bits(x), _np_bits(x))


def test_specials(orc):
    x = np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 1e10, -1e10,
                  2.0 ** -24, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  2.0 ** -26, 2.0 ** -14, np.nextafter(np.float32(2.0 ** -14), np.float32(0))],
                 dtype=np.float32)
    assert np.array_equal(orc.f32_to_f16_bits(x), _np_bits(x))


def test_random_bits(orc):
    rng = np.random.default_rng(7)
    u = rng.integers(0, 1 << 32, size=1 << 21, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    ok = ~np.isnan(x)
    assert np.array_equal(orc.f32_to_f16_bits(x)[ok], _np_bits(x)[ok])
