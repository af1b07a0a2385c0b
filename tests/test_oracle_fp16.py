"""Pins the oracle's binary16 arithmetic (oracle/mgemv_oracle.c) against independent evidence:
numpy's float16 (a different implementation), exact rational arithmetic, and IEEE special cases.
Every other oracle function is built from these primitives."""
from fractions import Fraction

import numpy as np

import oracle as orc

ALL = np.arange(65536, dtype=np.uint16)
FINITE = ALL[(ALL & 0x7C00) != 0x7C00]


def _rng(seed):
    return np.random.default_rng(seed)


def test_half_to_float_is_exact_for_every_half():
    got = orc.f16_to_f32_array(ALL)
    ref = ALL.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])
    assert np.isnan(got[nan]).all()


def test_float_to_half_round_trip_and_rne_against_numpy():
    # every half survives a round trip
    rt = orc.f32_to_f16_array(ALL.view(np.float16).astype(np.float32))
    nan = np.isnan(ALL.view(np.float16))
    assert np.array_equal(rt[~nan], ALL[~nan])
    # random binary32 bit patterns (all exponents, both signs)
    bits = _rng(1).integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    vals = bits.view(np.float32)
    ok = ~np.isnan(vals)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f32_to_f16_array(vals)[ok], vals.astype(np.float16).view(np.uint16)[ok])
    # dense sampling of the half range, where rounding actually happens
    dense = (_rng(2).random(2_000_000, dtype=np.float32) * 2 - 1) * np.float32(70000.0)
    dense[::2] *= np.float32(1e-4)
    dense[::5] *= np.float32(1e-3)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f32_to_f16_array(dense), dense.astype(np.float16).view(np.uint16))


def test_float_to_half_ties_go_to_even():
    # the exact midpoint between consecutive positive halves a < b rounds to the one with even mantissa
    pos = FINITE[(FINITE & 0x8000) == 0]
    a = pos[:-1].astype(np.uint16)
    b = (a + 1).astype(np.uint16)
    keep = (b & 0x7C00) != 0x7C00
    a, b = a[keep], b[keep]
    mid = (a.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)) / 2
    mid32 = mid.astype(np.float32)
    assert np.array_equal(mid32.astype(np.float64), mid)  # midpoints are exact in binary32
    got = orc.f32_to_f16_array(mid32)
    expect = np.where(a & 1, b, a)
    assert np.array_equal(got, expect)
    # overflow boundary: 65520 is the midpoint between 65504 and 2^16 -> rounds to infinity; just below stays finite
    assert orc.f32_to_f16(65520.0) == 0x7C00
    assert orc.f32_to_f16(np.nextafter(np.float32(65520.0), np.float32(0))) == 0x7BFF
    # underflow boundary: 2^-25 is a tie between 0 and the smallest subnormal -> 0; just above -> 1
    assert orc.f32_to_f16(2.0 ** -25) == 0
    assert orc.f32_to_f16(np.nextafter(np.float32(2.0 ** -25), np.float32(1))) == 1
    assert orc.f32_to_f16(-0.0) == 0x8000


def test_mul_and_add_match_numpy_half_arithmetic():
    r = _rng(3)
    a = r.choice(FINITE, size=3_000_000)
    b = r.choice(FINITE, size=3_000_000)
    with np.errstate(over="ignore", invalid="ignore"):
        ref_mul = (a.view(np.float16) * b.view(np.float16)).view(np.uint16)
        ref_add = (a.view(np.float16) + b.view(np.float16)).view(np.uint16)
    got_mul, got_add = orc.h_mul_array(a, b), orc.h_add_array(a, b)
    ok = ~np.isnan(ref_mul.view(np.float16))
    assert np.array_equal(got_mul[ok], ref_mul[ok])
    ok = ~np.isnan(ref_add.view(np.float16))
    assert np.array_equal(got_add[ok], ref_add[ok])


def test_mul_and_add_are_correctly_rounded_exact_rational():
    """numpy could share a double-rounding flaw with the oracle; exact rationals cannot."""
    r = _rng(4)
    a = r.choice(FINITE, size=4000)
    b = r.choice(FINITE, size=4000)
    mul, add = orc.h_mul_array(a, b), orc.h_add_array(a, b)

    grid = sorted(set(Fraction(float(v)) for v in FINITE.view(np.float16)))

    def nearest_even(x):
        # correctly rounded binary16 of the rational x, by search over the finite grid
        import bisect
        i = bisect.bisect_left(grid, x)
        if i == 0:
            return grid[0]
        if i == len(grid):
            top = grid[-1]
            return None if x >= Fraction(65520) else top
        lo, hi = grid[i - 1], grid[i]
        if x - lo < hi - x:
            return lo
        if x - lo > hi - x:
            return hi
        lo_bits = np.float16(float(lo)).view(np.uint16)
        return lo if (int(lo_bits) & 1) == 0 else hi

    for i in range(a.size):
        fa, fb = Fraction(float(a[i:i + 1].view(np.float16)[0])), Fraction(float(b[i:i + 1].view(np.float16)[0]))
        for got, exact in ((mul[i], fa * fb), (add[i], fa + fb)):
            want = nearest_even(exact)
            gv = float(np.uint16(got).view(np.float16))
            if want is None or abs(exact) >= Fraction(65520):
                assert np.isinf(gv)
            else:
                assert Fraction(gv) == want, (hex(int(a[i])), hex(int(b[i])), hex(int(got)))


def test_fma_single_rounding_exact_rational():
    r = _rng(5)
    # operands in a range where products and sums stay finite
    sel = FINITE[(FINITE & 0x7FFF) < 0x5C00]
    a, b, c = (r.choice(sel, size=3000) for _ in range(3))
    got = orc.h_fma_array(a, b, c)
    for i in range(a.size):
        fa, fb, fc = (Fraction(float(v[i:i + 1].view(np.float16)[0])) for v in (a, b, c))
        exact = fa * fb + fc
        # correctly rounded result via float64 -> float16 of an exactly representable value is
        # not available in general, so compare with the two neighbouring halves instead
        gv = Fraction(float(np.uint16(got[i]).view(np.float16)))
        up = Fraction(float(np.nextafter(np.float16(float(gv)), np.float16(np.inf))))
        dn = Fraction(float(np.nextafter(np.float16(float(gv)), np.float16(-np.inf))))
        assert abs(exact - gv) <= abs(exact - up) and abs(exact - gv) <= abs(exact - dn)
        if abs(exact - gv) == abs(exact - up) or abs(exact - gv) == abs(exact - dn):
            assert int(got[i]) & 1 == 0  # a tie must have gone to even


def test_fused_and_unfused_dequantisation_differ_somewhere():
    """The dequantiser is multiply THEN add (two roundings); a contracted FMA must be detectable."""
    r = _rng(6)
    q = np.array([orc.f32_to_f16(float(v)) for v in r.integers(-8, 8, size=20000)], dtype=np.uint16)
    s = orc.fill_uniform_f16(20000, 11, 0.001, 0.02).view(np.uint16)
    z = orc.fill_uniform_f16(20000, 12, -0.05, 0.05).view(np.uint16)
    two_step = orc.h_add_array(orc.h_mul_array(q, s), z)
    fused = orc.h_fma_array(q, s, z)
    assert (two_step != fused).sum() > 100
