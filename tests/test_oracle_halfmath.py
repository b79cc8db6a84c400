"""Pins the oracle's binary16 arithmetic against numpy.float16 and exact rationals."""
from fractions import Fraction

import numpy as np

import pyoracle as po

L = po.lib


def _bits(a):
    return np.asarray(a, np.float16).view(np.uint16)


def test_h2f_all_patterns_match_numpy():
    allh = np.arange(65536, dtype=np.uint16)
    ref = allh.view(np.float16).astype(np.float32)
    got = np.array([L.orc_h2f(int(h)) for h in allh], np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    # vectorised path (F16C) agrees with the scalar one
    vec = po.h2f(allh.view(np.float16))
    assert np.array_equal(vec[~nan].view(np.uint32), ref[~nan].view(np.uint32))


def test_f2h_matches_numpy_rtne_including_ties_and_subnormals():
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-8, 5, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  6.1e-5, 6.09e-5, np.inf, -np.inf], np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0,
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f2h(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, ref)
    assert np.array_equal(po.f2h(xs).view(np.uint16), ref)


def test_add_sub_mul_div_match_numpy_float16():
    rng = np.random.default_rng(1)
    a = rng.integers(0, 65536, 30000).astype(np.uint16)
    b = rng.integers(0, 65536, 30000).astype(np.uint16)
    af, bf = a.view(np.float16), b.view(np.float16)
    ok = np.isfinite(af) & np.isfinite(bf)
    a, b, af, bf = a[ok], b[ok], af[ok], bf[ok]
    with np.errstate(all="ignore"):
        for name, ref in (("orc_hadd", af + bf), ("orc_hsub", af - bf), ("orc_hmul", af * bf),
                          ("orc_hdiv", af / bf)):
            f = getattr(L, name)
            got = np.array([f(int(x), int(y)) for x, y in zip(a, b)], np.uint16)
            refb = ref.view(np.uint16)
            nan = np.isnan(ref)
            assert np.array_equal(np.isnan(got.view(np.float16)), nan), name
            assert np.array_equal(got[~nan], refb[~nan]), name


def _round_fraction_to_half(fr):
    """Correctly rounded (RTNE) binary16 of an exact rational, via integer arithmetic."""
    if fr == 0:
        return np.float16(0.0)
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2:
        fr /= 2
        e += 1
    while fr < 1:
        fr *= 2
        e -= 1
    if e < -14:  # subnormal: unit 2^-24
        scaled = fr * Fraction(2) ** (e + 24)
        unit = Fraction(2) ** -24
    else:
        scaled = fr * 1024
        unit = Fraction(2) ** (e - 10)
    q = scaled.numerator // scaled.denominator
    rem = scaled - q
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and q % 2 == 1):
        q += 1
    val = q * unit
    if val >= 65520:
        return np.float16(sign * np.inf)
    return np.float16(sign * float(val))


def test_hfma_is_a_single_rounding_of_the_exact_result():
    rng = np.random.default_rng(2)
    cases = []
    for _ in range(4000):
        a, b, c = (rng.integers(0, 0x7C00, 3) | (rng.integers(0, 2, 3) << 15)).astype(np.uint16)
        cases.append((int(a), int(b), int(c)))
    # product exactly on a tie of the result precision, addend far too small for a double sum
    tie_a = np.float16(1.0 + 2.0 ** -10).view(np.uint16)  # (1+2^-10)^2 = 1+2^-9+2^-20
    tiny = np.float16(6e-8).view(np.uint16)
    cases += [(int(tie_a), int(tie_a), int(tiny)), (int(tie_a), int(tie_a), int(tiny) | 0x8000)]
    big = np.float16(2048.0).view(np.uint16)
    odd = np.float16(2049.0 if False else 1025.0).view(np.uint16)
    cases += [(int(big), int(odd), int(tiny)), (int(big), int(odd), int(tiny) | 0x8000)]
    for a, b, c in cases:
        fa, fb, fc = (np.uint16(v).view(np.float16) for v in (a, b, c))
        exact = Fraction(float(fa)) * Fraction(float(fb)) + Fraction(float(fc))
        ref = _round_fraction_to_half(exact)
        got = np.uint16(L.orc_hfma(a, b, c)).view(np.float16)
        if exact == 0:
            assert float(got) == 0.0
        else:
            assert got.view(np.uint16) == ref.view(np.uint16), (a, b, c, float(got), float(ref))


def test_d2h_single_rounding_differs_from_double_rounding_where_it_should():
    # 1 + 2^-11 + 2^-30 lies just above a tie: direct rounding goes up, via-float stays a tie -> even
    d = 1.0 + 2.0 ** -11 + 2.0 ** -30
    assert np.uint16(L.orc_d2h(d)).view(np.float16) == np.float16(1.0 + 2.0 ** -10)
    assert np.float16(np.float32(d)) == np.float16(1.0)  # the double-rounding trap
