"""Pins the checker's binary16 arithmetic (oracle/orc_half.h) without the reference:
conversions against numpy.float16 (an independent IEEE implementation) exhaustively,
add/sub/mul/fma against exact rational arithmetic rounded by an integer routine
written here.  A wrong tie rule, a dropped sticky bit or a double rounding fails."""
from fractions import Fraction

import numpy as np
import pytest


def half_bits_to_fraction(h):
    s = -1 if h & 0x8000 else 1
    e = (h >> 10) & 0x1F
    m = h & 0x3FF
    assert e != 0x1F
    if e == 0:
        return s * Fraction(m, 1 << 24)
    return s * Fraction((1 << 10) | m, 1 << 10) * Fraction(2) ** (e - 15)


def round_fraction_to_half(x):
    """Exact value -> binary16 bits, round to nearest even, overflow to inf."""
    if x == 0:
        return 0
    sign = 0x8000 if x < 0 else 0
    a = abs(x)
    # exponent of the leading bit
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -14)                      # subnormals share the exponent of 2^-14
    ulp = Fraction(2) ** (e - 10)
    q = a / ulp                          # in [1024, 2048) for normals, [0,1024) for subnormals
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    v = n * ulp
    if v >= 65536:
        return sign | 0x7C00
    if n == 0:
        return sign
    if n == 2048:
        e += 1
        n = 1024
    if n < 1024:                         # subnormal
        return sign | n
    return sign | ((e + 15) << 10) | (n - 1024)


def test_rounding_helper_against_numpy():
    rng = np.random.default_rng(0)
    xs = rng.standard_normal(2000) * np.exp(rng.uniform(-18, 11, 2000))
    for x in xs:
        want = int(np.float16(x).view(np.uint16))
        assert round_fraction_to_half(Fraction(float(x))) == want


def test_widen_exhaustive(orc):
    h = np.arange(65536, dtype=np.uint16)
    got = orc.h2f(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))


@pytest.mark.parametrize("which", ["orc", "orc_soft"])
def test_narrow_round_trip_midpoints_and_random(which, request):
    o = request.getfixturevalue(which)
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(f)
    assert np.array_equal(o.f2h(f[finite]), h[finite])
    # every float that is the exact midpoint of two adjacent halves, and its two float neighbours
    pos = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = pos.view(np.float16).astype(np.float64)
    hi = (pos + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0                                      # the "next half" above 65504 for the overflow tie
    mid = ((lo + hi) / 2).astype(np.float32)
    cases = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    cases = np.concatenate([cases, -cases])
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    assert np.array_equal(o.f2h(cases), want)
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(o.f2h(x), want)
    assert np.isnan(o.h2f(o.f2h(np.array([np.nan], np.float32)))[0])


def test_double_to_half_single_rounding(orc):
    # 1 + 2^-11 + 2^-40 lies above the tie: binary32 rounding first would land on the tie and round to even
    x = 1.0 + 2.0 ** -11 + 2.0 ** -40
    assert orc.lib.orc_double2half(x) == 0x3C01
    assert orc.lib.orc_float2half(np.float32(x)) == 0x3C00
    rng = np.random.default_rng(2)
    xs = rng.standard_normal(5000) * np.exp(rng.uniform(-20, 12, 5000))
    for v in xs:
        assert orc.lib.orc_double2half(float(v)) == round_fraction_to_half(Fraction(float(v)))


def _random_halves(rng, n):
    h = rng.integers(0, 65536, n).astype(np.uint16)
    e = (h >> 10) & 0x1F
    return h[e != 0x1F]


def test_add_sub_mul_exact(orc):
    rng = np.random.default_rng(3)
    a = _random_halves(rng, 6000)
    b = _random_halves(rng, 6000)
    n = min(a.size, b.size)
    # bias half of the pairs to nearby exponents so cancellation and ties are exercised
    b[: n // 2] = (a[: n // 2] ^ rng.integers(0, 1 << 11, n // 2).astype(np.uint16))
    for x, y in zip(a[:n].tolist(), b[:n].tolist()):
        if ((y >> 10) & 0x1F) == 0x1F:
            continue
        fx, fy = half_bits_to_fraction(x), half_bits_to_fraction(y)
        for name, exact in (("orc_half_add", fx + fy), ("orc_half_sub", fx - fy), ("orc_half_mul", fx * fy)):
            got = getattr(orc.lib, name)(x, y)
            want = round_fraction_to_half(exact)
            if exact == 0:
                assert got & 0x7FFF == 0
            else:
                assert got == want, (name, hex(x), hex(y), hex(got), hex(want))


def test_add_mul_against_numpy_bulk(orc):
    rng = np.random.default_rng(4)
    a = _random_halves(rng, 300000)
    b = _random_halves(rng, 300000)
    n = min(a.size, b.size)
    a, b = a[:n], b[:n]
    af, bf = a.view(np.float16), b.view(np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        want_add = (af + bf).view(np.uint16)
        want_mul = (af * bf).view(np.uint16)
    add = np.vectorize(orc.lib.orc_half_add, otypes=[np.uint16])(a[:60000], b[:60000])
    mul = np.vectorize(orc.lib.orc_half_mul, otypes=[np.uint16])(a[:60000], b[:60000])
    ok = ~np.isnan(want_add[:60000].view(np.float16))
    assert np.array_equal(add[ok], want_add[:60000][ok])
    ok = ~np.isnan(want_mul[:60000].view(np.float16))
    assert np.array_equal(mul[ok], want_mul[:60000][ok])


def test_fma_exact(orc):
    rng = np.random.default_rng(5)
    a = _random_halves(rng, 9000)
    b = _random_halves(rng, 9000)
    c = _random_halves(rng, 9000)
    n = min(a.size, b.size, c.size)
    cases = list(zip(a[:n].tolist(), b[:n].tolist(), c[:n].tolist()))
    # the SGD shape: small lr times a gradient added to a parameter of comparable size
    lr = int(np.float16(0.01).view(np.uint16))
    for _ in range(4000):
        g = int(np.float16(rng.standard_normal() * 0.3).view(np.uint16))
        p = int(np.float16(rng.standard_normal() * 0.05).view(np.uint16))
        cases.append((lr, g, p))
    # directed: product exactly on a tie of the addend's grid, and a hair off it
    cases += [(0x3C00, 0x1000, 0x3C00), (0x3C01, 0x1000, 0x3C00), (0x0001, 0x3C00, 0x3C00), (0x0400, 0x0400, 0x3C00),
              (0x7BFF, 0x3C00, 0x7BFF), (0x3800, 0x0001, 0x0000), (0x3800, 0x0001, 0x0001), (0x3800, 0x0003, 0x8001)]
    for x, y, z in cases:
        exact = half_bits_to_fraction(x) * half_bits_to_fraction(y) + half_bits_to_fraction(z)
        got = orc.lib.orc_half_fma(x, y, z)
        if exact == 0:
            assert got & 0x7FFF == 0
        else:
            assert got == round_fraction_to_half(exact), (hex(x), hex(y), hex(z), hex(got))


def test_f16c_and_software_builds_agree_on_updates(orc, orc_soft):
    """The F16C build and the software build must give identical MASCOT half/half and MPT updates."""
    rng = np.random.default_rng(6)
    for k in (64, 128):
        for _ in range(200):
            p = (rng.standard_normal(k) * 0.1).astype(np.float32)
            q = (rng.standard_normal(k) * 0.1).astype(np.float32)
            r = float(rng.integers(1, 6))
            outs = []
            for o in (orc, orc_soft):
                ph, qh = o.f2h(p), o.f2h(q)
                gp = np.zeros(k, np.float32)
                gq = np.zeros(k, np.float32)
                import ctypes as C
                npv, nqv = C.c_float(), C.c_float()
                o.lib.orc_mascot_update(k, ph.ctypes.data, 0, qh.ctypes.data, 0, r, 0.01, 0.05,
                                        gp.ctypes.data, gq.ctypes.data, C.byref(npv), C.byref(nqv))
                pm, qm = p.copy(), q.copy()
                o.lib.orc_mpt_update(k, pm.ctypes.data, qm.ctypes.data, r, 0.01, o.lib.orc_float2half(0.05 * 1000), 1000.0)
                outs.append((ph, qh, gp, gq, npv.value, nqv.value, pm, qm))
            for x, y in zip(*outs):
                assert np.array_equal(np.asarray(x), np.asarray(y))


def test_golden_half_vectors(orc, orc_soft):
    """tests/golden/half_vectors.npz (numpy float16 + exact rational arithmetic, see make_half_vectors.py): the
    checker's conversion and its add / sub / mul / fma, in the F16C build and in the software build."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "half_vectors.npz"))
    for o in (orc, orc_soft):
        assert np.array_equal(o.f2h(g["f2h_in"]), g["f2h_out"])
        for name, key in (("orc_half_mul", "mul"), ("orc_half_add", "add"), ("orc_half_sub", "sub")):
            got = np.vectorize(getattr(o.lib, name), otypes=[np.uint16])(g["a"], g["b"])
            assert np.array_equal(got, g[key]), name
        got = np.vectorize(o.lib.orc_half_fma, otypes=[np.uint16])(g["a"], g["b"], g["c"])
        assert np.array_equal(got, g["fma"])
