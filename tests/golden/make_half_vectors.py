"""Writes half_vectors.npz: known-answer vectors for binary16 conversion and arithmetic, computed with numpy's
float16 (IEEE-754 binary16, round-to-nearest-even) and exact rational arithmetic -- not with the checker under
oracle/ and not with the HIP library, both of which the tests hold against these vectors.

    python tests/golden/make_half_vectors.py

The reference ships no vectors of its own for this arithmetic (it relies on CUDA's __float2half_rn, __half2float
and the half operators), so the fixture pins the published IEEE behaviour those intrinsics implement."""
import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def round_to_half(x: Fraction) -> np.uint16:
    """Exact round-to-nearest-even of a rational to binary16, by integer arithmetic only."""
    if x == 0:
        return np.uint16(0)
    sign = 0x8000 if x < 0 else 0
    x = abs(x)
    e = 0
    while x >= 2:
        x /= 2; e += 1
    while x < 1:
        x *= 2; e -= 1
    if e < -14:                                    # subnormal: scale to units of 2^-24
        x = x * Fraction(2) ** (e + 24); e_bits = 0
        m = x.numerator // x.denominator
        r = x - m
        if r > Fraction(1, 2) or (r == Fraction(1, 2) and m & 1):
            m += 1
        return np.uint16(sign | m)                 # m == 1024 carries into the smallest normal by itself
    m_full = (x - 1) * 1024
    m = m_full.numerator // m_full.denominator
    r = m_full - m
    if r > Fraction(1, 2) or (r == Fraction(1, 2) and m & 1):
        m += 1
    if m == 1024:
        m = 0; e += 1
    if e > 15:
        return np.uint16(sign | 0x7C00)
    return np.uint16(sign | ((e + 15) << 10) | m)


def main():
    rng = np.random.default_rng(20211207)
    # conversion: every midpoint between adjacent halves, its float neighbours, range ends, subnormals, specials
    halves = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = halves.view(np.float16).astype(np.float64)
    hi = (halves + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0                               # the rounding boundary above the largest finite half
    mid = ((lo + hi) / 2).astype(np.float32)       # exactly representable in binary32
    cand = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                           np.array([0.0, 65504.0, 65519.9, 65520.0, 1e-8, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                                     np.inf, 3.4e38], np.float32),
                           rng.standard_normal(4096).astype(np.float32) * np.float32(0.3)])
    cand = np.concatenate([cand, -cand]).astype(np.float32)
    f2h_in = cand
    with np.errstate(over="ignore"):
        f2h_out = cand.astype(np.float16).view(np.uint16)
    # cross-check numpy against the integer routine on the finite ones
    for v, want in zip(f2h_in[::97], f2h_out[::97]):
        if np.isfinite(v):
            assert round_to_half(Fraction(float(v))) == want, (v, want)
    # arithmetic: a*b, a+b, a-b, fma(a,b,c), each rounded once
    n = 6000
    a = (rng.standard_normal(n) * 0.5).astype(np.float16)
    b = (rng.standard_normal(n) * 2.0).astype(np.float16)
    c = (rng.standard_normal(n) * 0.01).astype(np.float16)
    a[:8] = np.array([6.1e-5, 6.0e-8, 65504, -65504, 1.0, 0.0999755859375, 0.33325195, 1024], np.float16)
    b[:8] = np.array([0.5, 0.5, 2.0, 2.0, 1.0009765625, 10.0, 3.0, 0.00048828125], np.float16)
    fa, fb, fc = ([Fraction(float(x)) for x in v] for v in (a, b, c))
    mul = np.array([round_to_half(x * y) for x, y in zip(fa, fb)], np.uint16)
    add = np.array([round_to_half(x + y) for x, y in zip(fa, fb)], np.uint16)
    sub = np.array([round_to_half(x - y) for x, y in zip(fa, fb)], np.uint16)
    fma = np.array([round_to_half(x * y + z) for x, y, z in zip(fa, fb, fc)], np.uint16)
    np.savez_compressed(os.path.join(HERE, "half_vectors.npz"), f2h_in=f2h_in, f2h_out=f2h_out,
                        a=a.view(np.uint16), b=b.view(np.uint16), c=c.view(np.uint16), mul=mul, add=add, sub=sub, fma=fma)
    print("wrote half_vectors.npz:", f2h_in.size, "conversions,", n, "operand triples")


if __name__ == "__main__":
    main()
