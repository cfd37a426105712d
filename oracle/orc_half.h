/*
 * TEST INFRASTRUCTURE ONLY -- CPU checker, never part of the shipped path.
 *
 * IEEE-754 binary16 arithmetic in software, restating what the reference gets
 * from CUDA's __half type (cuda_fp16.h): __float2half_rn / __float2half
 * (round-to-nearest-even, overflow -> inf, subnormals kept), __half2float
 * (exact), operator+ - * on __half (each result rounded once to binary16) and
 * __hfma (one rounding of a*b+c).  Used by mascot/mascot_sgd_kernel.h:79-229
 * and mpt/mpt_sgd_kernel.h:24-91 of the reference.
 *
 * Pinning (see tests/test_oracle_half.py): conversions are checked
 * exhaustively against numpy.float16 and against the host's F16C unit; add,
 * sub, mul and fma are checked against exact rational arithmetic rounded by an
 * independent integer routine.
 */
#ifndef ORC_HALF_H
#define ORC_HALF_H
#include <stdint.h>
#include <string.h>
#include <math.h>

typedef uint16_t orc_half; /* raw binary16 bits */

static inline uint32_t orc_f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float orc_bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint64_t orc_f64_bits(double f) { uint64_t u; memcpy(&u, &f, 8); return u; }
static inline double orc_bits_f64(uint64_t u) { double f; memcpy(&f, &u, 8); return f; }

/* binary32 -> binary16, round to nearest even (__float2half_rn, model_init.cu:51-54,103). */
static inline orc_half orc_f2h(float f)
{
    uint32_t x = orc_f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) {                 /* inf or NaN */
        if (ax > 0x7f800000u) return (orc_half)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (orc_half)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) return (orc_half)(sign | 0x7c00u);  /* >= 65520 rounds to inf */
    if (ax < 0x38800000u) {                  /* below 2^-14: binary16 subnormal or zero */
        if (ax < 0x33000000u) return (orc_half)sign;           /* < 2^-25 */
        uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - (ax >> 23);  /* 14..24 */
        uint32_t q = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (orc_half)(sign | q);
    }
    uint32_t h = (((ax >> 23) - 112u) << 10) | ((ax & 0x7fffffu) >> 13);
    uint32_t rem = ax & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (orc_half)(sign | h);
}

/* binary16 -> binary32, exact (__half2float). */
static inline float orc_h2f(orc_half h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0x1fu) return orc_bits_f32(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        if (m == 0) return orc_bits_f32(sign);
        /* subnormal: m * 2^-24 */
        float v = (float)m * 5.9604644775390625e-08f;
        return (sign ? -v : v);
    }
    return orc_bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* binary64 -> binary16 with a single rounding (never through binary32). */
static inline orc_half orc_d2h(double d)
{
    uint64_t x = orc_f64_bits(d);
    uint32_t sign = (uint32_t)((x >> 48) & 0x8000u);
    uint64_t ax = x & 0x7fffffffffffffffull;
    uint32_t e = (uint32_t)(ax >> 52);
    if (e == 0x7ffu) {
        if (ax > 0x7ff0000000000000ull) return (orc_half)(sign | 0x7e00u);
        return (orc_half)(sign | 0x7c00u);
    }
    if (fabs(d) >= 65520.0) return (orc_half)(sign | 0x7c00u);
    if (e < 1023u - 25u) return (orc_half)sign;          /* |d| < 2^-25 */
    uint64_t mant = (ax & 0xfffffffffffffull) | 0x10000000000000ull;
    uint32_t shift;
    uint32_t h;
    if (e >= 1023u - 14u) { shift = 42u; h = ((e - 1008u) << 10); mant &= 0xfffffffffffffull; }
    else { shift = 42u + (1009u - e); h = 0; }
    uint64_t q = mant >> shift;
    uint64_t rem = mant & ((1ull << shift) - 1ull);
    uint64_t half = 1ull << (shift - 1u);
    h += (uint32_t)q;
    if (rem > half || (rem == half && (h & 1u))) h++;
    return (orc_half)(sign | h);
}

/* operator+, -, * on __half: exact result rounded once.  binary32 holds the
 * exact product (22 bits) and, for sums, 24 >= 2*11+2 bits make the double
 * rounding through binary32 innocuous (Figueroa); done in binary64 anyway so
 * that the sum itself is exact. */
static inline orc_half orc_hadd(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) + (double)orc_h2f(b)); }
static inline orc_half orc_hsub(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) - (double)orc_h2f(b)); }
static inline orc_half orc_hmul(orc_half a, orc_half b) { return orc_d2h((double)orc_h2f(a) * (double)orc_h2f(b)); }

/* __hfma(a,b,c): round(a*b+c) once.  The product is exact in binary64; the
 * sum is formed with round-to-odd (TwoSum error term) so that the final
 * rounding to binary16 sees a sticky bit and cannot double-round. */
static inline orc_half orc_hfma(orc_half a, orc_half b, orc_half c)
{
    double p = (double)orc_h2f(a) * (double)orc_h2f(b);
    double cc = (double)orc_h2f(c);
    double s = p + cc;
    if (isfinite(s)) {
        double bb = s - p;
        double err = (p - (s - bb)) + (cc - bb);
        if (err != 0.0) {
            uint64_t sb = orc_f64_bits(s);
            /* s is RN(exact); exact = s + err.  Truncate toward zero, then set the LSB. */
            int s_neg = (s < 0.0) || (s == 0.0 && err < 0.0);
            int err_away = s_neg ? (err < 0.0) : (err > 0.0); /* exact lies further from zero than s */
            if (s == 0.0) { sb = orc_f64_bits(err); }      /* cannot happen for finite halves, kept for safety */
            else if (!err_away) sb -= 1;                    /* step one ulp toward zero */
            sb |= 1ull;
            s = orc_bits_f64(sb);
        }
    }
    return orc_d2h(s);
}

#endif
