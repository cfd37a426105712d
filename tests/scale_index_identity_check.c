/* The MuPPET scale index from the bits of x against its definition, floor(log2f(bound / x)) converted to unsigned with
 * saturation (muppet/muppet_sgd_kernel.h:7-18): every exponent, mantissas spread over the whole range and dense around
 * the threshold, for the two bounds of every bit width.  Lanes within 64 ulps of the threshold mantissa are excluded
 * (the kernel evaluates the definition itself there).  Prints the number of disagreements. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static uint32_t f2u_sat(float f) { if (!(f > 0.0f)) return 0u; if (f >= 4294967296.0f) return 0xffffffffu; return (uint32_t)f; }
static uint32_t by_definition(float bound, float x) { return f2u_sat(floorf(log2f(fabsf(bound / x)))); }
static int by_bits(unsigned bitwidth, int upper, float x, uint32_t* out)
{
    const uint32_t eb = upper ? bitwidth - 1u : bitwidth - 2u;
    const uint32_t t_mant = upper ? (0x800000u >> bitwidth) : 0x800000u - (0x800000u >> (bitwidth - 1u));
    uint32_t xb; memcpy(&xb, &x, 4); xb &= 0x7fffffffu;
    const uint32_t mant = xb & 0x7fffffu;
    const int idx = (int)(eb + 127u) - (int)(xb >> 23) - (mant > t_mant ? 1 : 0);
    if (mant - t_mant + 64u <= 128u) return 0;                      /* near the threshold: not decided from the bits */
    *out = xb == 0u ? 0xffffffffu : (idx < 0 ? 0u : (idx >= 128 ? 0xffffffffu : (uint32_t)idx));
    return 1;
}
int main(void)
{
    const unsigned widths[4] = {8, 12, 14, 16};
    unsigned long long bad = 0, checked = 0;
    for (int w = 0; w < 4; w++)
        for (int upper = 0; upper < 2; upper++) {
            const float val = (float)(1 << (widths[w] - 1));
            const float bound = upper ? (-val) - 0.5f : (val - 1) + 0.5f;
            const uint32_t t_mant = upper ? (0x800000u >> widths[w]) : 0x800000u - (0x800000u >> (widths[w] - 1u));
            for (uint32_t ex = 0; ex < 256; ex++) {
                for (uint32_t step = 0; step < 40000; step++) {
                    uint32_t mant;
                    if (step < 20000) mant = (uint32_t)(((uint64_t)step * 0x800000u) / 20000u + (step * 2654435761u >> 25)) & 0x7fffffu;
                    else mant = (t_mant + (step - 30000u)) & 0x7fffffu;        /* -10000 .. +9999 ulps around the threshold */
                    for (int sign = 0; sign < 2; sign++) {
                        const uint32_t b = ((uint32_t)sign << 31) | (ex << 23) | mant;
                        float x; memcpy(&x, &b, 4);
                        uint32_t got;
                        if (!by_bits(widths[w], upper, x, &got)) continue;
                        checked++;
                        if (got != by_definition(bound, x)) { if (bad++ < 10) fprintf(stderr, "width %u upper %d x %a: bits %u definition %u\n", widths[w], upper, x, got, by_definition(bound, x)); }
                    }
                }
            }
        }
    if (checked < 100000000ull) { fprintf(stderr, "only %llu cases\n", checked); return 1; }
    printf("%llu\n", bad);
    return 0;
}
