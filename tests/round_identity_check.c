/* Exhaustive check of an identity the fixed-point update kernels rely on:
 *   roundf(x) == truncf(x + copysignf(0x1.fffffep-2f, x))   for every binary32 x that is not a NaN, bit for bit.
 * Built and run by tests/test_host_io.py (gcc -fopenmp); prints the number of mismatches. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

int main(void)
{
    unsigned long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long long i = 0; i < (1LL << 32); i++) {
        uint32_t b = (uint32_t)i, gb, wb;
        float x;
        memcpy(&x, &b, 4);
        if (x != x) continue;
        volatile float sum = x + copysignf(0x1.fffffep-2f, x);
        float got = truncf(sum), want = roundf(x);
        memcpy(&gb, &got, 4);
        memcpy(&wb, &want, 4);
        bad += gb != wb;
    }
    printf("%llu\n", bad);
    return 0;
}
