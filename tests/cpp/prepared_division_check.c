/* Host check of the division that the kernels use for a Div<float..> of a chain's tail (include/fk/exec/kernels.h,
 * prepared_divide): with r = RN(1 / d) and rl = RN(1 / d - r) from the host,
 *     q = fma(x, r, x * rl);  q = fma(fma(-d, q, x), r, q)
 * must be the correctly rounded x / d for every x in [2^-40, 2^40].  Scaling x by a power of two scales every
 * intermediate value exactly, so all 2^23 significands of x at one exponent cover all x of the range; the ends of the
 * range and both signs are run as well.  Divisors: the ones of the benchmark chains, awkward significands, the ends of the
 * divisor range, and seeded random ones.
 * usage: prepared_division_check <number of divisors>; prints "mismatches 0" and returns 0 when all agree. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float short_division(float x, float d, float r, float rl) {
    float q = fmaf(x, r, x * rl);
    return fmaf(fmaf(-d, q, x), r, q);
}
static uint64_t splitmix(uint64_t* s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
int main(int argc, char** argv) {
    const int want = argc > 1 ? atoi(argv[1]) : 48;
    float ds[1024];
    int nd = 0;
    const float fixed[] = { 255.f, 0.229f, 0.224f, 0.225f, 3.f, 6.f, 7.f, 1.f / 3.f, -7.f, 9.09494702e-13f, 1.09951163e+12f, 1.99999988f,
                            1.00000012f, 0.5f, 127.5f, 65535.f, 1023.f, 0.485f, 58.395f, 57.12f, 57.375f };
    for (unsigned i = 0; i < sizeof(fixed) / 4 && nd < want; ++i) ds[nd++] = fixed[i];
    uint64_t s = 7;
    while (nd < want && nd < 1024) {
        uint32_t b = (uint32_t)splitmix(&s);
        const uint32_t e = 127 - 40 + (uint32_t)(splitmix(&s) % 80);
        b = (b & 0x807fffffu) | (e << 23);
        memcpy(&ds[nd++], &b, 4);
    }
    long bad = 0;
    for (int k = 0; k < nd; ++k) {
        const volatile float dv = ds[k];
        const float d = dv, r = 1.0f / dv, rl = (float)(1.0 / (double)d - (double)r);
        long b = 0;
#pragma omp parallel for reduction(+ : b)
        for (uint32_t m = 0; m < (1u << 23); ++m) {
            const uint32_t exps[3] = { 127, 127 - 40, 127 + 39 };
            for (int e = 0; e < 3; ++e) {
                for (uint32_t sign = 0; sign < 2; ++sign) {
                    const uint32_t bits = m | (exps[e] << 23) | (sign << 31);
                    float x;
                    memcpy(&x, &bits, 4);
                    const volatile float xv = x;
                    const float quotient = xv / dv, got = short_division(x, d, r, rl);
                    if (memcmp(&quotient, &got, 4) != 0) ++b;
                }
            }
        }
        if (b != 0) printf("d = %.9g: %ld mismatches\n", (double)d, b);
        bad += b;
    }
    printf("divisors %d, mismatches %ld\n", nd, bad);
    return bad != 0;
}
