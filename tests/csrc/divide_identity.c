/* Brute-force check of the identity the quantization kernel relies on
 * (flagattention_amd/csrc/quant.hip): with r = RN(1/s), q0 = x*r and two residual corrections
 * q <- fma(fma(-q, s, x), r, q), the result is the correctly rounded x/s in IEEE fp32.
 * Usage: divide_identity <scales swept over every significand of x> [<scales swept over sampled significands>];
 * exits non-zero when any quotient differs. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
static inline float asf(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t asu(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float corrected(float x, float s, float r) {
    float q = x * r;
    q = fmaf(fmaf(-q, s, x), r, q);
    q = fmaf(fmaf(-q, s, x), r, q);
    return q;
}
int main(int argc, char** argv) {
    const int nscale = argc > 1 ? atoi(argv[1]) : 12;
    static const uint32_t special[] = {0, 0x7ffffe, 1, 0x400000, 0x3fffff, 0x555555, 0x2aaaaa, 0x7ffffd};
    uint64_t bad = 0, total = 0;
    uint32_t seed = 12345;
    for (int si = 0; si < nscale; si++) {
        seed = seed * 1664525u + 1013904223u;
        uint32_t mant = si < 8 ? special[si] : ((seed >> 9) & 0x7fffff);
        if (mant == 0x7fffff) mant = 0x7ffffe; /* the kernel sends an all-ones significand to the hardware divide */
        const int ex = 127 + ((int)((seed >> 3) % 81) - 40);
        const float s = asf(((uint32_t)ex << 23) | mant), r = 1.0f / s;
        for (uint32_t m = 0; m < (1u << 23); m += 1) {
            const int e2 = ex - 2 + (int)(m % 9); /* |x/s| in [0.25, 128): the nine binades that reach the int8 range */
            const float x = asf(((uint32_t)e2 << 23) | m);
            const float exact = x / s;
            if (fabsf(exact) > 127.5f) continue;
            bad += asu(corrected(x, s, r)) != asu(exact);
            bad += asu(corrected(-x, s, r)) != asu(-exact);
            total += 2;
        }
    }
    /* many more scales (random significand and exponent over the kernel's fast range 2^-60 .. 2^60), each against
     * a random sample of x: 8192 significands in each of the nine binades */
    const int nsampled = argc > 2 ? atoi(argv[2]) : 0;
    for (int si = 0; si < nsampled; si++) {
        seed = seed * 1664525u + 1013904223u;
        uint32_t mant = (seed >> 9) & 0x7fffff;
        if (mant == 0x7fffff) mant = 0x7ffffe;
        seed = seed * 1664525u + 1013904223u;
        const int ex = 127 + ((int)((seed >> 8) % 119) - 59);
        const float s = asf(((uint32_t)ex << 23) | mant), r = 1.0f / s;
        for (int i = 0; i < 9 * 8192; i++) {
            seed = seed * 1664525u + 1013904223u;
            const uint32_t m = (seed >> 9) & 0x7fffff;
            const int e2 = ex - 2 + i % 9;
            if (e2 <= 0 || e2 >= 255) continue;
            const float x = asf(((uint32_t)e2 << 23) | m);
            const float exact = x / s;
            if (fabsf(exact) > 127.5f) continue;
            bad += asu(corrected(x, s, r)) != asu(exact);
            bad += asu(corrected(-x, s, r)) != asu(-exact);
            total += 2;
        }
    }
    printf("%llu quotients, %llu mismatches\n", (unsigned long long)total, (unsigned long long)bad);
    return bad != 0;
}
