/* Exhaustive check of the arithmetic the int8 append uses for binary16 rows
 * (breccia_amd/csrc/quant_encode.hpp, codes8_f16_on_biased_reciprocal): for every block amax that
 * is a binary16 number above 2^-6, the scale the layout stores for it, and every binary16 x with
 * |x| <= amax (subnormal codes included, either sign),
 *
 *     low byte of bits(fmaf(x, r * (1 + 2^-21), 1.5 * 2^23))
 *
 * must be the code the rule defines, round-half-away(clamp(flush(x) / scale, +-127)) -- for the
 * correctly rounded reciprocal r of the scale and for r one ulp off either way (the hardware
 * reciprocal is good to one ulp).  Prints the number of pairs walked; exits 1 at the first
 * difference.  Host code only; test infrastructure.
 *
 * Build: gcc -O2 -fopenmp -ffp-contract=off i8h_f16_codes_exhaustive.c -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static float bits_f32(uint32_t b) {
    float x;
    memcpy(&x, &b, 4);
    return x;
}
static uint32_t f32_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return b;
}
/* exact value of a binary16 code (subnormals keep their value) */
static float half_value(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3ffu;
    if (e == 0) return (sign ? -1.0f : 1.0f) * (float)m * 0x1p-24f;
    if (e == 31) return bits_f32(sign | 0x7f800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}
/* f32 -> binary16, round to nearest even, for numbers in the normal binary16 range */
static uint32_t half_code_normal(float x) {
    const uint32_t b = f32_bits(x);
    const uint32_t sign = (b >> 16) & 0x8000u;
    int32_t e = (int32_t)((b >> 23) & 0xff) - 127;
    uint32_t m = (b & 0x7fffffu) | 0x800000u, q = m >> 13, rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q;
    if (q >= 2048u) {
        q >>= 1;
        ++e;
    }
    if (e > 15) return sign | 0x7c00u;
    return sign | (uint32_t)(e + 15) << 10 | (q & 0x3ffu);
}

int main(void) {
    const float tie_bias = 1.0f + 0x1p-21f, magic = 12582912.0f;
    unsigned long long pairs = 0;
    int bad = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : pairs)
    for (uint32_t ab = 0x2401u; ab <= 0x7bffu; ++ab) { /* amax codes: above 2^-6, finite */
        if (bad) continue;
        const float amax = half_value(ab);
        const float s0 = amax / 127.0f;
        if (!(fabsf(s0) >= 0x1p-14f)) continue; /* cannot happen above 2^-6; the rule would raise it */
        const uint32_t hb = half_code_normal(s0);
        if (hb == 0x7c00u) continue;
        const float sh = half_value(hb);
        const float r0 = 1.0f / sh;
        float rb[3];
        rb[0] = bits_f32(f32_bits(r0) - 1u) * tie_bias;
        rb[1] = r0 * tie_bias;
        rb[2] = bits_f32(f32_bits(r0) + 1u) * tie_bias;
        for (uint32_t xb = 0; xb <= ab; ++xb) {
            for (int neg = 0; neg < 2; ++neg) {
                const float x = neg ? -half_value(xb) : half_value(xb);
                const float xf = (xb & 0x7c00u) == 0 ? 0.0f : x; /* the load rule's flush */
                float t = xf / sh;
                if (!(t >= -127.0f)) t = -127.0f;
                if (t > 127.0f) t = 127.0f;
                const int want = (int)roundf(t);
                for (int k = 0; k < 3; ++k) {
                    const uint32_t y = f32_bits(fmaf(x, rb[k], magic));
                    const int got = (int)(int8_t)(y & 0xffu);
                    if (got != want) {
#pragma omp critical
                        {
                            if (!bad)
                                printf("MISMATCH amax %a scale %a x %a reciprocal %+d ulp: code %d, rule %d\n", amax,
                                       sh, x, k - 1, got, want);
                            bad = 1;
                        }
                    }
                }
                ++pairs;
            }
        }
    }
    printf("%llu (amax, x) pairs, 3 reciprocals each: %s\n", pairs, bad ? "FAILED" : "all codes equal the rule's");
    return bad;
}
