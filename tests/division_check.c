/* Exhaustive check of the per-token activation quantiser's division (test infrastructure, CPU only).
 *
 * The kernel divides every value of a row by the row's scale s = max(amax / qmax, 1e-6) (reference:
 * gemlite/quant_utils.py:467-539, `x / scales`).  For inputs that came from a 16-bit float it computes the
 * quotient as q = v r, e = fma(-q, s, v), q + e r with r = 1 / s correctly rounded.  This program runs that
 * sequence and the IEEE division over every pair the kernel can meet -- v any finite value of the 16-bit type,
 * amax any non-negative finite value of it with |v| <= amax -- and counts the pairs whose results differ in
 * any bit (the sign of a zero quotient is taken from v in both; quotients below 2^-20, which quantise to zero,
 * are only required to stay that small).
 *
 *   usage: division_check <type: 0 = fp16, 1 = bf16> <qmax: 127 or 448>      prints: <pairs> <mismatches>
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static float bits_to_float(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static uint32_t float_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

static float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31, man = h & 1023;
    if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
    if (exp == 0) return (sign ? -1.0f : 1.0f) * ldexpf((float)man, -24);
    return bits_to_float(sign | ((exp + 112) << 23) | (man << 13));
}

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    const int bf16 = atoi(argv[1]);
    const float qmax = (float)atof(argv[2]);
    static float val[65536];
    for (int i = 0; i < 65536; ++i) val[i] = bf16 ? bits_to_float((uint32_t)i << 16) : half_to_float((uint16_t)i);
    long long pairs = 0, bad = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : pairs, bad)
    for (int a = 0; a < 32768; ++a) {          /* amax: the non-negative half of the code space */
        const float amax = val[a];
        if (!(amax <= 3.4e38f)) continue;      /* infinities and NaNs */
        const float s = fmaxf(amax / qmax, 1e-6f);
        const float r = 1.0f / s;
        for (int i = 0; i < 65536; ++i) {
            const float v = val[i];
            if (!(fabsf(v) <= amax)) continue;
            const float q = v * r;
            const float e = fmaf(-q, s, v);
            const float c = fmaf(e, r, q);
            const uint32_t fast = (float_to_bits(c) & 0x7fffffffu) | (float_to_bits(v) & 0x80000000u);
            const uint32_t ieee = float_to_bits(v / s);
            ++pairs;
            /* quotients below 2^-20 become the code 0 whatever their last bits (the smallest rounding boundary
               of either output type is 2^-10): there the residual can leave the range of normal numbers and the
               two need not agree bit for bit, only in being that small and in sign */
            if (fabsf(v / s) < 9.5367431640625e-07f)
                bad += !(fabsf(bits_to_float(fast)) < 1.9073486328125e-06f) || ((fast ^ ieee) >> 31);
            else
                bad += fast != ieee;
        }
    }
    printf("%lld %lld\n", pairs, bad);
    return 0;
}
