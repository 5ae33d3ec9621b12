// Device-side pieces of the activation quantisers, shared by the quantiser kernels (actquant.hip) and by the
// streaming matmul kernels that quantise their activations on the fly: whoever uses them produces the same codes
// and scales bit for bit.
// (reference: gemlite/quant_utils.py:467-539 per token, :2005-2135 and :697-705 MXFP4.)
#pragma once
#include "common.hpp"

namespace gla {

// float -> OCP e4m3fn byte, round to nearest even, input already clamped to +-448
__device__ __forceinline__ uint32_t f32_to_fp8_pair(float a, float b) {
    // v_cvt_pk_fp8_f32 packs two conversions into the low 16 bits
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

// v / s, correctly rounded, for v that came from a 16-bit float and s = max(amax / qmax, 1e-6) of such values:
// q = v * r with r the correctly rounded 1 / s, one residual e = v - q s (exact in the fused multiply-add)
// and q + e r.  That this equals the IEEE quotient bit for bit for every such pair (65536 x 32768 per input
// type and qmax; quotients below 2^-20, which become the code 0 either way, only have to stay that small)
// is checked exhaustively on the CPU by tests/test_division.py; the sign is copied from v because the
// correction step turns a quotient of -0 into +0.  One division per row instead of one per element.
__device__ __forceinline__ float div_by_row_scale(float v, float s, float r) {
    const float q = v * r;
    const float e = __builtin_fmaf(-q, s, v);
    const float c = __builtin_fmaf(e, r, q);
    return __builtin_bit_cast(float, (__builtin_bit_cast(uint32_t, c) & 0x7fffffffu) | (__builtin_bit_cast(uint32_t, v) & 0x80000000u));
}

template <bool TO_INT8, bool FROM16>
__device__ __forceinline__ uint2 quantise8(float (&v)[8], float s) {
    const float qmax = TO_INT8 ? 127.0f : 448.0f;
    const float qmin = TO_INT8 ? -128.0f : -448.0f;
    uint32_t lo = 0, hi = 0;
    const float r = 1.0f / s;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(FROM16 ? div_by_row_scale(v[j], s, r) : v[j] / s, qmin), qmax);
    if constexpr (TO_INT8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            lo |= ((uint32_t)(int)floorf(v[j] + 0.5f) & 0xffu) << (8 * j);
            hi |= ((uint32_t)(int)floorf(v[4 + j] + 0.5f) & 0xffu) << (8 * j);
        }
    } else {
        lo = f32_to_fp8_pair(v[0], v[1]) | (f32_to_fp8_pair(v[2], v[3]) << 16);
        hi = f32_to_fp8_pair(v[4], v[5]) | (f32_to_fp8_pair(v[6], v[7]) << 16);
    }
    return make_uint2(lo, hi);
}

// e2m1 code of v (already divided by the block scale): ties toward zero, -0 keeps its sign bit
// only through the v >= 0 test, exactly like the reference's threshold path.
__device__ __forceinline__ uint32_t e2m1_code(float v) {
    const float a = fabsf(v);
    uint32_t idx = (a > 0.25f) + (a > 0.75f) + (a > 1.25f) + (a > 1.75f) + (a > 2.5f) + (a > 3.5f) + (a > 5.0f);
    return (v >= 0.0f) ? idx : (idx + 8u);
}

// e8m0 byte of amax / qmax (qmax 6 for e2m1, 448 for e4m3) = biased exponent of the quotient, plus one unless the
// quotient is a power of two (reference: the exponent of the scale is rounded up), clamped to 97 .. 254.
// qmax = 1.5 * 2^2 or 1.75 * 2^8, so the quotient's exponent and whether its mantissa is zero follow from amax's own
// fields without a division: significand above qmax's -> exponent(amax) - log2 part + 1, equal or below -> one less
// (equal: an exact power of two; below: the quotient drops a binade and is never a power of two).
template <bool FP8OUT>
__device__ __forceinline__ uint32_t e8m0_of_amax(float amax) {
    const uint32_t abits = __builtin_bit_cast(uint32_t, amax);
    const int ea = (int)(abits >> 23), ma = (int)(abits & 0x7fffffu);
    int ei = ea - (FP8OUT ? 8 : 2) + (ma > (FP8OUT ? 0x600000 : 0x400000) ? 1 : 0);
    if (ea == 255) ei = 254;  // an infinite amax: inf / qmax has exponent 255, clamped below
    ei = ei > 254 ? 254 : ei;
    ei = ei < 97 ? 97 : ei;
    return (uint32_t)ei;
}

// Eight values of a 32-group whose e8m0 byte is e -> eight e2m1 codes, value j in bits 4j .. 4j+3.
// The hardware conversion divides by the block scale and rounds to nearest even; the reference counts the
// thresholds strictly below |x / s|, i.e. rounds ties toward zero, and gives -0.0 the code 0.  The two differ at
// exact ties whose upper neighbour is the even one (0.75, 1.75 and 3.5 times the scale: those go one ulp toward
// zero first) and at -0.0 (x + 0.0 is +0.0 for both zeros and x otherwise).  An input that is not a number takes
// the reference's route.  FROM16: the values came from fp16 / bf16.
template <bool FROM16>
__device__ __forceinline__ uint32_t mxfp4_pack8(const float (&v)[8], uint32_t e) {
    const int down = 127 - (int)e;
    const float sc = __builtin_bit_cast(float, e << 23);
    bool odd = false;
    float w[8];
    if constexpr (!FROM16) {
        const uint32_t shift = (e - 127u) << 23;
        const uint32_t t1 = 0x3f400000u + shift, t2 = 0x3fe00000u + shift, t3 = 0x40600000u + shift;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float z = v[j] + 0.0f;
            const uint32_t zb = __builtin_bit_cast(uint32_t, z), mag = zb & 0x7fffffffu;
            const bool tie = mag == t1 || mag == t2 || mag == t3;
            w[j] = __builtin_bit_cast(float, zb - (tie ? 1u : 0u));
            odd |= mag > 0x7f800000u;
        }
    } else {
        // 16-bit inputs have at most 11 significant bits, so a value that is not exactly on a tie is at least
        // 2^-12 of itself away from it: scaling everything by 1 - 2^-16 moves the ties below their midpoint (they
        // round toward zero, as the reference has them) and nothing else across one.  The fused add of +0.0 turns
        // -0.0 into +0.0.  Not-a-number and infinite inputs make the second sum a NaN and take the reference's route.
        float chk = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            w[j] = __builtin_fmaf(v[j], 0.9999847412109375f, 0.0f);
            chk = __builtin_fmaf(v[j], 0.0f, chk);
        }
        odd = chk != chk;
    }
    uint32_t packed = 0;
    if (__builtin_expect(!odd, 1)) {
        packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, w[0], w[1], sc, 0);
        packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, w[2], w[3], sc, 1);
        packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, w[4], w[5], sc, 2);
        packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, w[6], w[7], sc, 3);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) packed |= e2m1_code(__builtin_ldexpf(v[j], down)) << (4 * j);
    }
    return packed;
}

}  // namespace gla
