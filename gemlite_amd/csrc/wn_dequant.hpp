// Dequantisation of 32-bit packed codes in registers, shared by the tiled packed-weight GEMM (gemm_wn.hip) and the
// mid-batch kernel (wn_mid.hip).  Reference: gemlite/triton_kernels/utils.py:73-105 (the five W_group_mode forms).
#pragma once

#include "common.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Interleave two runs of 4 consecutive 16-bit values (lo0:lo1 and hi0:hi1) so that register r
// holds (lo[r], hi[r]): the K-slot order of the unpacked B operand.
__device__ __forceinline__ u32x4 pair_order(uint32_t lo0, uint32_t lo1, uint32_t hi0, uint32_t hi1) {
    u32x4 o;
    o.x = __builtin_amdgcn_perm(hi0, lo0, 0x05040100u);
    o.y = __builtin_amdgcn_perm(hi0, lo0, 0x07060302u);
    o.z = __builtin_amdgcn_perm(hi1, lo1, 0x05040100u);
    o.w = __builtin_amdgcn_perm(hi1, lo1, 0x07060302u);
    return o;
}

// Per-column dequant constants of one quantisation group.
template <bool BF16>
struct ColMeta;
template <>
struct ColMeta<false> {
    half2_t s, z;  // (s, s) and (z', z') in fp16
};
template <>
struct ColMeta<true> {
    float s, z;  // s and z' - 128 s in fp32: the offset of the unpacking trick is folded into the constant
    uint32_t lut01, lut23;  // 2-bit codes: the four dequantised values of the group as bf16 pairs (w0, w1), (w2, w3)
};

// OFF: the offset the unpacking leaves on the codes in the fp32 path (128, or 0 for byte codes)
template <bool BF16, int OFF = 128>
__device__ __forceinline__ ColMeta<BF16> make_meta(float s, float zp) {
    ColMeta<BF16> m;
    if constexpr (BF16) {
        m.s = s;
        m.z = __builtin_fmaf(-(float)OFF, s, zp);
    } else {
        m.s = half2_t{(half_t)s, (half_t)s};
        m.z = half2_t{(half_t)zp, (half_t)zp};
    }
    return m;
}

__device__ __forceinline__ float fold_zero(float s, float z, int wgm) {
    switch (wgm) {
        case GLA_WGM_SHIFT: return -z;
        case GLA_WGM_SHIFT_SCALE: return -z * s;
        case GLA_WGM_FMA: return z;
        default: return 0.0f;
    }
}

// pair register holding (OFF + q_lo, OFF + q_hi) -> dequantised pair in the activation type
template <bool BF16>
__device__ __forceinline__ uint32_t dequant_pair(uint32_t t, const ColMeta<BF16>& m, float off_lo = 1024.0f, float off_hi = 1024.0f) {
    if constexpr (BF16) {
        // bf16 bits are the top half of an fp32, where 128 + q is exact too; (128 + q) s + (z' - 128 s)
        // in fp32, then one hardware round-to-nearest-even conversion of the pair
        const float lo = __builtin_bit_cast(float, t << 16);
        const float hi = __builtin_bit_cast(float, t & 0xffff0000u);
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 w = {__builtin_fmaf(lo, m.s, m.z), __builtin_fmaf(hi, m.s, m.z)};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(w, bf16x2_t));
    } else {
        half2_t q = __builtin_bit_cast(half2_t, t) - half2_t{(half_t)off_lo, (half_t)off_hi};
        half2_t w = __builtin_elementwise_fma(q, m.s, m.z);
        return __builtin_bit_cast(uint32_t, w);
    }
}

}  // namespace

}  // namespace gla
