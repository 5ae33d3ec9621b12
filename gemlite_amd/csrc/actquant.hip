// Fused dynamic activation quantisation.
//
// per-token (reference: gemlite/quant_utils.py:467-539):
//   s = max(amax(|row|) / qmax, 1e-6); y = clamp(row / s, qmin, qmax);
//   int8 rounds with floor(y + 0.5) (reference: gemlite/quant_utils.py:289-296),
//   fp8 is the round-to-nearest-even e4m3fn cast of the clamped value.
// MXFP4 (reference: gemlite/quant_utils.py:2005-2135, :697-705):
//   per 32 values: e = clamp(exp(amax/6) + (mantissa != 0), 97, 254), s = 2^(e-127),
//   code = #{thresholds < |x/s|} over {.25,.75,1.25,1.75,2.5,3.5,5} (strict, so
//   ties round toward zero), +8 when x/s < 0; two codes per byte, even k low.
//
// Both kernels are HBM-bound: one read of x, one write of the codes.  A wave
// owns a row (per-token) or a run of 32-value groups (MXFP4); every lane moves
// 16 bytes per load.
#include "common.hpp"
#include "dispatch.hpp"
#include "actquant_device.hpp"

namespace gla {

namespace {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Load 8 consecutive elements starting at element index k (k % 8 == 0) as floats.
template <int XDT>
__device__ __forceinline__ void load8(const void* row, int k, float (&v)[8]) {
    if constexpr (XDT == GLA_DT_FP32) {
        const float4 a = ((const float4*)((const float*)row + k))[0];
        const float4 b = ((const float4*)((const float*)row + k))[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 raw = *(const uint4*)((const uint16_t*)row + k);
        const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (XDT == GLA_DT_FP16) {
                v[2 * i] = half_bits_to_float((uint16_t)(r[i] & 0xffffu));
                v[2 * i + 1] = half_bits_to_float((uint16_t)(r[i] >> 16));
            } else {
                v[2 * i] = bf16_bits_to_float((uint16_t)(r[i] & 0xffffu));
                v[2 * i + 1] = bf16_bits_to_float((uint16_t)(r[i] >> 16));
            }
        }
    }
}

// Raw 8-element chunk as loaded from memory (16 bytes for 16-bit types, 32 for fp32).
template <int XDT>
struct Raw8 {
    uint4 a;
};
template <>
struct Raw8<GLA_DT_FP32> {
    uint4 a, b;
};

// (plain loads: the part of a long row that a wave reads twice should stay in the L2 between the passes)
template <int XDT>
__device__ __forceinline__ Raw8<XDT> load_raw8_cached(const void* row, int k) {
    Raw8<XDT> r;
    if constexpr (XDT == GLA_DT_FP32) {
        r.a = ((const uint4*)((const float*)row + k))[0];
        r.b = ((const uint4*)((const float*)row + k))[1];
    } else {
        r.a = *(const uint4*)((const uint16_t*)row + k);
    }
    return r;
}

// (streaming loads: read once)
template <int XDT>
__device__ __forceinline__ Raw8<XDT> load_raw8(const void* row, int k) {
    Raw8<XDT> r;
    if constexpr (XDT == GLA_DT_FP32) {
        r.a = load_streaming_u4((const float*)row + k);
        r.b = load_streaming_u4((const float*)row + k + 4);
    } else {
        r.a = load_streaming_u4((const uint16_t*)row + k);
    }
    return r;
}

template <int XDT>
__device__ __forceinline__ void decode_raw8(const Raw8<XDT>& r, float (&v)[8]) {
    if constexpr (XDT == GLA_DT_FP32) {
        const uint32_t w[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = __builtin_bit_cast(float, w[i]);
    } else {
        const uint32_t w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (XDT == GLA_DT_FP16) {
                v[2 * i] = half_bits_to_float((uint16_t)(w[i] & 0xffffu));
                v[2 * i + 1] = half_bits_to_float((uint16_t)(w[i] >> 16));
            } else {
                v[2 * i] = bf16_bits_to_float((uint16_t)(w[i] & 0xffffu));
                v[2 * i + 1] = bf16_bits_to_float((uint16_t)(w[i] >> 16));
            }
        }
    }
}

// 8-element chunks a lane keeps in registers between the two passes
// (16-bit inputs: rows up to 64*8*16 = 8192 elements stay resident).
template <int XDT>
constexpr int row_cache() { return XDT == GLA_DT_FP32 ? 8 : 16; }

// One wave per row.  The amax pass keeps the raw row in registers; the part of a longer row that does not
// fit is read again (from L2) in the quantise pass.  (kRowsPerWave = 2, the loads of a wave's second row in
// flight under the divisions of its first, measured slower: M=4096, K=8192 31 against 28 us.)
constexpr int kRowsPerWave = 1;

template <int XDT, bool TO_INT8>
__global__ __launch_bounds__(256) void per_token_kernel(const void* __restrict__ x, int64_t xsm, int M, int K,
                                                        uint8_t* __restrict__ y, float* __restrict__ scales) {
    constexpr int RC = row_cache<XDT>();
    const int lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * kRowsPerWave;
    if (row0 >= M) return;
    const int chunks = K / 8;  // K % 8 == 0 enforced by the launcher

    Raw8<XDT> cache[kRowsPerWave][RC];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        // a row past the end repeats the last one (loaded, never reduced or stored)
        const int row = row0 + r < M ? row0 + r : M - 1;
        const char* xrow = (const char*)x + (int64_t)row * xsm * (XDT == GLA_DT_FP32 ? 4 : 2);
#pragma unroll
        for (int ci = 0; ci < RC; ++ci) {
            const int c = lane + ci * kWave;
            if (c < chunks) cache[r][ci] = load_raw8<XDT>(xrow, c * 8);
        }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int row = row0 + r;
        if (row >= M) break;
        const char* xrow = (const char*)x + (int64_t)row * xsm * (XDT == GLA_DT_FP32 ? 4 : 2);
        float amax = 0.0f;
#pragma unroll
        for (int ci = 0; ci < RC; ++ci) {
            const int c = lane + ci * kWave;
            if (c < chunks) {
                float v[8];
                decode_raw8<XDT>(cache[r][ci], v);
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
            }
        }
        for (int c = lane + RC * kWave; c < chunks; c += kWave) {
            float v[8];
            decode_raw8<XDT>(load_raw8_cached<XDT>(xrow, c * 8), v);
#pragma unroll
            for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
        }
        amax = wave_max(amax);
        const float qmax = TO_INT8 ? 127.0f : 448.0f;
        const float s = fmaxf(amax / qmax, 1e-6f);
        if (lane == 0) scales[row] = s;

        uint8_t* yrow = y + (int64_t)row * K;
#pragma unroll
        for (int ci = 0; ci < RC; ++ci) {
            const int c = lane + ci * kWave;
            if (c < chunks) {
                float v[8];
                decode_raw8<XDT>(cache[r][ci], v);
                *(uint2*)(yrow + c * 8) = quantise8<TO_INT8, XDT != GLA_DT_FP32>(v, s);
            }
        }
        for (int c = lane + RC * kWave; c < chunks; c += kWave) {
            float v[8];
            decode_raw8<XDT>(load_raw8_cached<XDT>(xrow, c * 8), v);
            *(uint2*)(yrow + c * 8) = quantise8<TO_INT8, XDT != GLA_DT_FP32>(v, s);
        }
    }
}

// Four lanes share one 32-value group (8 values each): a wave step covers 16 groups = 512 values, and a
// wave takes kMxSteps consecutive steps of the row-major [M_pad, steps per row] grid, all of whose loads
// it issues before it converts anything (one step per wave left a CU with too few bytes in flight).
// FP8OUT: MXFP8 (codes are e4m3fn bytes, y is [M, K]; the largest magnitude is 448) instead of MXFP4
// (e2m1 nibbles, y is [M, K/2]; 6).
constexpr int kMxSteps = 8;

template <int XDT, bool FP8OUT>
__global__ __launch_bounds__(256) void mxfp4_kernel(const void* __restrict__ x, int64_t xsm, int M, int M_pad, int K,
                                                    uint8_t* __restrict__ y, uint8_t* __restrict__ scales) {
    const int groups = K / 32;
    const int gpr = (groups + 15) / 16;  // wave steps per row
    const int64_t total = (int64_t)M_pad * gpr;
    const int64_t first = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kMxSteps;
    const int lane = threadIdx.x & 63;
    if (first >= total) return;

    Raw8<XDT> raw[kMxSteps];
    int rows[kMxSteps], gs[kMxSteps];
#pragma unroll
    for (int u = 0; u < kMxSteps; ++u) {
        const int64_t id = first + u < total ? first + u : total - 1;  // surplus steps repeat the last one (same values, same place)
        rows[u] = (int)(id / gpr);
        gs[u] = (int)(id % gpr) * 16 + (lane >> 2);
        // loads stay in bounds: padding rows and groups past the row read the first chunk of row 0 and drop it
        const bool live = rows[u] < M && gs[u] < groups;
        const char* xrow = (const char*)x + (int64_t)(live ? rows[u] : 0) * xsm * (XDT == GLA_DT_FP32 ? 4 : 2);
        raw[u] = load_raw8<XDT>(xrow, live ? gs[u] * 32 + (lane & 3) * 8 : 0);
    }
#pragma unroll
    for (int u = 0; u < kMxSteps; ++u) {
        const int row = rows[u], g = gs[u];
        if (row >= M) {  // padding rows carry the identity scale and no codes
            if ((lane & 3) == 0 && g < groups) scales[(int64_t)row * groups + g] = 127;
            continue;
        }
        const bool active = g < groups;
        const int k = g * 32 + (lane & 3) * 8;
        float v[8];
        decode_raw8<XDT>(raw[u], v);
        if (!active) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = 0.0f;
        }
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
        amax = fmaxf(amax, __shfl_xor(amax, 1, kWave));
        amax = fmaxf(amax, __shfl_xor(amax, 2, kWave));

        const uint32_t e = e8m0_of_amax<FP8OUT>(amax);

        if (!active) continue;
        // the scale is a power of two, so v / s is an exact exponent shift: ldexp gives the same value (signed
        // zeros and denormal results included) in one instruction instead of a division sequence
        const int down = 127 - (int)e;
        if constexpr (FP8OUT) {
            uint32_t w[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float q[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) q[j] = fminf(fmaxf(__builtin_ldexpf(v[4 * h + j], down), -448.0f), 448.0f);
                w[h] = f32_to_fp8_pair(q[0], q[1]) | (f32_to_fp8_pair(q[2], q[3]) << 16);
            }
            *(uint2*)(y + (int64_t)row * K + k) = make_uint2(w[0], w[1]);
        } else {
            const uint32_t packed = mxfp4_pack8<XDT != GLA_DT_FP32>(v, e);
            *(uint32_t*)(y + (int64_t)row * (K / 2) + k / 2) = packed;
        }
        if ((lane & 3) == 0) scales[(int64_t)row * groups + g] = (uint8_t)e;
    }
}

}  // namespace

int launch_act_per_token(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y, int y_dtype,
                         float* scales, hipStream_t stream) {
    if (x == nullptr || y == nullptr || scales == nullptr || M < 0 || K <= 0) {
        set_error("scale_activations_per_token: null pointer or bad size");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (K % 8 != 0 || x_stride_m % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)y & 7)) {
        set_error("scale_activations_per_token: K and the row stride must be multiples of 8, x 16-byte aligned");
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    if (y_dtype != GLA_DT_INT8 && y_dtype != GLA_DT_FP8) {
        set_error("scale_activations_per_token: output type %d not supported (int8 or fp8-e4m3fn)", y_dtype);
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    if (M == 0) return GLA_OK;
    dim3 grid(ceil_div(M, 4 * kRowsPerWave)), block(256);
    const bool i8 = (y_dtype == GLA_DT_INT8);
#define GLA_PT(XDT)                                                                                         \
    do {                                                                                                    \
        if (i8) hipLaunchKernelGGL((per_token_kernel<XDT, true>), grid, block, 0, stream, x, x_stride_m, M, K, \
                                   (uint8_t*)y, scales);                                                    \
        else hipLaunchKernelGGL((per_token_kernel<XDT, false>), grid, block, 0, stream, x, x_stride_m, M, K,  \
                                (uint8_t*)y, scales);                                                       \
    } while (0)
    switch (x_dtype) {
        case GLA_DT_FP16: GLA_PT(GLA_DT_FP16); break;
        case GLA_DT_BF16: GLA_PT(GLA_DT_BF16); break;
        case GLA_DT_FP32: GLA_PT(GLA_DT_FP32); break;
        default:
            set_error("scale_activations_per_token: input type %d not supported", x_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
    }
#undef GLA_PT
    return check_hip(hipGetLastError(), "per-token activation quant launch");
}

// Per (row, 128-value block) dynamic quantisation to int8 / fp8-e4m3: s = max(amax / qmax, 1e-6),
// y = clamp(x * (1 / s)); int8 rounds floor(y + 0.5) (reference: gemlite/quant_utils.py:2614-2676,
// the kernel multiplies by the reciprocal of the scale).  Sixteen lanes share a block, eight
// consecutive values each; a wave covers four consecutive blocks of a row-major [M, K/128] grid.
template <int XDT, bool TO_INT8>
__global__ __launch_bounds__(256) void per_block_kernel(const void* __restrict__ x, int64_t xsm, int M, int K,
                                                        uint8_t* __restrict__ y, float* __restrict__ scales) {
    const int lane = threadIdx.x & 63;
    const int bpr = K / 128;
    const int64_t blk = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);
    const bool live = blk < (int64_t)M * bpr;
    const int row = live ? (int)(blk / bpr) : 0;
    const int kb = live ? (int)(blk % bpr) : 0;
    const int k = kb * 128 + (lane & 15) * 8;
    const char* xrow = (const char*)x + (int64_t)row * xsm * (XDT == GLA_DT_FP32 ? 4 : 2);
    float v[8];
    decode_raw8<XDT>(load_raw8<XDT>(xrow, k), v);
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, kWave));
    const float qmax = TO_INT8 ? 127.0f : 448.0f;
    const float qmin = TO_INT8 ? -128.0f : -448.0f;
    const float s = fmaxf(amax / qmax, 1e-6f);
    const float r = 1.0f / s;
    if (!live) return;
    if ((lane & 15) == 0) scales[(int64_t)row * bpr + kb] = s;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(v[j] * r, qmin), qmax);
    uint32_t lo = 0, hi = 0;
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
    *(uint2*)(y + (int64_t)row * K + k) = make_uint2(lo, hi);
}

int launch_act_per_block(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y, int y_dtype,
                         float* scales, hipStream_t stream) {
    if (x == nullptr || y == nullptr || scales == nullptr || M < 0 || K <= 0) {
        set_error("scale_activations_per_block: null pointer or bad size");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (y_dtype != GLA_DT_INT8 && y_dtype != GLA_DT_FP8) {
        set_error("scale_activations_per_block: output type %d not supported (int8 or fp8-e4m3fn)", y_dtype);
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    if (K % 128 != 0 || x_stride_m % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)y & 7)) {
        set_error("scale_activations_per_block: K must be a multiple of 128, the row stride of 8, x 16-byte aligned");
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    if (M == 0) return GLA_OK;
    const int64_t blocks = (int64_t)M * (K / 128);
    dim3 grid((unsigned)((blocks + 15) / 16)), block(256);
    const bool i8 = (y_dtype == GLA_DT_INT8);
#define GLA_PB(XDT)                                                                                         \
    do {                                                                                                    \
        if (i8) hipLaunchKernelGGL((per_block_kernel<XDT, true>), grid, block, 0, stream, x, x_stride_m, M, K, \
                                   (uint8_t*)y, scales);                                                    \
        else hipLaunchKernelGGL((per_block_kernel<XDT, false>), grid, block, 0, stream, x, x_stride_m, M, K,  \
                                (uint8_t*)y, scales);                                                       \
    } while (0)
    switch (x_dtype) {
        case GLA_DT_FP16: GLA_PB(GLA_DT_FP16); break;
        case GLA_DT_BF16: GLA_PB(GLA_DT_BF16); break;
        case GLA_DT_FP32: GLA_PB(GLA_DT_FP32); break;
        default:
            set_error("scale_activations_per_block: input type %d not supported", x_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
    }
#undef GLA_PB
    return check_hip(hipGetLastError(), "per-block activation quant launch");
}

static int launch_act_mx(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                         bool fp8, hipStream_t stream);

int launch_act_mxfp4(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                     hipStream_t stream) {
    return launch_act_mx(x, x_dtype, x_stride_m, M, K, y, scales, false, stream);
}

int launch_act_mxfp8(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                     hipStream_t stream) {
    return launch_act_mx(x, x_dtype, x_stride_m, M, K, y, scales, true, stream);
}

static int launch_act_mx(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                         bool fp8, hipStream_t stream) {
    if (x == nullptr || y == nullptr || scales == nullptr || M < 0 || K <= 0) {
        set_error("scale_activations_mxfp: null pointer or bad size");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (K % 32 != 0 || x_stride_m % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)y & (fp8 ? 7 : 3))) {
        set_error("scale_activations_mxfp: K must be a multiple of 32, the row stride of 8, x 16-byte aligned");
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    if (M == 0) return GLA_OK;
    const int M_pad = (M + 31) / 32 * 32;
    const int groups = K / 32;
    const int gpr = (groups + 15) / 16;
    const int64_t waves = ((int64_t)M_pad * gpr + kMxSteps - 1) / kMxSteps;
    dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    switch (x_dtype) {
        case GLA_DT_FP16:
            if (fp8) hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_FP16, true>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            else hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_FP16, false>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            break;
        case GLA_DT_BF16:
            if (fp8) hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_BF16, true>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            else hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_BF16, false>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            break;
        case GLA_DT_FP32:
            if (fp8) hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_FP32, true>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            else hipLaunchKernelGGL((mxfp4_kernel<GLA_DT_FP32, false>), grid, block, 0, stream, x, x_stride_m, M, M_pad, K, y, scales);
            break;
        default:
            set_error("scale_activations_mxfp: input type %d not supported", x_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    return check_hip(hipGetLastError(), "MXFP activation quant launch");
}

}  // namespace gla
