// Shared device/host helpers for the gfx950 quantized-matmul kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/gemlite_amd.h"

namespace gla {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef int int8_t_v __attribute__((ext_vector_type(8)));
typedef int int16_t_v __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// error reporting (host)
// ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);

// Function attributes (the dynamic LDS limit) are kept per device: true the first time a call site
// runs on the current device.  `seen` is the call site's own table (one per kernel instantiation).
struct DeviceOnce {
    std::atomic<bool> seen[64];
    bool first() {
        int d = 0;
        if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= 64) return true;
        return !seen[d].exchange(true);
    }
};
int check_hip(hipError_t e, const char* what);

// ---------------------------------------------------------------------------
// scalar conversions (device)
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// Two floats -> two bf16 in one register (lo in bits 15:0), round to nearest even: one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// round-to-nearest-even float -> bf16 bits
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) { return (uint16_t)pack_bf16x2(f, 0.0f); }

// Two floats -> two fp16 in one register (lo in bits 15:0), round to nearest even.
__device__ __forceinline__ uint32_t pack_half2(float lo, float hi) {
    const half2_t v = {(half_t)lo, (half_t)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float half_bits_to_float(uint16_t b) {
    return (float)__builtin_bit_cast(half_t, b);
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
    return __builtin_bit_cast(uint16_t, (half_t)f);
}

// OCP e4m3fn byte -> float (gfx950 converts OCP fp8 natively)
__device__ __forceinline__ float fp8_to_float(uint8_t b) {
    return __builtin_amdgcn_cvt_f32_fp8((int)b, 0);
}

// e2m1 nibble -> float: sign | {0, .5, 1, 1.5, 2, 3, 4, 6}
__device__ __forceinline__ float e2m1_to_float(uint32_t nib) {
    const uint32_t mag = nib & 7u;
    // exponent/mantissa decode without a table: values are m * 2^(e-1)
    float v;
    switch (mag) {
        case 0: v = 0.0f; break;
        case 1: v = 0.5f; break;
        case 2: v = 1.0f; break;
        case 3: v = 1.5f; break;
        case 4: v = 2.0f; break;
        case 5: v = 3.0f; break;
        case 6: v = 4.0f; break;
        default: v = 6.0f; break;
    }
    return (nib & 8u) ? -v : v;
}

// e8m0 byte -> float 2^(b-127)  (b = 0 maps to 2^-127, a subnormal; 255 = NaN)
__device__ __forceinline__ float e8m0_to_float(uint8_t b) {
    if (b == 0) return __builtin_bit_cast(float, 0x00400000u);
    if (b == 255) return __builtin_bit_cast(float, 0x7fc00000u);
    return __builtin_bit_cast(float, (uint32_t)b << 23);
}

// Load element `idx` of an array of element type `dt` as float.
__device__ __forceinline__ float load_as_float(const void* p, int dt, int64_t idx) {
    switch (dt) {
        case GLA_DT_FP32: return ((const float*)p)[idx];
        case GLA_DT_FP16: return half_bits_to_float(((const uint16_t*)p)[idx]);
        case GLA_DT_BF16: return bf16_bits_to_float(((const uint16_t*)p)[idx]);
        case GLA_DT_FP8: return fp8_to_float(((const uint8_t*)p)[idx]);
        case GLA_DT_INT8: return (float)((const int8_t*)p)[idx];
        case GLA_DT_UINT8: return (float)((const uint8_t*)p)[idx];
        case GLA_DT_INT32: return (float)((const int32_t*)p)[idx];
        case GLA_DT_E8M0: return e8m0_to_float(((const uint8_t*)p)[idx]);
        default: return 0.0f;
    }
}

// Store `v` to element `idx` of an array of element type `dt`.
__device__ __forceinline__ void store_from_float(void* p, int dt, int64_t idx, float v) {
    switch (dt) {
        case GLA_DT_FP32: ((float*)p)[idx] = v; break;
        case GLA_DT_FP16: ((uint16_t*)p)[idx] = float_to_half_bits(v); break;
        case GLA_DT_BF16: ((uint16_t*)p)[idx] = float_to_bf16_bits(v); break;
        case GLA_DT_INT32: ((int32_t*)p)[idx] = (int32_t)v; break;
        default: break;
    }
}

// `v` as the output type `dt` holds it (fp16 / bf16 rounding; fp32 as it is).
__device__ __forceinline__ float round_to_dtype(int dt, float v) {
    if (dt == GLA_DT_FP16) return half_bits_to_float(float_to_half_bits(v));
    if (dt == GLA_DT_BF16) return bf16_bits_to_float(float_to_bf16_bits(v));
    return v;
}

// Store with the element type fixed at compile time (DT is a GLA_DT_* id).
template <int DT>
__device__ __forceinline__ void store_typed(void* p, int64_t idx, float v) {
    if constexpr (DT == GLA_DT_FP32) ((float*)p)[idx] = v;
    else if constexpr (DT == GLA_DT_FP16) ((uint16_t*)p)[idx] = float_to_half_bits(v);
    else if constexpr (DT == GLA_DT_BF16) ((uint16_t*)p)[idx] = float_to_bf16_bits(v);
    else ((int32_t*)p)[idx] = (int32_t)v;
}

__host__ __device__ __forceinline__ int dtype_size(int dt) {
    switch (dt) {
        case GLA_DT_FP32: case GLA_DT_INT32: case 7: return 4;
        case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_INT16: case 10: return 2;
        case GLA_DT_INT64: return 8;
        default: return 1;
    }
}

template <typename T>
__device__ __forceinline__ T wave_xor(T v, int mask) {
    return __shfl_xor(v, mask, kWave);
}

static inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// Workspace layout shared by every family.  The first kWsPrivateBytes belong to the streaming GEMV
// kernels alone: kWsCounterBytes of ticket counters, then their tagged partial slots.  Nothing else
// ever writes there, so "all counters zero, all slots invalid" holds between launches (the buffer
// starts zero-filled and the last-arriving workgroup of a column tile clears what it consumed).
// Every other use of the workspace (split-K partials of the GEMMs, regrouped block scales, GEMV
// partials too large for the slot region) starts at kWsPrivateBytes.
constexpr int64_t kWsCounterBytes = 256 * 1024;
constexpr int64_t kWsPrivateBytes = 4 << 20;

// 128-bit load that is not kept in the caches on its way in (weights are read once per launch;
// measured on MI355X: 5-9 % more streaming bandwidth than a plain load).
__device__ __forceinline__ uint4 load_streaming_u4(const void* p) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_nontemporal_load((const u4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_streaming_u2(const void* p) {
    typedef unsigned int u2 __attribute__((ext_vector_type(2)));
    const u2 v = __builtin_nontemporal_load((const u2*)p);
    return make_uint2(v.x, v.y);
}

// ---------------------------------------------------------------------------
// kernel-family launchers (host); each returns a GLA_* status
// ---------------------------------------------------------------------------
struct MatmulPlan;  // defined in dispatch.hpp

}  // namespace gla
