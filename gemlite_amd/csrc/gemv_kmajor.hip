// Streaming GEMV / skinny GEMM (1..16 rows) for fp16/bf16 activations x unpacked 8-bit weights kept
// as the [K, N] view of an [N, K] array (K contiguous): int8, uint8 or fp8-e4m3 codes with
// per-channel scales (and optionally a zero point).  The decode path of weight-only A16W8 layers
// whose weights are not packed into 32-bit words.  The vector variant also takes fp8 x fp8 and int8 x int8
// operands (dynamically quantised A8W8 layers, per-token times per-channel scales) up to 4 rows, where
// the matrix-core GEMM with its split-K finishing launch costs twice the time on small layers.
//
// Takes the place of the reference's split-K GEMV for one element per sample (reference:
// gemlite/triton_kernels/gemv_splitK_kernels.py:257-542; dequant gemlite/triton_kernels/utils.py:73-105;
// the processor that builds such layers: gemlite/helper.py:89-171).
//
//  * A workgroup of 4 waves owns R = 4 weight rows (output columns).  A row is K contiguous bytes,
//    so a wave reads 1 KiB of a row with one 16-byte load per lane; the four waves take the 1 KiB
//    pieces of a row in turn, and every lane keeps 4 rows x 16 bytes in flight.
//  * Codes are converted to fp32 in registers (byte-to-float conversion for integers, with the
//    sign handled as "code xor 0x80, minus 128 times the sum of the activations" at the end; the
//    packed fp8 conversion for e4m3) and multiplied with fp32 activations; the activations come
//    straight from global memory through the vector cache, 32 bytes per row and lane.
//  * Per-channel dequantisation commutes with the sum over K, so the loop accumulates D = sum x w
//    and X = sum x only, and the epilogue forms s (D - z X), s D + z' X, ... per W_group_mode,
//    then applies the channel scales.  fp32 throughout; sums over lanes by butterfly, over the four
//    waves through LDS in fixed order (deterministic, no atomics, output need not be zeroed).
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"
#include "actquant_device.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4k __attribute__((ext_vector_type(4)));
typedef float f32x2k __attribute__((ext_vector_type(2)));

constexpr int kRowsK = 4;    // weight rows per workgroup
constexpr int kWavesK = 4;   // waves per workgroup, interleaved over K
constexpr int kLaneK = 16;   // K-values per lane and iteration
constexpr int kIterK = 64 * kLaneK;
constexpr int kRows8 = 4;    // rows up to which 8-bit activations are taken (vector variant)

struct GemvKArgs {
    const uint16_t* x;
    const uint8_t* w;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    int M, N, K;
    int64_t xsm, wsn, osm, msn, sxm;
    int wgm, csm, meta_dt, z_dt, z_scalar, out_dt, sx_dt;
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

// store v, or with a bias round(v) + bias[n]: the reference's `out += bias` on the rounded output
__device__ __forceinline__ void store_result(const GemvKArgs& a, int m, int n, float v) {
    if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n);
    store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + n, v);
}

// 16 codes (one 128-bit load) -> 16 floats.  Signed bytes come out biased by +128.
template <int WDT>
__device__ __forceinline__ void codes_to_float(const u32x4k& v, float (&f)[16]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        if constexpr (WDT == GLA_DT_FP8) {
            const f32x2k lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[q], false);
            const f32x2k hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[q], true);
            f[4 * q] = lo.x; f[4 * q + 1] = lo.y; f[4 * q + 2] = hi.x; f[4 * q + 3] = hi.y;
        } else {
            const uint32_t u = WDT == GLA_DT_INT8 ? v[q] ^ 0x80808080u : v[q];
            f[4 * q] = (float)(u & 0xffu);
            f[4 * q + 1] = (float)((u >> 8) & 0xffu);
            f[4 * q + 2] = (float)((u >> 16) & 0xffu);
            f[4 * q + 3] = (float)(u >> 24);
        }
    }
}

// activation kinds of the vector variant
constexpr int kXF16 = 0, kXBF16 = 1, kXFP8 = 2, kXI8 = 3;

template <bool BF16>
__device__ __forceinline__ void acts_to_float(const u32x4k& a, const u32x4k& b, float (&f)[16]) {
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const uint32_t v = q < 4 ? a[q] : b[q - 4];
        if constexpr (BF16) {
            f[2 * q] = __builtin_bit_cast(float, v << 16);
            f[2 * q + 1] = __builtin_bit_cast(float, v & 0xffff0000u);
        } else {
            f[2 * q] = half_bits_to_float((uint16_t)(v & 0xffffu));
            f[2 * q + 1] = half_bits_to_float((uint16_t)(v >> 16));
        }
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// MT: rows of x handled (power of two >= M).  XK: activation kind.  int8 x int8 sums exactly: a lane's fp32
// sums stay below 2^24 (the host bounds K), the sums over lanes and waves are taken in int32.
// QF (8-bit activation kinds only): 0 = x holds the codes; kXF16 + 1 / kXBF16 + 1 = x holds fp16 / bf16 rows and the
// workgroup quantises them per token itself (the quantiser launch in front of a decode matmul costs a third of the
// matmul's time): every workgroup takes the row's amax (the row is a few KB and sits in L2), forms the scale
// max(amax / qmax, 1e-6) and turns the 16 activations a lane multiplies into the quantiser's codes, with the
// quantiser's own arithmetic, before it multiplies them, so the result equals quantiser + matmul bit for bit.
// RK: weight rows per workgroup: 4; 8 when the rows are quantised here, so that the quantisation of a K-chunk is
// shared by twice the columns (every workgroup quantises the whole row).
template <int WDT, int XK, int MT, int QF = 0, int RK = kRowsK>
__global__ __launch_bounds__(kWavesK * 64) void gemv_kmajor_kernel(GemvKArgs a) {
    constexpr bool X8 = XK == kXFP8 || XK == kXI8;
    constexpr bool EXACT = XK == kXI8;
    constexpr bool FUSED = QF != 0;
    static_assert(!FUSED || X8, "on-the-fly quantisation makes 8-bit codes");
    __shared__ float red[kWavesK][RK * MT + MT];
    __shared__ float amax_sh[kWavesK][MT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * RK;
    const uint8_t* wrow[RK];
#pragma unroll
    for (int r = 0; r < RK; ++r) {
        const int n = n0 + r < a.N ? n0 + r : a.N - 1;  // rows past the end repeat the last one; never stored
        wrow[r] = a.w + (int64_t)n * a.wsn;
    }
    const uint8_t* xrow[MT];  // x_stride_m counts stored elements
#pragma unroll
    for (int m = 0; m < MT; ++m) xrow[m] = (const uint8_t*)a.x + (int64_t)(m < a.M ? m : a.M - 1) * a.xsm * ((X8 && !FUSED) ? 1 : 2);

    // per-token scales of the rows, as gla_scale_activations_per_token computes them
    float xs_s[MT], xs_r[MT];
    if constexpr (FUSED) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float am = 0.0f;
            for (int c = threadIdx.x; c < a.K / 8; c += kWavesK * 64) {
                const u32x4k raw = *(const u32x4k*)(xrow[m] + 16 * c);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float lo, hi;
                    if constexpr (QF == kXBF16 + 1) {
                        lo = __builtin_bit_cast(float, raw[q] << 16);
                        hi = __builtin_bit_cast(float, raw[q] & 0xffff0000u);
                    } else {
                        lo = half_bits_to_float((uint16_t)(raw[q] & 0xffffu));
                        hi = half_bits_to_float((uint16_t)(raw[q] >> 16));
                    }
                    am = fmaxf(am, fmaxf(fabsf(lo), fabsf(hi)));
                }
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) am = fmaxf(am, __shfl_xor(am, o, 64));
            if (lane == 0) amax_sh[wave][m] = am;
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float am = amax_sh[0][m];
#pragma unroll
            for (int w = 1; w < kWavesK; ++w) am = fmaxf(am, amax_sh[w][m]);
            xs_s[m] = fmaxf(am / (XK == kXI8 ? 127.0f : 448.0f), 1e-6f);
            xs_r[m] = 1.0f / xs_s[m];
        }
    }

    float acc[RK][MT], sumx[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        sumx[m] = 0.0f;
#pragma unroll
        for (int r = 0; r < RK; ++r) acc[r][m] = 0.0f;
    }

    for (int k = wave * kIterK + lane * kLaneK; k < a.K; k += kWavesK * kIterK) {  // K % 16 == 0
        u32x4k wv[RK];
#pragma unroll
        for (int r = 0; r < RK; ++r) wv[r] = *(const u32x4k*)(wrow[r] + k);
        float wf[RK <= 4 ? RK : 1][16];
        if constexpr (RK <= 4) {
#pragma unroll
            for (int r = 0; r < RK; ++r) codes_to_float<WDT>(wv[r], wf[r]);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float xf[16];
            if constexpr (FUSED) {
                const u32x4k xa = *(const u32x4k*)(xrow[m] + 2 * k), xb = *(const u32x4k*)(xrow[m] + 2 * k + 16);
                acts_to_float<QF == kXBF16 + 1>(xa, xb, xf);
                const float qmax = XK == kXI8 ? 127.0f : 448.0f, qmin = XK == kXI8 ? -128.0f : -448.0f;
#pragma unroll
                for (int q = 0; q < 16; ++q) xf[q] = fminf(fmaxf(div_by_row_scale(xf[q], xs_s[m], xs_r[m]), qmin), qmax);
                if constexpr (XK == kXI8) {
#pragma unroll
                    for (int q = 0; q < 16; ++q) xf[q] = floorf(xf[q] + 0.5f);  // the code itself, as a float
                } else {
#pragma unroll
                    for (int q = 0; q < 16; q += 2) {  // to e4m3 and back: the value the stored code would give
                        const f32x2k back = __builtin_amdgcn_cvt_pk_f32_fp8((int)f32_to_fp8_pair(xf[q], xf[q + 1]), false);
                        xf[q] = back.x;
                        xf[q + 1] = back.y;
                    }
                }
            } else if constexpr (XK == kXFP8) {
                codes_to_float<GLA_DT_FP8>(*(const u32x4k*)(xrow[m] + k), xf);
            } else if constexpr (XK == kXI8) {
                codes_to_float<GLA_DT_INT8>(*(const u32x4k*)(xrow[m] + k), xf);  // biased by +128
#pragma unroll
                for (int q = 0; q < 16; ++q) xf[q] -= 128.0f;
            } else {
                const u32x4k xa = *(const u32x4k*)(xrow[m] + 2 * k), xb = *(const u32x4k*)(xrow[m] + 2 * k + 16);
                acts_to_float<XK == kXBF16>(xa, xb, xf);
            }
            if constexpr (RK <= 4) {
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    sumx[m] += xf[q];
#pragma unroll
                    for (int r = 0; r < RK; ++r) acc[r][m] = __builtin_fmaf(xf[q], wf[r][q], acc[r][m]);
                }
            } else {  // more rows than registers for all their floats: one weight row at a time
#pragma unroll
                for (int q = 0; q < 16; ++q) sumx[m] += xf[q];
#pragma unroll
                for (int r = 0; r < RK; ++r) {
                    codes_to_float<WDT>(wv[r], wf[0]);
#pragma unroll
                    for (int q = 0; q < 16; ++q) acc[r][m] = __builtin_fmaf(xf[q], wf[0][q], acc[r][m]);
                }
            }
        }
    }

    // sums over the lanes of the wave, then over the waves in fixed order
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if constexpr (EXACT) {
            const int sx = wave_sum_int((int)sumx[m]);
            if (lane == 0) red[wave][RK * MT + m] = __builtin_bit_cast(float, sx);
#pragma unroll
            for (int r = 0; r < RK; ++r) {
                const int d = wave_sum_int((int)acc[r][m]);
                if (lane == 0) red[wave][r * MT + m] = __builtin_bit_cast(float, d);
            }
        } else {
            const float sx = wave_sum(sumx[m]);
            if (lane == 0) red[wave][RK * MT + m] = sx;
#pragma unroll
            for (int r = 0; r < RK; ++r) {
                const float d = wave_sum(acc[r][m]);
                if (lane == 0) red[wave][r * MT + m] = d;
            }
        }
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t >= RK * MT) return;
    const int r = t / MT, m = t % MT, n = n0 + r;
    if (n >= a.N || m >= a.M) return;
    float D = 0.0f, X = 0.0f;
    if constexpr (EXACT) {
        int Di = 0, Xi = 0;
#pragma unroll
        for (int w = 0; w < kWavesK; ++w) {
            Di += __builtin_bit_cast(int, red[w][r * MT + m]);
            Xi += __builtin_bit_cast(int, red[w][RK * MT + m]);
        }
        if (WDT == GLA_DT_INT8) Di -= 128 * Xi;  // undo the bias of the byte conversion
        D = (float)Di;                            // the int32 accumulator of the reference, converted once
        X = (float)Xi;
    } else {
#pragma unroll
        for (int w = 0; w < kWavesK; ++w) {
            D += red[w][r * MT + m];
            X += red[w][RK * MT + m];
        }
        if (WDT == GLA_DT_INT8) D = __builtin_fmaf(-128.0f, X, D);  // undo the bias of the byte conversion
    }
    const bool uses_s = a.wgm >= GLA_WGM_SCALE;
    const bool uses_z = a.wgm == GLA_WGM_SHIFT || a.wgm >= GLA_WGM_SHIFT_SCALE;
    const float s = uses_s ? load_as_float(a.scales, a.meta_dt, (int64_t)n * a.msn) : 1.0f;
    const float z = uses_z ? load_as_float(a.zeros, a.z_dt, a.z_scalar ? 0 : (int64_t)n * a.msn) : 0.0f;
    float v;
    switch (a.wgm) {
        case GLA_WGM_SHIFT: v = D - z * X; break;
        case GLA_WGM_SCALE: v = s * D; break;
        case GLA_WGM_SHIFT_SCALE: v = s * (D - z * X); break;
        case GLA_WGM_FMA: v = __builtin_fmaf(s, D, z * X); break;
        default: v = D; break;
    }
    float post = 1.0f;
    if (a.csm & 1) post *= load_as_float(a.scales, a.meta_dt, (int64_t)n * a.msn);
    if (a.csm & 2) {
        if constexpr (FUSED) {
            float sx = xs_s[0];
#pragma unroll
            for (int mm = 1; mm < MT; ++mm) sx = m == mm ? xs_s[mm] : sx;
            post *= sx;
        } else {
            post *= load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm);
        }
    }
    store_result(a, m, n, v * post);
}

// ---- 3..16 rows: the same streaming on the matrix cores.  A workgroup of 16 waves owns 16 weight
// rows; the waves take 64-byte pieces of the rows in turn.  Per step a lane (row l%16, quarter l/16)
// loads 16 weight bytes, converts them to two 8-element fp16/bf16 operands (exactly: |code| <= 255
// fits either format) and feeds two v_mfma_f32_16x16x32 whose other operand is the matching 16
// activations of row l%16 of x.  Four steps are in flight per lane.  Sums over the waves go
// through LDS in fixed order.
typedef _Float16 half8_k __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_k __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_k __attribute__((ext_vector_type(2)));
typedef float f32x4_k __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2k __attribute__((ext_vector_type(2)));

constexpr int kWavesKM = 16;

// 8 codes (two dwords) -> the four registers of an 8-element 16-bit operand, K order kept
template <int WDT, bool BF16>
__device__ __forceinline__ u32x4k codes_to_operand(uint32_t d0, uint32_t d1) {
    u32x4k o;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t d = h ? d1 : d0;
        if constexpr (WDT == GLA_DT_FP8) {
            const f32x2k lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)d, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)d, true);
            if constexpr (BF16) {
                o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2_k));
                o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2_k));
            } else {
                o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo.x, lo.y));
                o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(hi.x, hi.y));
            }
        } else if constexpr (BF16) {
            const uint32_t u = WDT == GLA_DT_INT8 ? d ^ 0x80808080u : d;
            const float off = WDT == GLA_DT_INT8 ? -128.0f : 0.0f;
            const f32x2k lo = {(float)(u & 0xffu) + off, (float)((u >> 8) & 0xffu) + off};
            const f32x2k hi = {(float)((u >> 16) & 0xffu) + off, (float)(u >> 24) + off};
            o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2_k));
            o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2_k));
        } else {
            // fp16: bytes into the mantissa of 1024.0, two per register, then minus 1024 (+128 for signed codes)
            const uint32_t u = WDT == GLA_DT_INT8 ? d ^ 0x80808080u : d;
            const half2_t off = WDT == GLA_DT_INT8 ? half2_t{(half_t)1152.0f, (half_t)1152.0f} : half2_t{(half_t)1024.0f, (half_t)1024.0f};
            const uint32_t t0 = __builtin_amdgcn_perm(u, u, 0x0c010c00u) | 0x64006400u;
            const uint32_t t1 = __builtin_amdgcn_perm(u, u, 0x0c030c02u) | 0x64006400u;
            o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, t0) - off);
            o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, t1) - off);
        }
    }
    return o;
}

template <bool BF16>
__device__ __forceinline__ f32x4_k mfma16(const u32x4k& a, const u32x4k& b, f32x4_k c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_k, a), __builtin_bit_cast(bf16x8_k, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_k, a), __builtin_bit_cast(half8_k, b), c, 0, 0, 0);
}

// RT: tiles of 16 weight rows per workgroup; the activations a lane loads serve all of them
template <int WDT, bool BF16, int RT>
__global__ __launch_bounds__(kWavesKM * 64) void gemv_kmajor_mfma_kernel(GemvKArgs a) {
    __shared__ f32x4_k red[kWavesKM][RT][64];
    __shared__ float redx[kWavesKM][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16 * RT;
    const uint8_t* wrow[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int n = n0 + 16 * t + r16;
        wrow[t] = a.w + (int64_t)(n < a.N ? n : a.N - 1) * a.wsn + 16 * kq;
    }
    const uint16_t* xrow = a.x + (int64_t)(r16 < a.M ? r16 : a.M - 1) * a.xsm + 16 * kq;
    const bool need_x = a.wgm == GLA_WGM_SHIFT || a.wgm >= GLA_WGM_SHIFT_SCALE;  // modes with a zero point
    f32x4_k acc[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[t] = f32x4_k{0.0f, 0.0f, 0.0f, 0.0f};
    float sumx = 0.0f;
    constexpr int UN = 4;                          // steps in flight per lane
    constexpr int STRIDE = kWavesKM * 64;          // K-values between a wave's steps
    for (int k0 = wave * 64; k0 < a.K; k0 += UN * STRIDE) {  // K % 64 == 0
        u32x4k wv[UN][RT], xa[UN], xb[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            // steps past the end re-read the wave's first piece and are not multiplied
            const int k = k0 + u * STRIDE < a.K ? k0 + u * STRIDE : wave * 64;
#pragma unroll
            for (int t = 0; t < RT; ++t) wv[u][t] = *(const u32x4k*)(wrow[t] + k);
            xa[u] = *(const u32x4k*)(xrow + k);
            xb[u] = *(const u32x4k*)(xrow + k + 8);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (k0 + u * STRIDE < a.K) {
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    acc[t] = mfma16<BF16>(codes_to_operand<WDT, BF16>(wv[u][t][0], wv[u][t][1]), xa[u], acc[t]);
                    acc[t] = mfma16<BF16>(codes_to_operand<WDT, BF16>(wv[u][t][2], wv[u][t][3]), xb[u], acc[t]);
                }
                if (need_x) {
                    float xf[16];
                    acts_to_float<BF16>(xa[u], xb[u], xf);
#pragma unroll
                    for (int q = 0; q < 16; ++q) sumx += xf[q];
                }
            }
        }
    }
    // lane holds D[n0 + 16 t + 4 kq + e][m = r16]; X[m]: sum over the four K quarters of the lane group, then over waves
    sumx += __shfl_xor(sumx, 16, 64);
    sumx += __shfl_xor(sumx, 32, 64);
#pragma unroll
    for (int t = 0; t < RT; ++t) red[wave][t][lane] = acc[t];
    if (lane < 16) redx[wave][lane] = sumx;
    __syncthreads();
    if (wave != 0) return;
    float X = 0.0f;
#pragma unroll
    for (int w = 0; w < kWavesKM; ++w) X += redx[w][r16];
    const int m = r16;
    if (m >= a.M) return;
    const bool uses_s = a.wgm >= GLA_WGM_SCALE;
    const float sxm = (a.csm & 2) ? load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm) : 1.0f;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        f32x4_k D = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < kWavesKM; ++w) D += red[w][t][lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = n0 + 16 * t + 4 * kq + e;
            if (n >= a.N) continue;
            const float s = uses_s ? load_as_float(a.scales, a.meta_dt, (int64_t)n * a.msn) : 1.0f;
            const float z = need_x ? load_as_float(a.zeros, a.z_dt, a.z_scalar ? 0 : (int64_t)n * a.msn) : 0.0f;
            float v;
            switch (a.wgm) {
                case GLA_WGM_SHIFT: v = D[e] - z * X; break;
                case GLA_WGM_SCALE: v = s * D[e]; break;
                case GLA_WGM_SHIFT_SCALE: v = s * (D[e] - z * X); break;
                case GLA_WGM_FMA: v = __builtin_fmaf(s, D[e], z * X); break;
                default: v = D[e]; break;
            }
            float post = sxm;
            if (a.csm & 1) post *= load_as_float(a.scales, a.meta_dt, (int64_t)n * a.msn);
            store_result(a, m, n, v * post);
        }
    }
}

template <int WDT, bool BF16>
int launch_k(const GemvKArgs& a, hipStream_t stream) {
    if (a.M > 2 && a.K % 64 == 0) {
        // two row tiles per workgroup while that still leaves every CU a workgroup
        if (a.N >= 32 * 256)
            hipLaunchKernelGGL((gemv_kmajor_mfma_kernel<WDT, BF16, 2>), dim3(ceil_div(a.N, 32)), dim3(kWavesKM * 64), 0, stream, a);
        else
            hipLaunchKernelGGL((gemv_kmajor_mfma_kernel<WDT, BF16, 1>), dim3(ceil_div(a.N, 16)), dim3(kWavesKM * 64), 0, stream, a);
        return check_hip(hipGetLastError(), "gemv_kmajor launch");
    }
    constexpr int XK = BF16 ? kXBF16 : kXF16;
    const dim3 grid(ceil_div(a.N, kRowsK)), block(kWavesK * 64);
    if (a.M == 1) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 1>), grid, block, 0, stream, a);
    else if (a.M == 2) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 2>), grid, block, 0, stream, a);
    else if (a.M <= 4) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 4>), grid, block, 0, stream, a);
    else if (a.M <= 8) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 8>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 16>), grid, block, 0, stream, a);
    return check_hip(hipGetLastError(), "gemv_kmajor launch");
}

// 8-bit activations of the weights' own type (fp8 x fp8, int8 x int8), up to 4 rows; QF: see the kernel
template <int WDT, int XK, int QF = 0>
int launch_k8(const GemvKArgs& a, hipStream_t stream) {
    if constexpr (QF != 0) {
        // one and two rows on layers wide enough to give every CU four workgroups of 8 columns
        if (a.M <= 2 && a.N >= 8 * 1024) {
            const dim3 grid8(ceil_div(a.N, 8)), block8(kWavesK * 64);
            if (a.M == 1) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 1, QF, 8>), grid8, block8, 0, stream, a);
            else hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 2, QF, 8>), grid8, block8, 0, stream, a);
            return check_hip(hipGetLastError(), "gemv_kmajor launch");
        }
    }
    const dim3 grid(ceil_div(a.N, kRowsK)), block(kWavesK * 64);
    if (a.M == 1) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 1, QF>), grid, block, 0, stream, a);
    else if (a.M == 2) hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 2, QF>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gemv_kmajor_kernel<WDT, XK, 4, QF>), grid, block, 0, stream, a);
    return check_hip(hipGetLastError(), "gemv_kmajor launch");
}

}  // namespace

bool gemv_kmajor_eligible(const gla_matmul_args& p) {
    if (p.M < 1 || p.M > 16) return false;
    if (p.W_nbits != 8 || p.elements_per_sample != 1) return false;
    if (!(p.w_dtype == GLA_DT_INT8 || p.w_dtype == GLA_DT_UINT8 || p.w_dtype == GLA_DT_FP8)) return false;
    const bool x8 = (p.input_dtype == GLA_DT_FP8 && p.w_dtype == GLA_DT_FP8 && p.acc_dtype == GLA_DT_FP32) ||
                    (p.input_dtype == GLA_DT_INT8 && p.w_dtype == GLA_DT_INT8 &&
                     (p.acc_dtype == GLA_DT_INT32 || p.acc_dtype == GLA_DT_FP32));
    if (x8) {
        // the vector variant only; a lane's fp32 sum of |x| <= 128 times a biased code <= 255 over K / 256 values
        // must stay below 2^24 for the int8 sums to be exact
        if (p.M > kRows8 || p.K > 131072 || p.x_stride_m % (p.x_quant_from ? 8 : 16) != 0) return false;
        // quantised on the fly from fp16 / bf16 rows: per-token scales only, and they come from the kernel
        if (p.x_quant_from && !(p.x_quant_from == GLA_DT_FP16 || p.x_quant_from == GLA_DT_BF16)) return false;
        if (p.x_quant_from && !(p.channel_scale_mode & 2)) return false;
        // 3 and 4 rows only on layers of 20 MB or less (4096^2: 13 against 15 us for the matrix-core GEMM and its
        // finishing launch; 8192^2: 29 against 21); 1 and 2 rows everywhere (4096^2 6.7 against 14.7, 8192^2 15.6
        // against 21.6 us)
        if (p.M > 2 && (int64_t)p.N * p.K > 20000000) return false;
    } else if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16) || p.acc_dtype != GLA_DT_FP32) {
        return false;
    }
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if (p.W_group_mode < GLA_WGM_NONE || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.K % kLaneK != 0 || p.w_stride_n % 16 != 0 || (!x8 && p.x_stride_m % 8 != 0)) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    const bool uses_s = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_z = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    // dequantisation must be per channel: one group spanning K (or a scalar zero point alone)
    if ((uses_s || (uses_z && !p.zero_is_scalar)) && p.group_size != p.K) return false;
    if (uses_s && p.scales == nullptr) return false;
    if (uses_z && p.zeros == nullptr) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr && !(x8 && p.x_quant_from)) return false;
    if (!x8 && p.x_quant_from) return false;
    return true;
}

int launch_gemv_kmajor(const gla_matmul_args& p, hipStream_t stream) {
    GemvKArgs a;
    a.x = (const uint16_t*)p.x; a.w = (const uint8_t*)p.w; a.scales = p.scales; a.zeros = p.zeros; a.scales_x = p.scales_x;
    a.out = p.out; a.M = p.M; a.N = p.N; a.K = p.K;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.msn = p.meta_stride_n; a.sxm = p.sx_stride_m;
    a.wgm = p.W_group_mode; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.z_dt = p.zeros_dtype;
    a.z_scalar = p.zero_is_scalar; a.out_dt = p.output_dtype; a.sx_dt = p.sx_dtype;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    if (p.x_quant_from == GLA_DT_FP16) {
        return p.input_dtype == GLA_DT_FP8 ? launch_k8<GLA_DT_FP8, kXFP8, kXF16 + 1>(a, stream)
                                           : launch_k8<GLA_DT_INT8, kXI8, kXF16 + 1>(a, stream);
    }
    if (p.x_quant_from == GLA_DT_BF16) {
        return p.input_dtype == GLA_DT_FP8 ? launch_k8<GLA_DT_FP8, kXFP8, kXBF16 + 1>(a, stream)
                                           : launch_k8<GLA_DT_INT8, kXI8, kXBF16 + 1>(a, stream);
    }
    if (p.input_dtype == GLA_DT_FP8) return launch_k8<GLA_DT_FP8, kXFP8>(a, stream);
    if (p.input_dtype == GLA_DT_INT8) return launch_k8<GLA_DT_INT8, kXI8>(a, stream);
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.w_dtype) {
        case GLA_DT_INT8: return bf16 ? launch_k<GLA_DT_INT8, true>(a, stream) : launch_k<GLA_DT_INT8, false>(a, stream);
        case GLA_DT_UINT8: return bf16 ? launch_k<GLA_DT_UINT8, true>(a, stream) : launch_k<GLA_DT_UINT8, false>(a, stream);
        default: return bf16 ? launch_k<GLA_DT_FP8, true>(a, stream) : launch_k<GLA_DT_FP8, false>(a, stream);
    }
}

}  // namespace gla
