// Layout-agnostic quantized matmul: one lane per output column, a loop over K.
//
// This kernel accepts every operand layout, packing width, element type and
// mode combination the C ABI admits.  It is the path for shapes the tuned
// kernels do not cover (odd packing widths, strided views, N not a multiple of
// 4, ...); the tuned kernels are checked against the same arithmetic contract:
//
//   w(k,n)   = dequant(code(k,n))            per W_group_mode, in fp32
//   acc(m,n) = sum_k x(m,k) * w(k,n)         fp32, or exact int32
//   out(m,n) = cast(acc * channel scales)    per channel_scale_mode
//
// (reference: gemlite/triton_kernels/utils.py:73-105 for dequant,
//  gemlite/triton_kernels/gemm_kernels.py:405-496 for the loop and epilogue,
//  gemlite/triton_kernels/gemm_kernels.py:696-726 for the micro-scaled form).
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

constexpr int kRows = 4;  // output rows per thread

struct GenericArgs {
    const void* x;
    const void* w;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    int M, N, K;
    int64_t xsm, xsk, wsk, wsn, osm, osn, msg, msn, sxm, sxg;
    int nbits, gs, mask, e;
    int in_dt, out_dt, acc_dt, meta_dt, csm, wgm;
    int w_dt, z_dt, z_scalar, sx_dt;
};

__device__ __forceinline__ int64_t load_word(const void* p, int dt, int64_t idx) {
    switch (dt) {
        case GLA_DT_UINT8: return ((const uint8_t*)p)[idx];
        case GLA_DT_INT8: return ((const int8_t*)p)[idx];
        case GLA_DT_INT16: return ((const int16_t*)p)[idx];
        case GLA_DT_INT32: return ((const int32_t*)p)[idx];
        case GLA_DT_INT64: return ((const int64_t*)p)[idx];
        default: return 0;
    }
}

__device__ __forceinline__ bool is_float_dt(int dt) {
    return dt == GLA_DT_FP32 || dt == GLA_DT_FP16 || dt == GLA_DT_BF16 || dt == GLA_DT_FP8;
}

// Integer and float grouped-dequant matmul.
__global__ __launch_bounds__(64) void generic_int_kernel(GenericArgs a) {
    const int n = blockIdx.x * 64 + threadIdx.x;
    const int m0 = blockIdx.y * kRows;
    if (n >= a.N) return;

    const bool int_acc = (a.acc_dt == GLA_DT_INT32);
    const bool w_is_float = is_float_dt(a.w_dt);
    const int groups = (a.wgm == GLA_WGM_NONE) ? 1 : (a.K / a.gs);
    const int klen = (a.wgm == GLA_WGM_NONE) ? a.K : a.gs;
    const bool has_scale = (a.wgm == GLA_WGM_SCALE || a.wgm == GLA_WGM_SHIFT_SCALE || a.wgm == GLA_WGM_FMA);
    const bool has_zero = (a.wgm == GLA_WGM_SHIFT || a.wgm == GLA_WGM_SHIFT_SCALE || a.wgm == GLA_WGM_FMA);

    float facc[kRows] = {0.f, 0.f, 0.f, 0.f};
    int iacc[kRows] = {0, 0, 0, 0};

    for (int g = 0; g < groups; ++g) {
        float s = 1.0f, z = 0.0f;
        if (has_scale) s = load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + (int64_t)n * a.msn);
        if (has_zero)
            z = a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0)
                           : load_as_float(a.zeros, a.z_dt, (int64_t)g * a.msg + (int64_t)n * a.msn);
        const int k0 = g * klen;
        for (int kk = 0; kk < klen; ++kk) {
            const int k = k0 + kk;
            const int64_t widx = (int64_t)(k / a.e) * a.wsk + (int64_t)n * a.wsn;
            float qf;
            int qi = 0;
            if (w_is_float) {
                qf = load_as_float(a.w, a.w_dt, widx);
            } else {
                int64_t word = load_word(a.w, a.w_dt, widx);
                if (a.e > 1) word = (word >> ((k % a.e) * a.nbits)) & (int64_t)a.mask;
                qi = (int)word;
                qf = (float)qi;
            }
            if (int_acc) {
                const int wi = has_zero ? (qi - (int)z) : qi;
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const int m = m0 + r;
                    if (m < a.M)
                        iacc[r] += (int)((const int8_t*)a.x)[(int64_t)m * a.xsm + (int64_t)k * a.xsk] * wi;
                }
            } else {
                float wv;
                switch (a.wgm) {
                    case GLA_WGM_SHIFT: wv = qf - z; break;
                    case GLA_WGM_SCALE: wv = qf * s; break;
                    case GLA_WGM_SHIFT_SCALE: wv = (qf - z) * s; break;
                    case GLA_WGM_FMA: wv = __builtin_fmaf(qf, s, z); break;
                    default: wv = qf; break;
                }
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const int m = m0 + r;
                    if (m < a.M)
                        facc[r] = __builtin_fmaf(
                            load_as_float(a.x, a.in_dt, (int64_t)m * a.xsm + (int64_t)k * a.xsk), wv, facc[r]);
                }
            }
        }
    }

    float sb = 1.0f;
    if (a.csm == GLA_CSM_WEIGHT || a.csm == GLA_CSM_BOTH) sb = load_as_float(a.scales, a.meta_dt, n);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        const int m = m0 + r;
        if (m >= a.M) continue;
        const int64_t oidx = (int64_t)m * a.osm + (int64_t)n * a.osn;
        if (int_acc && a.csm == GLA_CSM_NONE && a.out_dt == GLA_DT_INT32) {
            ((int32_t*)a.out)[oidx] = iacc[r];
            continue;
        }
        float v = int_acc ? (float)iacc[r] : facc[r];
        float sa = 1.0f;
        if (a.csm == GLA_CSM_ACTIVATION || a.csm == GLA_CSM_BOTH)
            sa = load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm);
        if (a.csm == GLA_CSM_WEIGHT) v *= sb;
        else if (a.csm == GLA_CSM_ACTIVATION) v *= sa;
        else if (a.csm == GLA_CSM_BOTH) v *= (sa * sb);
        store_from_float(a.out, a.out_dt, oidx, v);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Packed int32 words x fp16 / bf16 activations, any group size that is a whole number of words: the arithmetic of
// generic_int_kernel for the packings whose groups are shorter than one step of the tuned kernels (1-bit codes in
// groups of 32 or 64, 2-bit codes in groups of 16 or 32, ...).  One lane per output column as there, but the K range
// is split over the 16 waves of a workgroup, every word is loaded once, the activations of a word come as 128-bit
// loads, and the group's scale and zero are applied to the two sums of a group segment (sum x q, sum x) instead of
// to every code; the waves' partial sums meet in LDS and are added in wave order.
constexpr int kPackedWaves = 16;

template <int NBITS, bool BF16, int RP>
__global__ __launch_bounds__(64 * kPackedWaves) void generic_packed_kernel(GenericArgs a) {
    constexpr int E = 32 / NBITS;            // codes per word
    constexpr int CH = E < 8 ? E : 8;        // activations per load (4 for byte codes)
    constexpr uint32_t MASK = (1u << NBITS) - 1u;
    __shared__ float red[kPackedWaves][RP][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n_raw = blockIdx.x * 64 + lane;
    const int n = n_raw < a.N ? n_raw : a.N - 1;  // lanes past N repeat the last column and store nothing
    const int R = a.K / E;                         // word rows
    const int gw = a.wgm == GLA_WGM_NONE ? R : a.gs / E;  // word rows per group
    const int rpw = (R + kPackedWaves - 1) / kPackedWaves;
    int r = wv * rpw;
    const int r_end = r + rpw < R ? r + rpw : R;
    const bool has_scale = (a.wgm == GLA_WGM_SCALE || a.wgm == GLA_WGM_SHIFT_SCALE || a.wgm == GLA_WGM_FMA);
    const bool has_zero = (a.wgm == GLA_WGM_SHIFT || a.wgm == GLA_WGM_SHIFT_SCALE || a.wgm == GLA_WGM_FMA);
    // row blocks of RP rows: the grid's second dimension strides over them (it is capped at 65535 blocks)
    for (int m0 = blockIdx.y * RP; m0 < a.M; m0 += gridDim.y * RP) {
    r = wv * rpw;
    const uint16_t* xrow[RP];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) {
        const int m = m0 + rr < a.M ? m0 + rr : a.M - 1;
        xrow[rr] = (const uint16_t*)a.x + (int64_t)m * a.xsm;
    }
    const uint32_t* wcol = (const uint32_t*)a.w + n;
    float tot[RP];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) tot[rr] = 0.0f;
    while (r < r_end) {
        const int g = r / gw;
        int seg_end = (g + 1) * gw;
        if (seg_end > r_end) seg_end = r_end;
        float s = 1.0f, z = 0.0f;
        if (has_scale) s = load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + (int64_t)n * a.msn);
        if (has_zero)
            z = a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0)
                           : load_as_float(a.zeros, a.z_dt, (int64_t)g * a.msg + (int64_t)n * a.msn);
        float acc[RP], xs[RP];
#pragma unroll
        for (int rr = 0; rr < RP; ++rr) acc[rr] = xs[rr] = 0.0f;
        for (; r < seg_end; ++r) {
            const uint32_t word = wcol[(int64_t)r * a.wsk];
#pragma unroll
            for (int c = 0; c < E / CH; ++c) {
                uint32_t xw[RP][CH / 2];
#pragma unroll
                for (int rr = 0; rr < RP; ++rr) {
                    const uint16_t* src = xrow[rr] + (int64_t)r * E + c * CH;
                    if constexpr (CH == 8) {
                        const uint4 v = *(const uint4*)src;
                        xw[rr][0] = v.x; xw[rr][1] = v.y; xw[rr][2] = v.z; xw[rr][3] = v.w;
                    } else {
                        const uint2 v = *(const uint2*)src;
                        xw[rr][0] = v.x; xw[rr][1] = v.y;
                    }
                }
#pragma unroll
                for (int j = 0; j < CH; ++j) {
                    const float qf = (float)((word >> ((c * CH + j) * NBITS)) & MASK);
#pragma unroll
                    for (int rr = 0; rr < RP; ++rr) {
                        const uint16_t bits = (uint16_t)(xw[rr][j / 2] >> ((j % 2) * 16));
                        const float xv = BF16 ? bf16_bits_to_float(bits) : half_bits_to_float(bits);
                        acc[rr] = __builtin_fmaf(xv, qf, acc[rr]);
                        xs[rr] += xv;
                    }
                }
            }
        }
#pragma unroll
        for (int rr = 0; rr < RP; ++rr) {
            float v;
            switch (a.wgm) {
                case GLA_WGM_SHIFT: v = __builtin_fmaf(-z, xs[rr], acc[rr]); break;
                case GLA_WGM_SCALE: v = s * acc[rr]; break;
                case GLA_WGM_SHIFT_SCALE: v = s * __builtin_fmaf(-z, xs[rr], acc[rr]); break;
                case GLA_WGM_FMA: v = __builtin_fmaf(s, acc[rr], z * xs[rr]); break;
                default: v = acc[rr]; break;
            }
            tot[rr] += v;
        }
    }
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) red[wv][rr][lane] = tot[rr];
    __syncthreads();
    if (wv == 0 && n_raw < a.N) {
    float sb = 1.0f;
    if (a.csm == GLA_CSM_WEIGHT || a.csm == GLA_CSM_BOTH) sb = load_as_float(a.scales, a.meta_dt, n);
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) {
        const int m = m0 + rr;
        if (m >= a.M) continue;
        float v = 0.0f;
        for (int w = 0; w < kPackedWaves; ++w) v += red[w][rr][lane];
        float sa = 1.0f;
        if (a.csm == GLA_CSM_ACTIVATION || a.csm == GLA_CSM_BOTH) sa = load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm);
        if (a.csm == GLA_CSM_WEIGHT) v *= sb;
        else if (a.csm == GLA_CSM_ACTIVATION) v *= sa;
        else if (a.csm == GLA_CSM_BOTH) v *= (sa * sb);
        store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)n * a.osn, v);
    }
    }
    __syncthreads();  // the next row block reuses the reduction buffer
    }
}

// what generic_packed_kernel assumes of a call
bool packed_words_ok(const gla_matmul_args& p) {
    if (p.w_dtype != GLA_DT_INT32 || p.w == nullptr || p.x == nullptr) return false;
    if (!(p.W_nbits == 1 || p.W_nbits == 2 || p.W_nbits == 4 || p.W_nbits == 8)) return false;
    const int E = 32 / p.W_nbits;
    if (p.elements_per_sample != E || p.unpack_mask != (1 << p.W_nbits) - 1) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16) || p.acc_dtype != GLA_DT_FP32) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.W_group_mode < GLA_WGM_NONE || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.M < 1 || p.N < 1 || p.K < E || p.K % E != 0 || p.K % 8 != 0) return false;
    if (p.x_stride_k != 1 || p.w_stride_n != 1 || p.x_stride_m % 8 != 0 || ((uintptr_t)p.x & 15)) return false;
    if (p.W_group_mode != GLA_WGM_NONE && (p.group_size < E || p.group_size % E != 0 || p.K % p.group_size != 0)) return false;
    const bool has_scale = p.W_group_mode == GLA_WGM_SCALE || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    const bool has_zero = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if ((has_scale || (p.channel_scale_mode & 1)) && p.scales == nullptr) return false;
    if (has_zero && p.zeros == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

template <int NBITS, bool BF16>
void launch_packed_rows(const GenericArgs& a, hipStream_t stream) {
    const int rp = a.M >= 3 ? 4 : a.M;
    const int row_blocks = ceil_div(a.M, rp);
    const dim3 grid(ceil_div(a.N, 64), row_blocks < 65535 ? row_blocks : 65535), block(64 * kPackedWaves);
    if (rp == 4) hipLaunchKernelGGL((generic_packed_kernel<NBITS, BF16, 4>), grid, block, 0, stream, a);
    else if (rp == 2) hipLaunchKernelGGL((generic_packed_kernel<NBITS, BF16, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((generic_packed_kernel<NBITS, BF16, 1>), grid, block, 0, stream, a);
}

template <bool BF16>
void launch_packed_bits(const GenericArgs& a, hipStream_t stream) {
    switch (a.nbits) {
        case 1: return launch_packed_rows<1, BF16>(a, stream);
        case 2: return launch_packed_rows<2, BF16>(a, stream);
        case 4: return launch_packed_rows<4, BF16>(a, stream);
        default: return launch_packed_rows<8, BF16>(a, stream);
    }
}

// 16-bit weights [K, N] (no codes, no groups) x 16-bit activations: the same K split over 16 waves, 8 K-values per
// step with their 8 weight loads in flight together.
template <bool WBF16, bool XBF16, int RP>
__global__ __launch_bounds__(64 * kPackedWaves) void generic_w16_kernel(GenericArgs a) {
    __shared__ float red[kPackedWaves][RP][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n_raw = blockIdx.x * 64 + lane;
    const int n = n_raw < a.N ? n_raw : a.N - 1;
    const int m0 = blockIdx.y * RP;
    const int steps = a.K / 8;
    const int spw = (steps + kPackedWaves - 1) / kPackedWaves;
    const int s_end = (wv + 1) * spw < steps ? (wv + 1) * spw : steps;
    const uint16_t* xrow[RP];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) {
        const int m = m0 + rr < a.M ? m0 + rr : a.M - 1;
        xrow[rr] = (const uint16_t*)a.x + (int64_t)m * a.xsm;
    }
    const uint16_t* wcol = (const uint16_t*)a.w + n;
    float acc[RP];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) acc[rr] = 0.0f;
    for (int st = wv * spw; st < s_end; ++st) {
        uint16_t wb[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) wb[j] = wcol[(int64_t)(st * 8 + j) * a.wsk];
        uint32_t xw[RP][4];
#pragma unroll
        for (int rr = 0; rr < RP; ++rr) {
            const uint4 v = *(const uint4*)(xrow[rr] + (int64_t)st * 8);
            xw[rr][0] = v.x; xw[rr][1] = v.y; xw[rr][2] = v.z; xw[rr][3] = v.w;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float wf = WBF16 ? bf16_bits_to_float(wb[j]) : half_bits_to_float(wb[j]);
#pragma unroll
            for (int rr = 0; rr < RP; ++rr) {
                const uint16_t bits = (uint16_t)(xw[rr][j / 2] >> ((j % 2) * 16));
                acc[rr] = __builtin_fmaf(XBF16 ? bf16_bits_to_float(bits) : half_bits_to_float(bits), wf, acc[rr]);
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) red[wv][rr][lane] = acc[rr];
    __syncthreads();
    if (wv != 0 || n_raw >= a.N) return;
    float sb = 1.0f;
    if (a.csm == GLA_CSM_WEIGHT || a.csm == GLA_CSM_BOTH) sb = load_as_float(a.scales, a.meta_dt, n);
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) {
        const int m = m0 + rr;
        if (m >= a.M) continue;
        float v = 0.0f;
        for (int w = 0; w < kPackedWaves; ++w) v += red[w][rr][lane];
        float sa = 1.0f;
        if (a.csm == GLA_CSM_ACTIVATION || a.csm == GLA_CSM_BOTH) sa = load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm);
        if (a.csm == GLA_CSM_WEIGHT) v *= sb;
        else if (a.csm == GLA_CSM_ACTIVATION) v *= sa;
        else if (a.csm == GLA_CSM_BOTH) v *= (sa * sb);
        store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)n * a.osn, v);
    }
}

// what generic_w16_kernel assumes of a call
bool w16_ok(const gla_matmul_args& p) {
    if (!(p.w_dtype == GLA_DT_FP16 || p.w_dtype == GLA_DT_BF16) || p.w == nullptr || p.x == nullptr) return false;
    if (p.elements_per_sample != 1 || p.W_group_mode != GLA_WGM_NONE) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16) || p.acc_dtype != GLA_DT_FP32) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.M < 1 || p.N < 1 || p.K < 8 || p.K % 8 != 0) return false;
    if (p.x_stride_k != 1 || p.x_stride_m % 8 != 0 || ((uintptr_t)p.x & 15)) return false;
    // N contiguous, or K contiguous with rows that 128-bit loads can read
    const bool kmajor = p.w_stride_k == 1 && p.w_stride_n % 8 == 0 && !((uintptr_t)p.w & 15);
    if (p.w_stride_n != 1 && !kmajor) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

template <bool WBF16, bool XBF16>
void launch_w16_rows(const GenericArgs& a, hipStream_t stream) {
    const int rp = a.M >= 3 ? 4 : a.M;
    const dim3 grid(ceil_div(a.N, 64), ceil_div(a.M, rp)), block(64 * kPackedWaves);
    if (rp == 4) hipLaunchKernelGGL((generic_w16_kernel<WBF16, XBF16, 4>), grid, block, 0, stream, a);
    else if (rp == 2) hipLaunchKernelGGL((generic_w16_kernel<WBF16, XBF16, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((generic_w16_kernel<WBF16, XBF16, 1>), grid, block, 0, stream, a);
}

// 16-bit weights as the layer classes keep them, [N, K] with K contiguous: one wave per two output columns, the
// lanes along K with 128-bit loads, a butterfly sum over the wave at the end.
template <bool WBF16, bool XBF16, int RP>
__global__ __launch_bounds__(256) void generic_w16_kmajor_kernel(GenericArgs a) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wv) * 2;
    if (n0 >= a.N) return;  // (no barrier below)
    const bool two = n0 + 1 < a.N;
    const int m0 = blockIdx.y * RP;
    const uint16_t* wrow[2] = {(const uint16_t*)a.w + (int64_t)n0 * a.wsn, (const uint16_t*)a.w + (int64_t)(two ? n0 + 1 : n0) * a.wsn};
    const uint16_t* xrow[RP];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) {
        const int m = m0 + rr < a.M ? m0 + rr : a.M - 1;
        xrow[rr] = (const uint16_t*)a.x + (int64_t)m * a.xsm;
    }
    float acc[RP][2];
#pragma unroll
    for (int rr = 0; rr < RP; ++rr) acc[rr][0] = acc[rr][1] = 0.0f;
    for (int k = lane * 8; k < a.K; k += 512) {
        uint32_t ww[2][4];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const uint4 v = *(const uint4*)(wrow[c] + k);
            ww[c][0] = v.x; ww[c][1] = v.y; ww[c][2] = v.z; ww[c][3] = v.w;
        }
#pragma unroll
        for (int rr = 0; rr < RP; ++rr) {
            const uint4 v = *(const uint4*)(xrow[rr] + k);
            const uint32_t xw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint16_t xb = (uint16_t)(xw[j / 2] >> ((j % 2) * 16));
                const float xf = XBF16 ? bf16_bits_to_float(xb) : half_bits_to_float(xb);
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const uint16_t wb = (uint16_t)(ww[c][j / 2] >> ((j % 2) * 16));
                    acc[rr][c] = __builtin_fmaf(xf, WBF16 ? bf16_bits_to_float(wb) : half_bits_to_float(wb), acc[rr][c]);
                }
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < RP; ++rr)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) acc[rr][c] += __shfl_xor(acc[rr][c], off, 64);
    if (lane != 0) return;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        if (c == 1 && !two) break;
        const int n = n0 + c;
        float sb = 1.0f;
        if (a.csm == GLA_CSM_WEIGHT || a.csm == GLA_CSM_BOTH) sb = load_as_float(a.scales, a.meta_dt, n);
#pragma unroll
        for (int rr = 0; rr < RP; ++rr) {
            const int m = m0 + rr;
            if (m >= a.M) continue;
            float v = acc[rr][c], sa = 1.0f;
            if (a.csm == GLA_CSM_ACTIVATION || a.csm == GLA_CSM_BOTH) sa = load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm);
            if (a.csm == GLA_CSM_WEIGHT) v *= sb;
            else if (a.csm == GLA_CSM_ACTIVATION) v *= sa;
            else if (a.csm == GLA_CSM_BOTH) v *= (sa * sb);
            store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)n * a.osn, v);
        }
    }
}

template <bool WBF16, bool XBF16>
void launch_w16_kmajor_rows(const GenericArgs& a, hipStream_t stream) {
    const int rp = a.M >= 3 ? 4 : a.M;
    const dim3 grid(ceil_div(a.N, 8), ceil_div(a.M, rp)), block(256);
    if (rp == 4) hipLaunchKernelGGL((generic_w16_kmajor_kernel<WBF16, XBF16, 4>), grid, block, 0, stream, a);
    else if (rp == 2) hipLaunchKernelGGL((generic_w16_kmajor_kernel<WBF16, XBF16, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((generic_w16_kmajor_kernel<WBF16, XBF16, 1>), grid, block, 0, stream, a);
}

// e2m1 x e2m1 with e8m0 block scales on both operands (block = 32 along K).
__global__ __launch_bounds__(64) void generic_mxfp4_kernel(GenericArgs a) {
    const int n = blockIdx.x * 64 + threadIdx.x;
    const int m0 = blockIdx.y * kRows;
    if (n >= a.N) return;
    float acc[kRows] = {0.f, 0.f, 0.f, 0.f};
    const int blocks = a.K / 32;
    for (int b = 0; b < blocks; ++b) {
        const float sw = e8m0_to_float(((const uint8_t*)a.scales)[(int64_t)b * a.msg + (int64_t)n * a.msn]);
        float part[kRows] = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < 16; ++j) {
            const int kb = b * 16 + j;  // byte index along K
            const uint32_t wb = ((const uint8_t*)a.w)[(int64_t)kb * a.wsk + (int64_t)n * a.wsn];
            const float w0 = e2m1_to_float(wb & 15u), w1 = e2m1_to_float(wb >> 4);
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                const int m = m0 + r;
                if (m < a.M) {
                    const uint32_t xb = ((const uint8_t*)a.x)[(int64_t)m * a.xsm + (int64_t)kb * a.xsk];
                    part[r] += e2m1_to_float(xb & 15u) * w0 + e2m1_to_float(xb >> 4) * w1;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            const int m = m0 + r;
            if (m < a.M) {
                const float sa =
                    e8m0_to_float(((const uint8_t*)a.scales_x)[(int64_t)m * a.sxm + (int64_t)b * a.sxg]);
                acc[r] = __builtin_fmaf(part[r], sa * sw, acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        const int m = m0 + r;
        if (m < a.M) store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)n * a.osn, acc[r]);
    }
}

// out[m, n] = cast(out[m, n] + bias[n]): the reference's `out += bias` on the finished output
// (reference: gemlite/core.py:271-272), for the kernel families that do not add the bias themselves.
__global__ __launch_bounds__(256) void bias_add_kernel(void* out, const void* bias, int M, int N, int64_t osm, int64_t osn,
                                                       int out_dt, int bias_dt) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    const int64_t o = (int64_t)m * osm + (int64_t)n * osn;
    store_from_float(out, out_dt, o, load_as_float(out, out_dt, o) + load_as_float(bias, bias_dt, n));
}

// fp8-e4m3 / int8 activations -> dense fp16 rows (both convert exactly): 8 values per thread
__global__ __launch_bounds__(256) void widen_x8_kernel(const uint8_t* x, int64_t xsm, int M, int K, int in_dt, uint16_t* out, int64_t osm) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int per_row = (K + 7) / 8;
    if (t >= (int64_t)M * per_row) return;
    const int m = (int)(t / per_row), k0 = (int)(t % per_row) * 8;
    const uint8_t* src = x + (int64_t)m * xsm + k0;
    uint16_t* dst = out + (int64_t)m * osm + k0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (k0 + i >= K) break;
        const float v = in_dt == GLA_DT_INT8 ? (float)(int8_t)src[i] : load_as_float(src, GLA_DT_FP8, i);
        dst[i] = float_to_half_bits(v);
    }
}

}  // namespace

int launch_widen_x8(const void* x, int64_t x_stride_m, int M, int K, int input_dtype, void* out_f16, int64_t out_stride_m, hipStream_t stream) {
    const int64_t items = (int64_t)M * ((K + 7) / 8);
    hipLaunchKernelGGL(widen_x8_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, (const uint8_t*)x, x_stride_m, M,
                       K, input_dtype, (uint16_t*)out_f16, out_stride_m);
    return check_hip(hipGetLastError(), "activation widening launch");
}

int launch_bias_add(const gla_matmul_args& p, hipStream_t stream) {
    const int out_dt = p.output_dtype == GLA_DT_MXFP16 ? GLA_DT_FP16 : (p.output_dtype == GLA_DT_MXBF16 ? GLA_DT_BF16 : p.output_dtype);
    const int64_t items = (int64_t)p.M * p.N;
    hipLaunchKernelGGL(bias_add_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, p.out, p.bias, p.M, p.N,
                       p.out_stride_m, p.out_stride_n, out_dt, p.bias_dtype);
    return check_hip(hipGetLastError(), "bias add launch");
}

int launch_generic(const gla_matmul_args& p, hipStream_t stream) {
    // the kernels below put blocks of 1-4 rows on the grid's second dimension (at most 65535 blocks): very tall
    // problems run as slices of rows
    constexpr int kSliceRows = 65532;
    if (p.M > kSliceRows) {
        if (p.input_dtype == GLA_DT_MXFP4) {
            set_error("generic matmul: more than %d rows of MXFP4 activations are not sliced (two codes per byte)", kSliceRows);
            return GLA_ERR_MISALIGNED_SHAPE;
        }
        for (int m0 = 0; m0 < p.M; m0 += kSliceRows) {
            gla_matmul_args q = p;
            q.M = p.M - m0 < kSliceRows ? p.M - m0 : kSliceRows;
            auto bytes_of = [](int dt) { return (dt == GLA_DT_MXFP16 || dt == GLA_DT_MXBF16) ? 2 : dtype_size(dt); };
            q.x = (const char*)p.x + (int64_t)m0 * p.x_stride_m * bytes_of(p.input_dtype);
            q.out = (char*)p.out + (int64_t)m0 * p.out_stride_m * bytes_of(p.output_dtype);
            if (p.scales_x != nullptr) q.scales_x = (const char*)p.scales_x + (int64_t)m0 * p.sx_stride_m * dtype_size(p.sx_dtype);
            const int rc = launch_generic(q, stream);
            if (rc != GLA_OK) return rc;
        }
        return GLA_OK;
    }
    GenericArgs a;
    a.x = p.x; a.w = p.w; a.scales = p.scales; a.zeros = p.zeros; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K;
    a.xsm = p.x_stride_m; a.xsk = p.x_stride_k; a.wsk = p.w_stride_k; a.wsn = p.w_stride_n;
    a.osm = p.out_stride_m; a.osn = p.out_stride_n; a.msg = p.meta_stride_g; a.msn = p.meta_stride_n;
    a.sxm = p.sx_stride_m; a.sxg = p.sx_stride_g;
    a.nbits = p.W_nbits; a.gs = p.group_size; a.mask = p.unpack_mask; a.e = p.elements_per_sample;
    a.in_dt = p.input_dtype; a.out_dt = p.output_dtype; a.acc_dt = p.acc_dtype; a.meta_dt = p.meta_dtype;
    a.csm = p.channel_scale_mode; a.wgm = p.W_group_mode;
    a.w_dt = p.w_dtype; a.z_dt = p.zeros_dtype; a.z_scalar = p.zero_is_scalar; a.sx_dt = p.sx_dtype;

    dim3 grid(ceil_div(p.N, 64), ceil_div(p.M, kRows));
    if (p.input_dtype == GLA_DT_MXFP4) {
        if (p.channel_scale_mode != GLA_CSM_MX || p.scales == nullptr || p.scales_x == nullptr) {
            set_error("MXFP4 activations need channel_scale_mode 4 with both block-scale tensors");
            return GLA_ERR_UNSUPPORTED_MODE;
        }
        hipLaunchKernelGGL(generic_mxfp4_kernel, grid, dim3(64), 0, stream, a);
    } else if (w16_ok(p)) {
        const bool wb = p.w_dtype == GLA_DT_BF16, xb = p.input_dtype == GLA_DT_BF16;
        if (p.w_stride_n != 1) {
            if (wb && xb) launch_w16_kmajor_rows<true, true>(a, stream);
            else if (wb) launch_w16_kmajor_rows<true, false>(a, stream);
            else if (xb) launch_w16_kmajor_rows<false, true>(a, stream);
            else launch_w16_kmajor_rows<false, false>(a, stream);
        } else if (wb && xb) launch_w16_rows<true, true>(a, stream);
        else if (wb) launch_w16_rows<true, false>(a, stream);
        else if (xb) launch_w16_rows<false, true>(a, stream);
        else launch_w16_rows<false, false>(a, stream);
    } else if (packed_words_ok(p)) {
        if (p.input_dtype == GLA_DT_BF16) launch_packed_bits<true>(a, stream);
        else launch_packed_bits<false>(a, stream);
    } else {
        hipLaunchKernelGGL(generic_int_kernel, grid, dim3(64), 0, stream, a);
    }
    return check_hip(hipGetLastError(), "generic matmul launch");
}

}  // namespace gla
