// Block-quantised 8-bit matmul (channel_scale_mode 5): int8 x int8 or fp8-e4m3 x fp8-e4m3 with one
// fp32 weight scale per 128 x 128 block of the [N, K] weight and one fp32 activation scale per
// (row, 128 values along K):
//
//   out(m,n) = sum_kb ( sum_{k in block kb} a(m,k) w(n,k) ) * sa(m,kb) * sb(kb, n / 128)
//
// (reference: gemlite/triton_kernels/gemm_kernels.py:396-400 and :441-450: the dot product of one
//  K-block is scaled by both block scales and added to an fp32 accumulator; layer set-up in
//  gemlite/helper.py:517-617, activation quantiser gemlite/quant_utils.py:2614-2676.)
//
// Both operands are K-contiguous bytes.  One wave owns four output columns: lane l takes the
// 16-byte pieces l, l+64, ... of their weight rows (eight pieces make a 128-block) and multiplies
// them with the same pieces of up to eight activation rows.  int8 products are summed exactly
// (4-way integer dot instruction) before the two scales are applied in fp32; fp8 codes become fp16
// pairs (exact) and go through the packed dot instruction with fp32 accumulation.  A lane scales
// its own piece of a block rather than the block's whole sum, which is the same value up to fp32
// rounding.  A streaming kernel for decode-sized batches: every group of eight activation rows
// streams the weights again.
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

struct BqArgs {
    const uint8_t* x;
    const uint8_t* w;
    const float* scales;    // [K/128, ceil(N/128)] by strides
    const float* scales_x;  // [M, K/128] by strides
    void* out;
    int M, N, pieces;  // pieces = K / 16
    int64_t xsm, wsn, osm, osn, msg, msn, sxm, sxg;
    int out_dt;
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

typedef uint32_t u32x4q __attribute__((ext_vector_type(4)));

template <bool FP8>
__device__ __forceinline__ float dot16(const u32x4q& a, const u32x4q& b) {
    if constexpr (FP8) {
        float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t ad = d == 0 ? a.x : d == 1 ? a.y : d == 2 ? a.z : a.w;
            const uint32_t bd = d == 0 ? b.x : d == 1 ? b.y : d == 2 ? b.z : b.w;
            p0 = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ad, 1.0f, false),
                                        __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(bd, 1.0f, false), p0, false);
            p1 = __builtin_amdgcn_fdot2(__builtin_amdgcn_cvt_scalef32_pk_f16_fp8(ad, 1.0f, true),
                                        __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(bd, 1.0f, true), p1, false);
        }
        return p0 + p1;
    } else {
        int s = __builtin_amdgcn_sdot4((int)a.x, (int)b.x, 0, false);
        s = __builtin_amdgcn_sdot4((int)a.y, (int)b.y, s, false);
        s = __builtin_amdgcn_sdot4((int)a.z, (int)b.z, s, false);
        s = __builtin_amdgcn_sdot4((int)a.w, (int)b.w, s, false);
        return (float)s;
    }
}

template <bool FP8, int RM, int NC>
__global__ __launch_bounds__(256) void blockq_stream_kernel(BqArgs a) {
    const int lane = threadIdx.x & 63;
    const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * NC;
    const int m0 = blockIdx.y * RM;
    if (n0 >= a.N) return;  // whole waves leave; no barrier follows

    // columns past N repeat the last one (loaded, never stored)
    const uint8_t* wrow[NC];
    const float* srow[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int n = n0 + c < a.N ? n0 + c : a.N - 1;
        wrow[c] = a.w + (int64_t)n * a.wsn;
        srow[c] = a.scales + (int64_t)(n / 128) * a.msn;
    }
    float acc[RM][NC];
#pragma unroll
    for (int r = 0; r < RM; ++r)
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[r][c] = 0.0f;

    for (int pc = lane; pc < a.pieces; pc += 64) {
        const int kb = pc >> 3;
        u32x4q wv[NC];
        float sb[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            wv[c] = *(const u32x4q*)(wrow[c] + (int64_t)pc * 16);
            sb[c] = srow[c][(int64_t)kb * a.msg];
        }
#pragma unroll
        for (int r = 0; r < RM; ++r) {
            const int m = m0 + r;
            if (m < a.M) {
                const u32x4q xv = *(const u32x4q*)(a.x + (int64_t)m * a.xsm + (int64_t)pc * 16);
                const float sa = a.scales_x[(int64_t)m * a.sxm + (int64_t)kb * a.sxg];
#pragma unroll
                for (int c = 0; c < NC; ++c) acc[r][c] = __builtin_fmaf(dot16<FP8>(xv, wv[c]), sa * sb[c], acc[r][c]);
            }
        }
    }

#pragma unroll
    for (int r = 0; r < RM; ++r) {
        const int m = m0 + r;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float v = acc[r][c];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += wave_xor(v, off);
            if (lane == 0 && m < a.M && n0 + c < a.N) {
                if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n0 + c);
                store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)(n0 + c) * a.osn, v);
            }
        }
    }
}

constexpr int kColsQ = 4;

template <bool FP8>
void launch_rows_q(const BqArgs& a, int rm, dim3 grid, hipStream_t s) {
    // narrow layers (fewer than 512 workgroups at 4 columns per wave: 4 waves per CU or less): 2 columns per wave
    if (rm <= 2 && ceil_div(a.N, 4 * kColsQ) < 512) {
        const dim3 g2(ceil_div(a.N, 4 * 2), grid.y);
        if (rm == 1) hipLaunchKernelGGL((blockq_stream_kernel<FP8, 1, 2>), g2, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((blockq_stream_kernel<FP8, 2, 2>), g2, dim3(256), 0, s, a);
        return;
    }
    if (rm == 1) hipLaunchKernelGGL((blockq_stream_kernel<FP8, 1, kColsQ>), grid, dim3(256), 0, s, a);
    else if (rm == 2) hipLaunchKernelGGL((blockq_stream_kernel<FP8, 2, kColsQ>), grid, dim3(256), 0, s, a);
    else if (rm == 4) hipLaunchKernelGGL((blockq_stream_kernel<FP8, 4, kColsQ>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((blockq_stream_kernel<FP8, 8, kColsQ>), grid, dim3(256), 0, s, a);
}

}  // namespace

bool blockq_stream_eligible(const gla_matmul_args& p) {
    if (p.channel_scale_mode != GLA_CSM_BLOCK || p.W_group_mode != GLA_WGM_NONE) return false;
    if (!(p.input_dtype == GLA_DT_INT8 || p.input_dtype == GLA_DT_FP8) || p.w_dtype != p.input_dtype) return false;
    if (p.W_nbits != 8 || p.elements_per_sample != 1 || p.K % 128 != 0) return false;
    if (p.scales == nullptr || p.scales_x == nullptr || p.meta_dtype != GLA_DT_FP32 || p.sx_dtype != GLA_DT_FP32) return false;
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    switch (p.output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: return true;
        default: return false;
    }
}

int launch_blockq_stream(const gla_matmul_args& p, hipStream_t stream) {
    if (!blockq_stream_eligible(p)) {
        set_error("blockq_stream: needs int8 or fp8 operands, both K-contiguous with 16-byte aligned rows, "
                  "K %% 128 == 0 and fp32 block scales on both sides");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    BqArgs a;
    a.x = (const uint8_t*)p.x; a.w = (const uint8_t*)p.w;
    a.scales = (const float*)p.scales; a.scales_x = (const float*)p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.pieces = p.K / 16;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.osn = p.out_stride_n;
    a.msg = p.meta_stride_g; a.msn = p.meta_stride_n; a.sxm = p.sx_stride_m; a.sxg = p.sx_stride_g;
    a.out_dt = p.output_dtype;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    const int rm = p.M >= 5 ? 8 : (p.M >= 3 ? 4 : p.M);
    dim3 grid(ceil_div(p.N, 4 * kColsQ), ceil_div(p.M, rm));
    if (p.input_dtype == GLA_DT_FP8) launch_rows_q<true>(a, rm, grid, stream);
    else launch_rows_q<false>(a, rm, grid, stream);
    return check_hip(hipGetLastError(), "blockq_stream launch");
}

}  // namespace gla
