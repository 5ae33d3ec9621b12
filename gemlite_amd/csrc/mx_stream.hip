// Streaming kernel for the micro-scaled (MX) formats whose operands are both K-contiguous:
//
//   activations  fp16 | bf16 (weight-only layers) | fp8-e4m3 bytes | e2m1 nibble pairs
//   weights      fp8-e4m3 bytes | e2m1 nibble pairs, one e8m0 scale per 32 values along K
//   act scales   none | one fp32 per row applied after the K sum | one e8m0 per 32 values
//
//   out(m,n) = sum_blocks ( sum_{k in block} a(m,k) w(n,k) ) * 2^(sw(n,block)-127) * 2^(sa(m,block)-127)
//
// (reference: gemlite/triton_kernels/gemm_kernels.py:509-737 and gemm_splitK_kernels.py:536-770:
//  `tl.dot_scaled(a, scales_a, a_dtype, b, scales_b, b_dtype, acc)` with a_dtype in
//  {fp16, bf16, e4m3, e2m1}, b_dtype in {e4m3, e2m1}, unit activation scales unless
//  channel_scale_mode is 4, and the per-row activation scale of channel_scale_mode 2 at :714-717.)
//
// One wave owns four output columns: lane l takes the 32-blocks l, l+64, ... of their weight rows
// (16 or 32 contiguous bytes per block and row, so a wave reads 1-2 KiB of consecutive bytes of
// each row per step) and multiplies them with the same blocks of up to eight activation rows, an
// activation block being loaded once for the four columns.  Codes become
// fp16 (bf16 for bf16 activations) pairs with the conversion instructions of gfx950 — exact, both
// code sets are subsets of either type — and pairs are multiplied and summed in fp32 by the packed
// dot instruction; the block's partial sum is then scaled once by the product of its two block
// scales, as the scaled matrix instruction does.  A shuffle tree sums the lanes.
//
// This is the decode path of every micro-scaled layer: weight-only MX layers up to 2 rows, MXFP4 x
// MXFP4 up to 2 rows (4 on layers of 40 MB or less), fp8 activations on MXFP4 or MXFP8 weights up to
// 4 rows (above that the matrix-core kernels are faster: the conversions and dot products here cost
// vector-unit time per row); and the path at any batch size for a K that the matrix-core kernels do not take (not tuned above
// a few rows: every group of eight activation rows streams the weights again).
#include "common.hpp"
#include "dispatch.hpp"
#include "actquant_device.hpp"

namespace gla {

namespace {

// A_Q4F16 / A_Q4BF16: fp16 / bf16 rows that the kernel quantises to MXFP4 itself, block by block, with the
// arithmetic of the activation quantiser (same codes, same e8m0 bytes), in place of a quantiser launch in front
enum { A_F16 = 0, A_BF16 = 1, A_FP8 = 2, A_FP4 = 3, A_Q4F16 = 4, A_Q4BF16 = 5 };
enum { B_FP8 = 0, B_FP4 = 1 };

struct MxArgs {
    const uint8_t* x;
    const uint8_t* w;
    const uint8_t* scales;
    const void* scales_x;
    void* out;
    int M, N, KB;  // KB = K / 32
    int64_t xsm_bytes, wsn_bytes, osm, osn, msg, msn, sxm, sxg;
    int csm, out_dt;
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <bool BF>
struct Pair {
    using type = half2_t;
};
template <>
struct Pair<true> {
    using type = bf16x2_t;
};

template <bool BF>
__device__ __forceinline__ float dot2(typename Pair<BF>::type a, typename Pair<BF>::type b, float c) {
    if constexpr (BF) return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
    else return __builtin_amdgcn_fdot2(a, b, c, false);
}

// The 32 values of one block as 16 pairs (k, k+1), from e2m1 nibbles (16 bytes) ...
template <bool BF>
__device__ __forceinline__ void block_from_fp4(const u32x4 q, typename Pair<BF>::type (&v)[16]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        if constexpr (BF) {
            v[4 * d + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], 1.0f, 0);
            v[4 * d + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], 1.0f, 1);
            v[4 * d + 2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], 1.0f, 2);
            v[4 * d + 3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], 1.0f, 3);
        } else {
            v[4 * d + 0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[d], 1.0f, 0);
            v[4 * d + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[d], 1.0f, 1);
            v[4 * d + 2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[d], 1.0f, 2);
            v[4 * d + 3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q[d], 1.0f, 3);
        }
    }
}

// ... from e4m3 bytes (32 bytes) ...
template <bool BF>
__device__ __forceinline__ void block_from_fp8(const u32x4 q0, const u32x4 q1, typename Pair<BF>::type (&v)[16]) {
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        const uint32_t w = d < 4 ? q0[d & 3] : q1[d & 3];
        if constexpr (BF) {
            v[2 * d + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
            v[2 * d + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
        } else {
            v[2 * d + 0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
            v[2 * d + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
        }
    }
}

// ... or taken as they lie (64 bytes of fp16 / bf16).
template <bool BF>
__device__ __forceinline__ void block_from_16bit(const u32x4 (&raw)[4], typename Pair<BF>::type (&v)[16]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const u32x4 q = raw[d];
        // element copies first: a bit cast applied to `q[j]` directly took element 0 for every j
        const uint32_t q0 = q.x, q1 = q.y, q2 = q.z, q3 = q.w;
        v[4 * d + 0] = __builtin_bit_cast(typename Pair<BF>::type, q0);
        v[4 * d + 1] = __builtin_bit_cast(typename Pair<BF>::type, q1);
        v[4 * d + 2] = __builtin_bit_cast(typename Pair<BF>::type, q2);
        v[4 * d + 3] = __builtin_bit_cast(typename Pair<BF>::type, q3);
    }
}

// One 32-block of 16-bit activations -> its MXFP4 codes (16 bytes, as the quantiser stores them) and e8m0 byte.
template <bool XBF>
__device__ __forceinline__ u32x4 quantise_block_mxfp4(const u32x4 (&raw)[4], uint32_t& e) {
    float v[4][8];
    float amax = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t w = raw[d][j];
            if constexpr (XBF) {
                v[d][2 * j] = __builtin_bit_cast(float, w << 16);
                v[d][2 * j + 1] = __builtin_bit_cast(float, w & 0xffff0000u);
            } else {
                v[d][2 * j] = half_bits_to_float((uint16_t)(w & 0xffffu));
                v[d][2 * j + 1] = half_bits_to_float((uint16_t)(w >> 16));
            }
            amax = fmaxf(amax, fmaxf(fabsf(v[d][2 * j]), fabsf(v[d][2 * j + 1])));
        }
    e = e8m0_of_amax<false>(amax);
    u32x4 codes;
#pragma unroll
    for (int d = 0; d < 4; ++d) codes[d] = mxfp4_pack8<true>(v[d], e);
    return codes;
}

// NC output columns per wave, RM activation rows per workgroup row.
template <int AK, int BK, int RM, int NC>
__global__ __launch_bounds__(256) void mx_stream_kernel(MxArgs a) {
    constexpr bool BF = (AK == A_BF16);
    constexpr bool QUANT = AK == A_Q4F16 || AK == A_Q4BF16;
    using pair_t = typename Pair<BF>::type;
    constexpr int kABytes = AK == A_FP4 ? 16 : (AK == A_FP8 ? 32 : 64);
    constexpr int kBBytes = BK == B_FP4 ? 16 : 32;

    const int lane = threadIdx.x & 63;
    const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * NC;
    const int m0 = blockIdx.y * RM;
    if (n0 >= a.N) return;  // whole waves leave; no barrier follows

    // columns past N repeat the last one (loaded, never stored)
    const uint8_t* wrow[NC];
    const uint8_t* srow[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int n = n0 + c < a.N ? n0 + c : a.N - 1;
        wrow[c] = a.w + (int64_t)n * a.wsn_bytes;
        srow[c] = a.scales + (int64_t)n * a.msn;
    }
    float acc[RM][NC];
#pragma unroll
    for (int r = 0; r < RM; ++r)
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[r][c] = 0.0f;

    // One step = the wave's 64 blocks at blk, blk + 64, ...; the weight bytes and scale bytes of step
    // i + 1 (and the activation blocks too while they fit eight 16-byte registers) are requested before step i is
    // multiplied, so that a wave always has two steps' loads in flight.  Weights are read once per
    // launch: streaming (non-temporal) loads.
    constexpr int WQ = kBBytes / 16;  // 16-byte pieces of a weight block
    constexpr int AQ = kABytes / 16;
    constexpr bool XPRE = RM * AQ <= 8;  // activation blocks ride along with the prefetch (up to 8 registers quads)
    struct Step {
        u32x4 w[NC][WQ];
        uint8_t s[NC];
        u32x4 x[XPRE ? RM : 1][AQ];
        uint8_t sa[XPRE ? RM : 1];
    };
    auto fetch = [&](int blk, Step& st) __attribute__((always_inline)) {
        const int b = blk < a.KB ? blk : a.KB - 1;  // lanes past the end re-read the last block and drop it
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int q = 0; q < WQ; ++q) {
                const uint4 t = load_streaming_u4(wrow[c] + (int64_t)b * kBBytes + 16 * q);
                st.w[c][q] = u32x4{t.x, t.y, t.z, t.w};
            }
            st.s[c] = srow[c][(int64_t)b * a.msg];
        }
        if constexpr (XPRE) {
#pragma unroll
            for (int r = 0; r < RM; ++r) {
                const int m = m0 + r < a.M ? m0 + r : a.M - 1;
                const uint8_t* xp = a.x + (int64_t)m * a.xsm_bytes + (int64_t)b * kABytes;
#pragma unroll
                for (int q = 0; q < AQ; ++q) st.x[r][q] = *(const u32x4*)(xp + 16 * q);
                if constexpr (!QUANT)
                    st.sa[r] = a.csm == GLA_CSM_MX ? ((const uint8_t*)a.scales_x)[(int64_t)m * a.sxm + (int64_t)b * a.sxg] : (uint8_t)127;
            }
        }
    };
    // (quantised on the fly: `e` receives the block's e8m0 byte)
    auto to_pairs_a = [&](const u32x4 (&raw)[AQ], pair_t (&xv)[16], uint32_t& e) __attribute__((always_inline)) {
        if constexpr (QUANT) block_from_fp4<BF>(quantise_block_mxfp4<AK == A_Q4BF16>(raw, e), xv);
        else if constexpr (AK == A_FP4) block_from_fp4<BF>(raw[0], xv);
        else if constexpr (AK == A_FP8) block_from_fp8<BF>(raw[0], raw[1], xv);
        else block_from_16bit<BF>(raw, xv);
    };
    auto multiply = [&](int blk, const Step& st) __attribute__((always_inline)) {
        if (blk >= a.KB) return;
        pair_t wv[NC][16];
        float sw[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if constexpr (BK == B_FP4) block_from_fp4<BF>(st.w[c][0], wv[c]);
            else block_from_fp8<BF>(st.w[c][0], st.w[c][WQ - 1], wv[c]);
            sw[c] = e8m0_to_float(st.s[c]);
        }
#pragma unroll
        for (int r = 0; r < RM; ++r) {
            const int m = m0 + r;
            if (m < a.M) {
                pair_t xv[16];
                float sa = 1.0f;
                uint32_t eq = 127;
                if constexpr (XPRE) {
                    to_pairs_a(st.x[r], xv, eq);
                    if constexpr (QUANT) sa = e8m0_to_float((uint8_t)eq);
                    else if (a.csm == GLA_CSM_MX) sa = e8m0_to_float(st.sa[r]);
                } else {
                    const uint8_t* xp = a.x + (int64_t)m * a.xsm_bytes + (int64_t)blk * kABytes;
                    u32x4 raw[AQ];
#pragma unroll
                    for (int q = 0; q < AQ; ++q) raw[q] = *(const u32x4*)(xp + 16 * q);
                    to_pairs_a(raw, xv, eq);
                    if constexpr (QUANT) sa = e8m0_to_float((uint8_t)eq);
                    else if (a.csm == GLA_CSM_MX)
                        sa = e8m0_to_float(((const uint8_t*)a.scales_x)[(int64_t)m * a.sxm + (int64_t)blk * a.sxg]);
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    float p0 = 0.0f, p1 = 0.0f;
#pragma unroll
                    for (int j = 0; j < 16; j += 2) {
                        p0 = dot2<BF>(xv[j], wv[c][j], p0);
                        p1 = dot2<BF>(xv[j + 1], wv[c][j + 1], p1);
                    }
                    acc[r][c] = __builtin_fmaf(p0 + p1, sw[c] * sa, acc[r][c]);
                }
            }
        }
    };
    {
        Step cur, nxt;
        fetch(lane, cur);
        for (int blk = lane; blk < a.KB + lane; blk += 128) {  // two steps per trip: the buffers alternate
            fetch(blk + 64, nxt);
            multiply(blk, cur);
            fetch(blk + 128, cur);
            multiply(blk + 64, nxt);
        }
    }

#pragma unroll
    for (int r = 0; r < RM; ++r) {
        const int m = m0 + r;
        float rs = 1.0f;
        if (a.csm == GLA_CSM_ACTIVATION && m < a.M) rs = ((const float*)a.scales_x)[(int64_t)m * a.sxm];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float v = acc[r][c];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += wave_xor(v, off);
            if (lane == 0 && m < a.M && n0 + c < a.N) {
                v *= rs;
                if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n0 + c);
                store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + (int64_t)(n0 + c) * a.osn, v);
            }
        }
    }
}

int a_kind(const gla_matmul_args& p) {
    switch (p.input_dtype) {
        case GLA_DT_MXFP16: return A_F16;
        case GLA_DT_MXBF16: return A_BF16;
        case GLA_DT_MXFP8: return A_FP8;
        case GLA_DT_MXFP4:
            return p.x_quant_from == GLA_DT_FP16 ? A_Q4F16 : (p.x_quant_from == GLA_DT_BF16 ? A_Q4BF16 : A_FP4);
        default: return -1;
    }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

constexpr int kCols = 4;  // output columns per wave

template <int AK, int BK>
void launch_rows(const MxArgs& a, int rm, dim3 grid, hipStream_t s) {
    // Narrow layers: with 4 columns per wave a layer of 4096 columns is 1024 waves, 4 per CU, too few to keep the
    // loads of a CU in flight.  1-2 rows then take 2 columns per wave (2048 x 8192: MXFP4 x MXFP4 7.1 -> 5.8 us, fp8 x
    // MXFP8 8.7 -> 6.3; 4096^2 7-15 % faster).  16-bit activations, which weigh as much as two columns of MXFP4
    // weights, only up to K = 8192 (4096 x 14336 was 6-9 % slower with them read twice as often).
    // (Rows quantised in the kernel: 8 columns per wave, which would halve the quantising work per column, measured
    // slower than 4: 16384^2 at one row 40.5 against 35.9 us.)
    if (rm <= 2 && ceil_div(a.N, 4 * kCols) < 512 && (AK == A_FP8 || AK == A_FP4 || a.KB <= 8192 / 32)) {
        const dim3 g2(ceil_div(a.N, 4 * 2), grid.y);
        if (rm == 1) hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 1, 2>), g2, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 2, 2>), g2, dim3(256), 0, s, a);
        return;
    }
    if (rm == 1) hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 1, kCols>), grid, dim3(256), 0, s, a);
    else if (rm == 2) hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 2, kCols>), grid, dim3(256), 0, s, a);
    else if (rm == 4) hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 4, kCols>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((mx_stream_kernel<AK, BK, 8, kCols>), grid, dim3(256), 0, s, a);
}

template <int AK>
void launch_b(const MxArgs& a, int bk, int rm, dim3 grid, hipStream_t s) {
    if (bk == B_FP4) launch_rows<AK, B_FP4>(a, rm, grid, s);
    else launch_rows<AK, B_FP8>(a, rm, grid, s);
}

}  // namespace

bool mx_stream_eligible(const gla_matmul_args& p) {
    const int ak = a_kind(p);
    if (ak < 0 || p.group_size != 32 || p.K % 32 != 0) return false;
    if (p.elements_per_sample != 1 && p.elements_per_sample != 2) return false;
    if (p.W_nbits != (p.elements_per_sample == 2 ? 4 : 8)) return false;
    if (p.scales == nullptr || p.x_stride_k != 1 || p.w_stride_k != 1) return false;
    // x_stride_m counts stored elements (bytes for the 8- and 4-bit kinds, 16-bit words otherwise)
    const int64_t xsm_bytes = p.x_stride_m * ((ak <= A_BF16 || ak >= A_Q4F16) ? 2 : 1);
    if (p.x_quant_from && ak < A_Q4F16) return false;  // only MXFP4 activations are made here
    if (ak >= A_Q4F16) return p.channel_scale_mode == GLA_CSM_MX && p.elements_per_sample == 2 && xsm_bytes % 16 == 0 &&
                              p.w_stride_n % 16 == 0 && aligned16(p.x) && aligned16(p.w) &&
                              (p.output_dtype == GLA_DT_FP32 || p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16);
    if (xsm_bytes % 16 != 0 || p.w_stride_n % 16 != 0 || !aligned16(p.x) || !aligned16(p.w)) return false;
    switch (p.output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_MXFP16: case GLA_DT_MXBF16: break;
        default: return false;
    }
    const int csm = p.channel_scale_mode;
    if (csm == GLA_CSM_MX) return p.scales_x != nullptr && ak >= A_FP8;
    if (csm == GLA_CSM_ACTIVATION) return p.scales_x != nullptr && p.sx_dtype == GLA_DT_FP32;
    return csm == GLA_CSM_NONE;
}

bool mx_stream_quantises(const gla_matmul_args& p) { return a_kind(p) >= A_Q4F16 && mx_stream_eligible(p); }

int launch_mx_stream(const gla_matmul_args& p, hipStream_t stream) {
    if (!mx_stream_eligible(p)) {
        set_error("mx_stream: operands must be K-contiguous with 16-byte aligned rows, group_size 32, "
                  "channel_scale_mode 0, 2 or 4");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    const int ak = a_kind(p);
    MxArgs a;
    a.x = (const uint8_t*)p.x; a.w = (const uint8_t*)p.w; a.scales = (const uint8_t*)p.scales;
    a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.KB = p.K / 32;
    a.xsm_bytes = p.x_stride_m * ((ak <= A_BF16 || ak >= A_Q4F16) ? 2 : 1);
    a.wsn_bytes = p.w_stride_n;
    a.osm = p.out_stride_m; a.osn = p.out_stride_n;
    a.msg = p.meta_stride_g; a.msn = p.meta_stride_n; a.sxm = p.sx_stride_m; a.sxg = p.sx_stride_g;
    a.csm = p.channel_scale_mode;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.out_dt = p.output_dtype == GLA_DT_MXFP16 ? GLA_DT_FP16 : (p.output_dtype == GLA_DT_MXBF16 ? GLA_DT_BF16 : p.output_dtype);
    const int rm = p.M >= 5 ? 8 : (p.M >= 3 ? 4 : p.M);
    const int bk = p.elements_per_sample == 2 ? B_FP4 : B_FP8;
    dim3 grid(ceil_div(p.N, 4 * kCols), ceil_div(p.M, rm));
    switch (ak) {
        case A_F16: launch_b<A_F16>(a, bk, rm, grid, stream); break;
        case A_BF16: launch_b<A_BF16>(a, bk, rm, grid, stream); break;
        case A_FP8: launch_b<A_FP8>(a, bk, rm, grid, stream); break;
        case A_Q4F16: launch_rows<A_Q4F16, B_FP4>(a, rm, grid, stream); break;
        case A_Q4BF16: launch_rows<A_Q4BF16, B_FP4>(a, rm, grid, stream); break;
        default: launch_b<A_FP4>(a, bk, rm, grid, stream); break;
    }
    return check_hip(hipGetLastError(), "mx_stream launch");
}

}  // namespace gla
