// Packed 1-, 2-, 4- and 8-bit codes written out as the fp16 / bf16 weights they stand for, [N, K] with K contiguous: the
// first half of the prefill path of packed layers from 2048 rows of bf16 (4096 of fp16) up, whose second half is the
// 16-bit matrix-core GEMM (gemm_16bit.hip).  The fused kernel (gemm_wn.hip) unpacks every weight once per 128 or 256
// rows of the batch, and its vector work stands beside the MFMAs; here a weight is unpacked once per call, at memory
// speed (4096^2 4-bit codes: 11.6 us), and the GEMM that follows runs at the rate of unquantised layers (4-bit codes in
// groups of 128, bf16, M = N = K = 4096: 161 us fused, 135 us for the pair; 8192 rows: 297 -> 246).
// Reference: gemlite/triton_kernels/gemm_kernels.py:405-452 with utils.py:73-105 - the same five W_group_mode forms,
// evaluated with the same arithmetic as the fused kernels (wn_dequant.hpp), so a layer's weights round the same way
// on either side of the hand-off.
//
// One thread: one column n and 64 consecutive K-values = 64 / e packed words of that column (a wave reads 256
// contiguous bytes per word row) -> 128 contiguous bytes of row n of the output, which the wave transposes through LDS
// so that its stores are whole lines too (16 bytes per lane at a stride of a row each ran at a third of the speed).
// With groups of whole multiples of 64 K-values (the fused GEMM's rule) a thread needs one (scale, zero) pair; groups of
// 16 / 32 (layers only the mid-batch kernel takes, which at thousands of rows would stream and unpack the weights once
// per 64 rows) change inside a thread's chunk, between words.
#include "common.hpp"
#include "dispatch.hpp"
#include "wn_dequant.hpp"

namespace gla {

namespace {

struct Unpack16Args {
    const uint32_t* w;        // [K / e, N] packed words
    const void* scales;       // [K / group, N]
    const void* zeros;        // [K / group, N] or one value
    uint16_t* out;            // [N, ldo]
    int N, chunks;            // chunks = K / 64
    int64_t wsk, msg, ldo;    // elements
    int gs;                   // K-values per group (a multiple of 64, or 16 / 32)
    int wgm, meta_dt, z_dt;
    bool has_s, has_zt, z_scalar;
};

template <int BITS, bool BF16>
__global__ __launch_bounds__(256) void wn_unpack16_kernel(Unpack16Args a) {
    constexpr int E = 32 / BITS, WORDS = 64 / E;
    constexpr int OFF = BITS == 8 ? 0 : 128;
    __shared__ __align__(16) unsigned char tile[4][64 * 128];  // per wave: 64 columns x 128 bytes, 16-byte slots swizzled by row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 64;
    const int chunk = blockIdx.y * 4 + wave;
    const bool live = chunk < a.chunks;          // wave-uniform
    int n = n0 + lane;
    if (n > a.N - 1) n = a.N - 1;                // lanes past N unpack the last column again and store nothing
    const int ch = live ? chunk : a.chunks - 1;
    uint32_t w[WORDS];
    const uint32_t* src = a.w + (int64_t)ch * WORDS * a.wsk + n;
#pragma unroll
    for (int j = 0; j < WORDS; ++j) w[j] = __builtin_nontemporal_load(src + (int64_t)j * a.wsk);
    const float c1 = a.wgm == GLA_WGM_SHIFT ? -1.0f : (a.wgm == GLA_WGM_FMA ? 1.0f : 0.0f);
    const float c2 = a.wgm == GLA_WGM_SHIFT_SCALE ? -1.0f : 0.0f;
    auto meta_of = [&](int g) __attribute__((always_inline)) {
        const float s = a.has_s ? load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + n) : 1.0f;
        const float z = a.has_zt ? load_as_float(a.zeros, a.meta_dt, (int64_t)g * a.msg + n)
                                 : (a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0) : 0.0f);
        return make_meta<BF16, OFF>(s, z * __builtin_fmaf(c2, s, c1));
    };
    // groups of 64 K-values or more: one per chunk; groups of 16 / 32: a word lies in one of them
    int g_have = ch * 64 / a.gs;
    ColMeta<BF16> meta = meta_of(g_have);
    uint32_t o[32];
#pragma unroll
    for (int j = 0; j < WORDS; ++j) {
        if (a.gs < 64) {
            const int g = (ch * 64 + j * E) / a.gs;
            if (g != g_have) {
                g_have = g;
                meta = meta_of(g);
            }
        }
#pragma unroll
        for (int i = 0; i < E / 2; ++i) {
            const uint32_t lo = (w[j] >> (BITS * 2 * i)) & ((1u << BITS) - 1u);
            const uint32_t hi = (w[j] >> (BITS * (2 * i + 1))) & ((1u << BITS) - 1u);
            uint32_t r;
            if constexpr (BF16 && BITS == 8) {
                // 128 + q is not exact in bf16 above 127: bytes straight to fp32, scaled there, packed once
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                const f32x2 v = {__builtin_fmaf((float)lo, meta.s, meta.z), __builtin_fmaf((float)hi, meta.s, meta.z)};
                r = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
            } else {
                const uint32_t magic = BF16 ? 0x43004300u : 0x64006400u;  // 128 + q in bf16, 1024 + q in fp16
                r = dequant_pair<BF16>(magic | lo | (hi << 16), meta);
            }
            o[j * (E / 2) + i] = r;
        }
    }
    // through LDS, so that a store instruction writes whole 128-byte lines: the lane's 128 bytes go to row `lane`,
    // then lane (row l / 8 of eight, slot l % 8) stores 16 bytes and eight lanes together one row's line
    unsigned char* mine = tile[wave];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        *(uint4*)(mine + lane * 128 + ((i ^ (lane & 7)) * 16)) = make_uint4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = 8 * i + (lane >> 3), c = lane & 7;
        const uint4 v = *(const uint4*)(mine + r * 128 + ((c ^ (r & 7)) * 16));
        if (live && n0 + r < a.N) *(uint4*)(a.out + (int64_t)(n0 + r) * a.ldo + (int64_t)chunk * 64 + c * 8) = v;
    }
}

template <int BITS>
void launch_bits(const Unpack16Args& a, bool bf16, hipStream_t stream) {
    const dim3 grid(ceil_div(a.N, 64), ceil_div(a.chunks, 4));
    if (bf16)
        hipLaunchKernelGGL((wn_unpack16_kernel<BITS, true>), grid, dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL((wn_unpack16_kernel<BITS, false>), grid, dim3(256), 0, stream, a);
}

// Unpacked int8 / uint8 / e4m3 weight bytes, [N, K] K-contiguous, as the same numbers in fp16 / bf16 (exact: every such
// byte value is a 16-bit float of either kind): 16 bytes in, 32 bytes out per thread, both coalesced.
template <int WDT, bool BF16>
__global__ __launch_bounds__(256) void kbytes_unpack16_kernel(const uint8_t* __restrict__ w, int64_t wsn, int N, int K,
                                                              uint16_t* __restrict__ out, int64_t ldo) {
    const int pieces = K / 16;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)N * pieces) return;
    const int n = (int)(id / pieces), k = (int)(id % pieces) * 16;
    const u32x4 v = __builtin_nontemporal_load((const u32x4*)(w + (int64_t)n * wsn + k));
    const uint32_t in[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float f[4];
        if constexpr (WDT == GLA_DT_FP8) {
            f[0] = __builtin_amdgcn_cvt_f32_fp8((int)in[i], 0);
            f[1] = __builtin_amdgcn_cvt_f32_fp8((int)in[i], 1);
            f[2] = __builtin_amdgcn_cvt_f32_fp8((int)in[i], 2);
            f[3] = __builtin_amdgcn_cvt_f32_fp8((int)in[i], 3);
        } else {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint32_t byte = (in[i] >> (8 * b)) & 0xffu;
                f[b] = WDT == GLA_DT_INT8 ? (float)(int)(int8_t)byte : (float)byte;
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if constexpr (BF16) {
                // exact: at most 8 significant bits
                o[2 * i + h] = (__builtin_bit_cast(uint32_t, f[2 * h]) >> 16) | (__builtin_bit_cast(uint32_t, f[2 * h + 1]) & 0xffff0000u);
            } else {
                o[2 * i + h] = (uint32_t)float_to_half_bits(f[2 * h]) | ((uint32_t)float_to_half_bits(f[2 * h + 1]) << 16);
            }
        }
    }
    uint4* dst = (uint4*)(out + (int64_t)n * ldo + k);
    dst[0] = make_uint4(o[0], o[1], o[2], o[3]);
    dst[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

}  // namespace

// The call must be one the byte-weight GEMM takes (gemm_kbytes_eligible); out: [N, ldo] values of the activation type.
int launch_kbytes_unpack16(const gla_matmul_args& p, void* out, int64_t ldo, hipStream_t stream) {
    if (!gemm_kbytes_eligible(p) || p.K % 16 != 0 || ldo < p.K || ldo % 8 != 0 || ((uintptr_t)out & 15)) {
        set_error("kbytes_unpack16: a call of the byte-weight GEMM and an aligned [N, ldo >= K] output are required");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    const int64_t items = (int64_t)p.N * (p.K / 16);
    const dim3 grid((unsigned)((items + 255) / 256));
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    const uint8_t* w = (const uint8_t*)p.w;
    uint16_t* o = (uint16_t*)out;
#define GLA_LAUNCH_KB16(WDT)                                                                                                 \
    if (bf16)                                                                                                                \
        hipLaunchKernelGGL((kbytes_unpack16_kernel<WDT, true>), grid, dim3(256), 0, stream, w, p.w_stride_n, p.N, p.K, o, ldo); \
    else                                                                                                                     \
        hipLaunchKernelGGL((kbytes_unpack16_kernel<WDT, false>), grid, dim3(256), 0, stream, w, p.w_stride_n, p.N, p.K, o, ldo)
    switch (p.w_dtype) {
        case GLA_DT_FP8: GLA_LAUNCH_KB16(GLA_DT_FP8); break;
        case GLA_DT_INT8: GLA_LAUNCH_KB16(GLA_DT_INT8); break;
        default: GLA_LAUNCH_KB16(GLA_DT_UINT8); break;
    }
#undef GLA_LAUNCH_KB16
    return check_hip(hipGetLastError(), "kbytes_unpack16 launch");
}

// The call must be one the fused packed-weight GEMM or the mid-batch kernel takes (operand types, layouts, alignments;
// groups of whole 64-K chunks, or of 16 / 32 with a packed word inside one group; 1-bit codes in groups of 32 or more);
// out: [N, ldo] 16-bit values of the activation type, ldo >= K, 16-byte aligned rows.
int launch_wn_unpack16(const gla_matmul_args& p, void* out, int64_t ldo, hipStream_t stream) {
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    const int gs = grouped ? p.group_size : p.K;
    const int e = p.elements_per_sample;
    const bool groups_ok = gs > 0 && e > 0 && (gs % 64 == 0 || (64 % gs == 0 && gs % e == 0));
    if (!(gemm_wn_eligible(p) || wn_mid_eligible(p)) || p.K % 64 != 0 || !groups_ok || ldo < p.K || ldo % 8 != 0 ||
        ((uintptr_t)out & 15)) {
        set_error("wn_unpack16: a call of the packed-weight GEMM or the mid-batch kernel and an aligned [N, ldo >= K] output are required");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    Unpack16Args a;
    a.w = (const uint32_t*)p.w; a.scales = p.scales; a.zeros = p.zeros; a.out = (uint16_t*)out;
    a.N = p.N; a.chunks = p.K / 64;
    a.wsk = p.w_stride_k; a.msg = gs == p.K ? 0 : p.meta_stride_g; a.ldo = ldo;
    a.gs = gs;
    a.wgm = p.W_group_mode; a.meta_dt = p.meta_dtype; a.z_dt = p.zeros_dtype;
    a.has_s = uses_scales; a.has_zt = uses_zeros && !p.zero_is_scalar; a.z_scalar = uses_zeros && p.zero_is_scalar;
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.W_nbits) {
        case 1: launch_bits<1>(a, bf16, stream); break;
        case 2: launch_bits<2>(a, bf16, stream); break;
        case 4: launch_bits<4>(a, bf16, stream); break;
        default: launch_bits<8>(a, bf16, stream); break;
    }
    return check_hip(hipGetLastError(), "wn_unpack16 launch");
}

}  // namespace gla
