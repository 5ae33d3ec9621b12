// MFMA GEMM for fp16/bf16 activations x 32-bit packed low-bit weights stored [K/e, N], N fastest:
// out[M,N] = x[M,K] * dequant(W)[K,N], dequantisation fused into the B-operand path.  The prefill
// path of A16W4 / A16W8 / A16W2 layers.
//
// Takes the place of the reference's GPTQ-style GEMM and, for mid-size batches, of its split-K
// GEMM (reference: gemlite/triton_kernels/gemm_kernels.py:285-496,
// gemlite/triton_kernels/gemm_splitK_kernels.py:300-523; dequant
// gemlite/triton_kernels/utils.py:73-105).
//
//  * Workgroup tile BM x 256, K step 64; waves in a (BM/64) x 2 grid, wave tile 64 x 128 of
//    v_mfma_f32_32x32x16 tiles, 128 accumulator registers per lane.
//  * Weights never pass through LDS.  A lane's 128-bit load holds the words of 4 adjacent
//    columns; word component j is the B operand of column tile j, so the wave's 128 columns are
//    the interleaved set {4r + j}.  A word is unpacked with the pair trick of the GEMV kernel
//    (codes OR-ed into the mantissa of 1024.0 / 128.0, two per VALU op), then (q - OFF) * s + z'
//    is applied with packed fp16 math (fp32 for bf16 activations) once per wave and reused for
//    both 32-row tiles.
//  * Activations go global -> registers -> LDS (double-buffered, rows padded to 144 bytes); each
//    16-byte chunk is reordered on the way in to the K-slot order the unpacking produces, so A
//    fragments are plain 128-bit LDS reads.
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBKw = 64;         // K per pipeline stage
constexpr int kRowB = 144;       // padded LDS row (128 bytes of fp16 + 16)
constexpr int kWavesNw = 2;
constexpr int kBNw = kWavesNw * 128;

struct GemmWnArgs {
    const uint16_t* x;
    const uint32_t* w;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    int M, N, K;
    int gs;       // K-values per quantisation group (K when ungrouped)
    int64_t xsm, wsk, osm, msg, sxm;
    int wgm, csm, meta_dt, z_dt, z_scalar, out_dt, sx_dt;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ void tile_coords_wn(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    int t = pid;
    if (total % 8 == 0) t = (pid % 8) * (total / 8) + pid / 8;  // one contiguous band of tiles per XCD
    constexpr int GROUP = 4;
    const int width = GROUP * tiles_n;
    const int group = t / width;
    const int first_m = group * GROUP;
    const int gsize = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    tm = first_m + (t % width) % gsize;
    tn = (t % width) / gsize;
}

// Reorder one 16-byte chunk of activations (8 consecutive K-values) to the K-slot order of the
// B operand: W4 pairs (j, j+4); W8 pairs (j, j+2) inside each half; W2 handled by the caller.
template <int BITS>
__device__ __forceinline__ u32x4 permute_chunk(u32x4 v) {
    u32x4 o;
    if constexpr (BITS == 4) {
        o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
        o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
        o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
        o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    } else {  // BITS == 8
        o.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
        o.y = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
        o.z = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
        o.w = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
    }
    return o;
}

// Per-column dequant constants of one quantisation group, prepared once per group.
template <bool BF16>
struct ColMeta;
template <>
struct ColMeta<false> {
    half2_t s, z;  // (s, s) and (z', z') in fp16
};
template <>
struct ColMeta<true> {
    float s, z;
};

template <bool BF16>
__device__ __forceinline__ ColMeta<BF16> make_meta(float s, float zp) {
    ColMeta<BF16> m;
    if constexpr (BF16) {
        m.s = s;
        m.z = zp;
    } else {
        m.s = half2_t{(half_t)s, (half_t)s};
        m.z = half2_t{(half_t)zp, (half_t)zp};
    }
    return m;
}

// pair register holding (OFF + q_lo, OFF + q_hi) -> dequantised pair in the activation type
template <bool BF16>
__device__ __forceinline__ uint32_t dequant_pair(uint32_t t, const ColMeta<BF16>& m) {
    if constexpr (BF16) {
        // bf16 bits are the top half of an fp32: 128 + q is exact there too
        const float lo = __builtin_bit_cast(float, t << 16) - 128.0f;
        const float hi = __builtin_bit_cast(float, t & 0xffff0000u) - 128.0f;
        const float wl = __builtin_fmaf(lo, m.s, m.z), wh = __builtin_fmaf(hi, m.s, m.z);
        return (uint32_t)float_to_bf16_bits(wl) | ((uint32_t)float_to_bf16_bits(wh) << 16);
    } else {
        half2_t q = __builtin_bit_cast(half2_t, t) - half2_t{(half_t)1024.0f, (half_t)1024.0f};
        half2_t w = __builtin_elementwise_fma(q, m.s, m.z);
        return __builtin_bit_cast(uint32_t, w);
    }
}

template <bool BF16>
__device__ __forceinline__ float16_t mfma32(const u32x4& a, const u32x4& b, float16_t c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}

// BITS in {2, 4, 8}; WAVES_M in {1, 2, 4}
template <int BITS, bool BF16, int WAVES_M>
__global__ __launch_bounds__(WAVES_M * kWavesNw * 64) void gemm_wn_kernel(GemmWnArgs p) {
    constexpr int E = 32 / BITS;
    constexpr int BM = WAVES_M * 64;
    constexpr int NT = WAVES_M * kWavesNw * 64;
    constexpr int TI = 2, TJ = 4;
    constexpr int WL = (BITS == 8) ? 8 : 4;             // 128-bit weight loads per lane per stage
    constexpr int A_CHUNKS = (BM * 8 + NT - 1) / NT;    // 16-byte chunks of A per thread per stage
    constexpr int STAGE = BM * kRowB;
    constexpr uint32_t kPairMask = ((1u << BITS) - 1u) * 0x00010001u;
    constexpr uint32_t kMagic = BF16 ? 0x43004300u : 0x64006400u;

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / kWavesNw, wn = wave % kWavesNw;
    const int r32 = lane & 31, kb = lane >> 5;
    int tm, tn;
    tile_coords_wn(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBNw;

    // ---- A staging slots
    int a_off[A_CHUNKS], a_off2[BITS == 2 ? A_CHUNKS : 1], a_dst[A_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int id = tid + i * NT, row = id >> 3, c = id & 7;
        int gm = m0 + row;
        if (gm > p.M - 1) gm = p.M - 1;
        a_off[i] = gm * (int)p.xsm + c * 8;  // element offset
        // 2-bit words hold 16 K-values: K-slots (j, j+8) need chunk c and its partner c^1 of the block
        if constexpr (BITS == 2) a_off2[i] = gm * (int)p.xsm + (c ^ 1) * 8;
        a_dst[i] = row * kRowB + c * 16;
    }
    u32x4 a_reg[A_CHUNKS];
    u32x4 a_reg2[BITS == 2 ? A_CHUNKS : 1];  // partner chunk for the 2-bit slot order

    // ---- B stream: lane owns columns n0 + wn*128 + 4*r32 + {0..3}
    int coln = n0 + wn * 128 + r32 * 4;
    const bool col_ok = coln + 3 < p.N;  // N % 4 == 0 is required, so a lane is all-in or all-out
    if (coln > p.N - 4) coln = p.N - 4;
    const uint32_t* wcol = p.w + coln;
    u32x4 w_reg[WL];

    auto issue_loads = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            a_reg[i] = *(const u32x4*)(p.x + (size_t)(unsigned)(a_off[i] + k0));
            if constexpr (BITS == 2) a_reg2[i] = *(const u32x4*)(p.x + (size_t)(unsigned)(a_off2[i] + k0));
        }
        const int wr0 = k0 / E;
#pragma unroll
        for (int u = 0; u < WL; ++u) {
            int row;
            if constexpr (BITS == 8) row = wr0 + 4 * (u / 2) + 2 * kb + (u % 2);   // step u/2: rows 4s + 2kb + {0,1}
            else if constexpr (BITS == 4) row = wr0 + 2 * u + kb;                  // step u: row 2s + kb
            else row = wr0 + u;                                                    // step u: row s (both K-halves read it)
            w_reg[u] = *(const u32x4*)(wcol + (int64_t)row * p.wsk);
        }
    };
    auto store_a = [&](int stage) {
        unsigned char* base = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int id = tid + i * NT;
            if (A_CHUNKS * NT > BM * 8 && id >= BM * 8) continue;
            u32x4 o;
            if constexpr (BITS == 2) {
                // chunk c of a 16-K block pairs with its partner: even chunk = K 0..7, odd = K 8..15.
                // destination chunk (kb = c & 1) holds slots (j, j+8), j = 4*kb .. 4*kb+3
                const bool odd = (id & 1) != 0;
                const u32x4 lo = odd ? a_reg2[i] : a_reg[i];   // K 0..7 of the block
                const u32x4 hi = odd ? a_reg[i] : a_reg2[i];   // K 8..15
                const uint32_t l0 = odd ? lo.z : lo.x, l1 = odd ? lo.w : lo.y;
                const uint32_t h0 = odd ? hi.z : hi.x, h1 = odd ? hi.w : hi.y;
                o.x = __builtin_amdgcn_perm(h0, l0, 0x05040100u);
                o.y = __builtin_amdgcn_perm(h0, l0, 0x07060302u);
                o.z = __builtin_amdgcn_perm(h1, l1, 0x05040100u);
                o.w = __builtin_amdgcn_perm(h1, l1, 0x07060302u);
            } else {
                o = permute_chunk<BITS>(a_reg[i]);
            }
            *(u32x4*)(base + a_dst[i]) = o;
        }
    };

    // ---- per-group dequant constants for the lane's 4 columns
    ColMeta<BF16> meta[TJ];
    const bool grouped = p.wgm >= GLA_WGM_SCALE || (p.wgm == GLA_WGM_SHIFT && !p.z_scalar);
    auto load_meta = [&](int g) {
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            float s = 1.0f, z = 0.0f;
            const int64_t idx = (int64_t)g * p.msg + coln + j;
            if (p.wgm >= GLA_WGM_SCALE) s = load_as_float(p.scales, p.meta_dt, idx);
            if (p.wgm == GLA_WGM_SHIFT || p.wgm >= GLA_WGM_SHIFT_SCALE)
                z = p.z_scalar ? load_as_float(p.zeros, p.z_dt, 0) : load_as_float(p.zeros, p.z_dt, idx);
            float zp;
            switch (p.wgm) {
                case GLA_WGM_SHIFT: zp = -z; break;
                case GLA_WGM_SHIFT_SCALE: zp = -z * s; break;
                case GLA_WGM_FMA: zp = z; break;
                default: zp = 0.0f; break;
            }
            meta[j] = make_meta<BF16>(s, zp);
        }
    };

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    uint32_t pair_mask = kPairMask, magic = kMagic;
    asm volatile("" : "+s"(pair_mask), "+v"(magic));  // registers, so that v_and_or_b32 is selected

    const int a_row0 = (wm * 64 + r32) * kRowB;
    const int steps = p.K / kBKw;
    const int stages_per_group = p.gs / kBKw;  // >= 1, checked on the host

    issue_loads(0);
    load_meta(0);
    store_a(0);
    __syncthreads();

#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
        const int cur = k & 1;
        u32x4 wc[WL];
#pragma unroll
        for (int u = 0; u < WL; ++u) wc[u] = w_reg[u];
        if (k + 1 < steps) issue_loads((k + 1) * kBKw);
        const unsigned char* base = smem + cur * STAGE;
#pragma unroll
        for (int s = 0; s < 4; ++s) {  // four MFMA K-steps of 16
            u32x4 af[TI];
#pragma unroll
            for (int i = 0; i < TI; ++i) af[i] = *(const u32x4*)(base + a_row0 + i * 32 * kRowB + s * 32 + kb * 16);
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                u32x4 bq;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    uint32_t t;
                    if constexpr (BITS == 4) {
                        const uint32_t w = wc[s][j];
                        t = ((w >> (r * 4)) & pair_mask) | magic;
                    } else if constexpr (BITS == 8) {
                        const uint32_t w = wc[2 * s + r / 2][j];
                        t = ((w >> ((r % 2) * 8)) & pair_mask) | magic;
                    } else {
                        const uint32_t w = wc[s][j];
                        t = ((w >> ((4 * kb + r) * 2)) & pair_mask) | magic;
                    }
                    bq[r] = dequant_pair<BF16>(t, meta[j]);
                }
#pragma unroll
                for (int i = 0; i < TI; ++i) acc[i][j] = mfma32<BF16>(af[i], bq, acc[i][j]);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the unpacking of later K-steps from being hoisted (register pressure)
        }
        if (k + 1 < steps) {
            store_a(cur ^ 1);
            if (grouped && ((k + 1) % stages_per_group) == 0) load_meta((k + 1) / stages_per_group);
        }
        __syncthreads();
    }

    // ---- epilogue: lane holds column 4*r32 + j of tile j, rows 8*(e/4) + 4*kb + e%4 of tile i
    if (!col_ok) return;
    float sb[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j)
        sb[j] = (p.csm & 1) ? load_as_float(p.scales, p.meta_dt, coln + j) : 1.0f;
    const bool row_scale = (p.csm & 2) != 0;
    auto emit = [&](auto dt_tag) {
        constexpr int DT = decltype(dt_tag)::value;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (e / 4) + 4 * kb + (e % 4);
                if (m < p.M) {
                    const float sa = row_scale ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
                    const int64_t o = (int64_t)m * p.osm + coln;
#pragma unroll
                    for (int j = 0; j < TJ; ++j) store_typed<DT>(p.out, o + j, acc[i][j][e] * (sa * sb[j]));
                }
            }
        }
    };
    if (p.out_dt == GLA_DT_FP16) emit(std::integral_constant<int, GLA_DT_FP16>{});
    else if (p.out_dt == GLA_DT_BF16) emit(std::integral_constant<int, GLA_DT_BF16>{});
    else emit(std::integral_constant<int, GLA_DT_FP32>{});
}

template <int BITS, bool BF16, int WAVES_M>
int launch_wn(const GemmWnArgs& a, hipStream_t stream) {
    constexpr int BM = WAVES_M * 64;
    const size_t smem = 2 * (size_t)BM * kRowB;
    static bool configured = false;
    auto kern = gemm_wn_kernel<BITS, BF16, WAVES_M>;
    if (!configured && smem > 48 * 1024) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_wn: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n), dim3(WAVES_M * kWavesNw * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "gemm_wn launch");
}

template <int BITS, bool BF16>
int launch_wn_m(const GemmWnArgs& a, int waves_m, hipStream_t stream) {
    if (waves_m == 4) return launch_wn<BITS, BF16, 4>(a, stream);
    if (waves_m == 2) return launch_wn<BITS, BF16, 2>(a, stream);
    return launch_wn<BITS, BF16, 1>(a, stream);
}

}  // namespace

bool gemm_wn_eligible(const gla_matmul_args& p) {
    if (p.w_dtype != GLA_DT_INT32) return false;
    if (!(p.W_nbits == 2 || p.W_nbits == 4 || p.W_nbits == 8)) return false;
    if (p.elements_per_sample * p.W_nbits != 32) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16)) return false;
    if (p.W_nbits == 8 && p.input_dtype == GLA_DT_BF16) return false;  // 128 + q is not exact in bf16 for q > 127
    if (p.acc_dtype != GLA_DT_FP32) return false;
    if (p.W_group_mode < 0 || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.channel_scale_mode < 0 || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if (p.N < 4 || p.N % 4 != 0 || p.w_stride_n != 1 || p.w_stride_k % 4 != 0) return false;
    if (p.x_stride_k != 1 || p.x_stride_m % 8 != 0 || p.out_stride_n != 1) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    if (p.K % kBKw != 0) return false;
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31)) return false;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if (uses_scales && (p.scales == nullptr || p.meta_stride_n != 1)) return false;
    if (uses_zeros && p.zeros == nullptr) return false;
    if (uses_zeros && !p.zero_is_scalar && p.meta_stride_n != 1) return false;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    if (grouped && (p.group_size % kBKw != 0 || p.K % p.group_size != 0)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int64_t gemm_wn_workspace_bytes(const gla_matmul_args&) { return 0; }

int launch_gemm_wn(const gla_matmul_args& p, hipStream_t stream) {
    GemmWnArgs a;
    a.x = (const uint16_t*)p.x; a.w = (const uint32_t*)p.w; a.scales = p.scales; a.zeros = p.zeros;
    a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K;
    const bool grouped = p.W_group_mode >= GLA_WGM_SCALE || (p.W_group_mode == GLA_WGM_SHIFT && !p.zero_is_scalar);
    a.gs = grouped ? p.group_size : p.K;
    a.xsm = p.x_stride_m; a.wsk = p.w_stride_k; a.osm = p.out_stride_m; a.msg = p.meta_stride_g; a.sxm = p.sx_stride_m;
    a.wgm = p.W_group_mode; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.z_dt = p.zeros_dtype;
    a.z_scalar = p.zero_is_scalar; a.out_dt = p.output_dtype; a.sx_dt = p.sx_dtype;
    int waves_m = p.tile_config > 0 ? p.tile_config : (p.M > 128 ? 4 : (p.M > 64 ? 2 : 1));
    if (!(waves_m == 1 || waves_m == 2 || waves_m == 4)) waves_m = 4;
    a.tiles_m = ceil_div(p.M, waves_m * 64);
    a.tiles_n = ceil_div(p.N, kBNw);
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.W_nbits) {
        case 2: return bf16 ? launch_wn_m<2, true>(a, waves_m, stream) : launch_wn_m<2, false>(a, waves_m, stream);
        case 4: return bf16 ? launch_wn_m<4, true>(a, waves_m, stream) : launch_wn_m<4, false>(a, waves_m, stream);
        default: return launch_wn_m<8, false>(a, waves_m, stream);
    }
}

}  // namespace gla
