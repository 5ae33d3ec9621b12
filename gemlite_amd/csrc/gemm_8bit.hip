// MFMA GEMM for K-contiguous narrow operands: out[M,N] = x[M,K] * w[N,K]^T with
//   fp8-e4m3 x fp8-e4m3 -> fp32      (v_mfma_f32_32x32x64_f8f6f4, unit block scales)
//   int8 x int8 -> int32             (v_mfma_i32_32x32x32_i8, exact)
//   MXFP4 x MXFP4 -> fp32            (v_mfma_scale_f32_32x32x64_f8f6f4 with one e8m0 scale per
//                                     32 K-values on either operand)
// and a per-row / per-column scale epilogue.  The prefill path of dynamically quantised A8W8
// and A4W4 layers.
//
// Takes the place of the reference's GEMM kernels for unpacked 8-bit weights and for the
// micro-scaled formats (reference: gemlite/triton_kernels/gemm_kernels.py:285-496 and :509-737,
// epilogue :471-488, tl.dot_scaled :696).
//
//  * Workgroup tile BM x 256, K step of 128 bytes per row (128 fp8/int8 values or 256 fp4
//    values); 8 waves in a 2 x 4 grid, wave tile (BM/2) x 64 of 32x32 MFMA tiles; the
//    accumulators stay in registers for the whole K loop.
//  * Operand tiles are copied global -> LDS by the load unit itself (global_load_lds, 16 bytes
//    per lane), double-buffered: the copy of step k+1 runs while step k is multiplied, and no
//    vector register is spent on staging.  The LDS image is dense; 16-byte chunk c of row r is
//    placed at chunk position c ^ ((r >> 1) & 7), chosen on the global side of the copy, so that
//    the 16 lanes of one LDS read phase hit 16 distinct bank groups.
//  * Workgroups are renumbered so that each of the 8 XCDs (one L2 each) works on its own band
//    of output tiles, and tiles inside a band are visited in groups that share operand panels.
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

enum Mode { kFP8 = 0, kINT8 = 1, kMXFP4 = 2 };

constexpr int kRowB8 = 128;  // bytes per LDS row = bytes of K per pipeline step
constexpr int kBN = 256;
constexpr int kWavesM = 2, kWavesN = 4;
constexpr int kThreads8 = kWavesM * kWavesN * 64;

struct Gemm8Args {
    const uint8_t* a;      // [M, Kb] bytes
    const uint8_t* b;      // [N, Kb] bytes
    const void* scales;    // weight scales: [N] (channel) or [N, K/32] e8m0 (MXFP4)
    const void* scales_x;  // activation scales: [M] or [M_pad, K/32] e8m0
    void* out;
    int M, N, Kb;          // Kb = bytes of K per row
    int64_t lda, ldb, osm, sxm, msn;
    int csm, meta_dt, sx_dt, out_dt;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    int t = pid;
    if (total % 8 == 0) t = (pid % 8) * (total / 8) + pid / 8;  // one contiguous band of tiles per XCD
    constexpr int GROUP = 4;  // tile rows visited together
    const int width = GROUP * tiles_n;
    const int group = t / width;
    const int first_m = group * GROUP;
    const int gsize = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    tm = first_m + (t % width) % gsize;
    tn = (t % width) / gsize;
}

template <int MODE, int BM>
__global__ __launch_bounds__(kThreads8) void gemm_8bit_kernel(Gemm8Args p) {
    constexpr int WM = BM / kWavesM;  // wave tile rows
    constexpr int TI = WM / 32;       // 32-row MFMA tiles per wave along M
    constexpr int TJ = 2;             // 64 columns per wave
    constexpr int STAGE = (BM + kBN) * kRowB8;
    constexpr int A_INSTR = BM / 8;        // copy instructions (8 rows each) for the A tile
    constexpr int INSTR = (BM + kBN) / 8;  // ... for both tiles
    constexpr int PER_WAVE = INSTR / 8;
    constexpr bool MX = MODE == kMXFP4;

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBN;

    // ---- global -> LDS copy plan: instruction q = wave + 8 i moves 8 rows of one tile; lane
    // (row l/8, position l%8) fetches the chunk that belongs at that position of the swizzled row
    const int crow = lane >> 3, cpos = lane & 7;
    const uint8_t* g_src[PER_WAVE];
    int l_off[PER_WAVE], chunk16[PER_WAVE];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int q = wave + 8 * i;  // wave-uniform
        const bool is_a = q < A_INSTR;
        const int row8 = (is_a ? q : q - A_INSTR) * 8;
        const int row = row8 + crow;
        const int chunk = cpos ^ ((row >> 1) & 7);
        chunk16[i] = chunk * 16;
        if (is_a) {
            int gm = m0 + row;
            if (gm > p.M - 1) gm = p.M - 1;
            g_src[i] = p.a + (int64_t)gm * p.lda + chunk * 16;
            l_off[i] = row8 * kRowB8;
        } else {
            int gn = n0 + row;
            if (gn > p.N - 1) gn = p.N - 1;
            g_src[i] = p.b + (int64_t)gn * p.ldb + chunk * 16;
            l_off[i] = (BM + row8) * kRowB8;
        }
    }
    // a row's last step may hold fewer than 128 bytes: chunks past the end re-read chunk 0 of the
    // step (always inside the row) and are never multiplied
    auto copy_step = [&](int k0, int stage) {
        const int limit = p.Kb - k0;
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) {
            const uint8_t* src = g_src[i] + k0 - (chunk16[i] < limit ? 0 : chunk16[i]);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(smem + stage * STAGE + l_off[i]),
                                             16, 0, 0);
        }
    };

    // ---- accumulators
    typedef typename std::conditional<MODE == kINT8, int16_t_v, float16_t>::type acc_t;
    acc_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int r32 = lane & 31, kb = lane >> 5;
    const int sw = (r32 >> 1) & 7;  // chunk swizzle of this lane's rows (tile offsets are multiples of 32)
    const int a_row0 = (wm * WM + r32) * kRowB8;
    const int b_row0 = (BM + wn * 64 + r32) * kRowB8;

    // ---- MXFP4 block scales: 8 bytes (8 blocks of 32) per row per step, fetched one step ahead
    u32x2 sa_next[MX ? TI : 1], sb_next[MX ? TJ : 1];
    const uint8_t* sa_ptr[MX ? TI : 1];
    const uint8_t* sb_ptr[MX ? TJ : 1];
    if constexpr (MX) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            int gm = m0 + wm * WM + i * 32 + r32;
            if (gm > p.M - 1) gm = p.M - 1;
            sa_ptr[i] = (const uint8_t*)p.scales_x + (int64_t)gm * p.sxm;
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            int gn = n0 + wn * 64 + j * 32 + r32;
            if (gn > p.N - 1) gn = p.N - 1;
            sb_ptr[j] = (const uint8_t*)p.scales + (int64_t)gn * p.msn;
        }
    }
    auto load_scales = [&](int step) {
        if constexpr (MX) {
            const bool upper = p.Kb - step * kRowB8 > 64;  // blocks 4..7 of the step exist
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                sa_next[i].x = *(const unsigned int*)(sa_ptr[i] + step * 8);
                sa_next[i].y = upper ? *(const unsigned int*)(sa_ptr[i] + step * 8 + 4) : 0u;
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                sb_next[j].x = *(const unsigned int*)(sb_ptr[j] + step * 8);
                sb_next[j].y = upper ? *(const unsigned int*)(sb_ptr[j] + step * 8 + 4) : 0u;
            }
        }
    };

    // ---- pipeline
    const int steps = (p.Kb + kRowB8 - 1) / kRowB8;
    copy_step(0, 0);
    load_scales(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
        const int cur = k & 1;
        u32x2 sa_cur[MX ? TI : 1], sb_cur[MX ? TJ : 1];
        if constexpr (MX) {
            // half-wave kb multiplies blocks kb, 2+kb, 4+kb, 6+kb: shift them into bytes 0 and 2
#pragma unroll
            for (int i = 0; i < TI; ++i) sa_cur[i] = u32x2{sa_next[i].x >> (8 * kb), sa_next[i].y >> (8 * kb)};
#pragma unroll
            for (int j = 0; j < TJ; ++j) sb_cur[j] = u32x2{sb_next[j].x >> (8 * kb), sb_next[j].y >> (8 * kb)};
        }
        if (k + 1 < steps) {
            copy_step((k + 1) * kRowB8, cur ^ 1);  // that buffer was last read in step k-1
            load_scales(k + 1);
        }
        const unsigned char* base = smem + cur * STAGE;
        const int limit = p.Kb - k * kRowB8;  // valid bytes of this step (>= 128 except in a ragged tail)
        if constexpr (MODE == kFP8) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {  // two MFMA K-steps of 64 bytes: chunks 4h + 2kb and the next
                if (h * 64 >= limit) break;
                const int c0 = ((4 * h + 2 * kb) ^ sw) << 4, c1 = ((4 * h + 2 * kb + 1) ^ sw) << 4;
                int8_t_v bf[TJ];
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const u32x4 lo = *(const u32x4*)(base + b_row0 + j * 32 * kRowB8 + c0);
                    const u32x4 hi = *(const u32x4*)(base + b_row0 + j * 32 * kRowB8 + c1);
                    bf[j] = int8_t_v{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
                }
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const u32x4 lo = *(const u32x4*)(base + a_row0 + i * 32 * kRowB8 + c0);
                    const u32x4 hi = *(const u32x4*)(base + a_row0 + i * 32 * kRowB8 + c1);
                    const int8_t_v af = int8_t_v{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
#pragma unroll
                    for (int j = 0; j < TJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, bf[j], acc[i][j], 0, 0, 0, 127, 0, 127);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {  // four MFMA K-steps of 32 bytes: chunk 2s + kb
                if (s * 32 >= limit) break;
                const int c0 = ((2 * s + kb) ^ sw) << 4;
                u32x4 bf[TJ];
#pragma unroll
                for (int j = 0; j < TJ; ++j) bf[j] = *(const u32x4*)(base + b_row0 + j * 32 * kRowB8 + c0);
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const u32x4 af = *(const u32x4*)(base + a_row0 + i * 32 * kRowB8 + c0);
#pragma unroll
                    for (int j = 0; j < TJ; ++j) {
                        if constexpr (MODE == kINT8) {
                            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                int4_t{(int)af.x, (int)af.y, (int)af.z, (int)af.w},
                                int4_t{(int)bf[j].x, (int)bf[j].y, (int)bf[j].z, (int)bf[j].w}, acc[i][j], 0, 0, 0);
                        } else {
                            const int8_t_v a8 = int8_t_v{(int)af.x, (int)af.y, (int)af.z, (int)af.w, 0, 0, 0, 0};
                            const int8_t_v b8 = int8_t_v{(int)bf[j].x, (int)bf[j].y, (int)bf[j].z, (int)bf[j].w, 0, 0, 0, 0};
                            const int sa = (int)((s < 2) ? sa_cur[i].x : sa_cur[i].y);
                            const int sb = (int)((s < 2) ? sb_cur[j].x : sb_cur[j].y);
                            if (s & 1)
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i][j], 4, 4, 2, sa, 2, sb);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[i][j], 4, 4, 0, sa, 0, sb);
                        }
                    }
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's part of step k+1 has landed
        __syncthreads();
    }

    // ---- epilogue: lane holds column r32 of each 32-wide tile, rows 8*(e/4) + 4*kb + e%4
    float sb[TJ];
    bool n_ok[TJ];
    const bool col_scale = !MX && (p.csm & 1);
    const bool row_scale = !MX && (p.csm & 2);
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int n = n0 + wn * 64 + j * 32 + r32;
        n_ok[j] = n < p.N;
        sb[j] = (col_scale && n_ok[j]) ? load_as_float(p.scales, p.meta_dt, n) : 1.0f;
    }
    auto emit = [&](auto dt_tag) {
        constexpr int DT = decltype(dt_tag)::value;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * WM + i * 32 + 8 * (e / 4) + 4 * kb + (e % 4);
                if (m < p.M) {
                    const float sa = row_scale ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
                    const int64_t o = (int64_t)m * p.osm + n0 + wn * 64 + r32;
#pragma unroll
                    for (int j = 0; j < TJ; ++j) {
                        if (!n_ok[j]) continue;
                        if constexpr (DT == GLA_DT_INT32) ((int32_t*)p.out)[o + j * 32] = (int32_t)acc[i][j][e];
                        else store_typed<DT>(p.out, o + j * 32, (float)acc[i][j][e] * (sa * sb[j]));
                    }
                }
            }
        }
    };
    if (p.out_dt == GLA_DT_FP16) emit(std::integral_constant<int, GLA_DT_FP16>{});
    else if (p.out_dt == GLA_DT_BF16) emit(std::integral_constant<int, GLA_DT_BF16>{});
    else if (p.out_dt == GLA_DT_INT32) emit(std::integral_constant<int, GLA_DT_INT32>{});
    else emit(std::integral_constant<int, GLA_DT_FP32>{});
}

template <int MODE, int BM>
int launch_bm(const Gemm8Args& a, hipStream_t stream) {
    const size_t smem = 2 * (size_t)(BM + kBN) * kRowB8;
    static bool configured = false;  // per instantiation; the attribute is sticky per function
    auto kern = gemm_8bit_kernel<MODE, BM>;
    if (!configured) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_8bit: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n), dim3(kThreads8), smem, stream, a);
    return check_hip(hipGetLastError(), "gemm_8bit launch");
}

template <int MODE>
int launch_mode(const Gemm8Args& a, int bm, hipStream_t stream) {
    if (bm == 256) return launch_bm<MODE, 256>(a, stream);
    if (bm == 128) return launch_bm<MODE, 128>(a, stream);
    return launch_bm<MODE, 64>(a, stream);
}

int pick_bm(int M, int tile_config) {
    int bm = tile_config > 0 ? tile_config : (M > 128 ? 256 : (M > 64 ? 128 : 64));
    if (bm != 64 && bm != 128 && bm != 256) bm = 256;
    return bm;
}

}  // namespace

bool gemm_8bit_eligible(const gla_matmul_args& p) {
    const bool fp8 = p.input_dtype == GLA_DT_FP8 && p.w_dtype == GLA_DT_FP8 && p.acc_dtype == GLA_DT_FP32;
    const bool i8 = p.input_dtype == GLA_DT_INT8 && p.w_dtype == GLA_DT_INT8;
    if (!fp8 && !i8) return false;
    if (p.elements_per_sample != 1 || p.W_nbits != 8 || p.W_group_mode != GLA_WGM_NONE) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.K % (fp8 ? 64 : 32) != 0 || p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    if (i8 && p.acc_dtype != GLA_DT_INT32) return false;
    if (p.output_dtype == GLA_DT_INT32 && !(i8 && p.channel_scale_mode == GLA_CSM_NONE)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int launch_gemm_8bit(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = 0; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype;
    const int bm = pick_bm(p.M, p.tile_config);
    a.tiles_n = ceil_div(p.N, kBN);
    a.tiles_m = ceil_div(p.M, bm);
    if (p.input_dtype == GLA_DT_INT8) return launch_mode<kINT8>(a, bm, stream);
    return launch_mode<kFP8>(a, bm, stream);
}

// MXFP4 x MXFP4: x is [M, K/2] bytes, w the [K/2, N] view of [N, K/2] bytes, and both e8m0
// scale arrays are [rows, K/32] with unit stride along K.
bool gemm_mxfp4_eligible(const gla_matmul_args& p) {
    if (p.input_dtype != GLA_DT_MXFP4 || p.channel_scale_mode != GLA_CSM_MX) return false;
    if (p.W_nbits != 4 || p.elements_per_sample != 2 || p.group_size != 32) return false;
    if (p.scales == nullptr || p.scales_x == nullptr) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.meta_stride_g != 1 || p.sx_stride_g != 1) return false;
    if (p.K % 128 != 0 || p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0) return false;
    if (p.meta_stride_n % 4 != 0 || p.sx_stride_m % 4 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15) || ((uintptr_t)p.scales & 3) || ((uintptr_t)p.scales_x & 3))
        return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    return true;
}

int launch_gemm_mxfp4(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K / 2; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = p.meta_stride_n; a.csm = 0; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype;
    const int bm = pick_bm(p.M, p.tile_config);
    a.tiles_n = ceil_div(p.N, kBN);
    a.tiles_m = ceil_div(p.M, bm);
    return launch_mode<kMXFP4>(a, bm, stream);
}

}  // namespace gla
