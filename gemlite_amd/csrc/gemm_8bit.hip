// MFMA GEMM for 8-bit operands, both K-contiguous: out[M,N] = x[M,K] * w[N,K]^T with
// fp8-e4m3 x fp8-e4m3 -> fp32 or int8 x int8 -> int32 accumulation and a per-row / per-column
// scale epilogue.  The prefill path of dynamically quantised A8W8 layers.
//
// Takes the place of the reference's GEMM kernel for unpacked 8-bit weights
// (reference: gemlite/triton_kernels/gemm_kernels.py:285-496, epilogue :471-488).
//
//  * Workgroup tile BM x 256 x 128 (K in bytes), 8 waves in a 2 x 4 grid, wave tile
//    (BM/2) x 64 built from 32x32 MFMAs (fp8: v_mfma_f32_32x32x64_f8f6f4, int8:
//    v_mfma_i32_32x32x32_i8).  Accumulators stay in registers for the whole K loop.
//  * Operand tiles go global -> registers -> LDS with 128-bit accesses, double-buffered: the
//    loads of step k+1 are in flight while step k is multiplied.  LDS rows are padded from 128
//    to 144 bytes, which makes the 16 lanes of one LDS access phase hit 16 distinct bank groups.
//  * Workgroups are renumbered so that the 8 XCDs (each with its own L2) work on disjoint
//    bands of output tiles, and tiles inside a band are visited in groups that share operand
//    panels.
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

constexpr int kBK = 128;          // K bytes per pipeline step
constexpr int kRowBytes = 144;    // padded LDS row
constexpr int kBN = 256;
constexpr int kWavesM = 2, kWavesN = 4;
constexpr int kThreads8 = kWavesM * kWavesN * 64;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct Gemm8Args {
    const uint8_t* a;  // [M, K]
    const uint8_t* b;  // [N, K]
    const void* scales;    // weight scales [N] or null
    const void* scales_x;  // activation scales [M] or null
    void* out;
    int M, N, K;
    int64_t lda, ldb, osm, sxm;
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

template <bool INT8, int BM>
__global__ __launch_bounds__(kThreads8) void gemm_8bit_kernel(Gemm8Args p) {
    constexpr int WM = BM / kWavesM;  // wave tile rows
    constexpr int TI = WM / 32;       // 32-row MFMA tiles per wave along M
    constexpr int TJ = 2;             // 64 columns per wave
    constexpr int A_CHUNKS = BM * 8 / kThreads8;   // 16-byte chunks per thread per step
    constexpr int B_CHUNKS = kBN * 8 / kThreads8;
    constexpr int STAGE = (BM + kBN) * kRowBytes;

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBN;

    // ---- global -> register staging: thread owns fixed (row, chunk) slots of both tiles
    int a_off[A_CHUNKS], b_off[B_CHUNKS];  // byte offsets from p.a / p.b (< 2^31, checked on the host)
    int a_dst[A_CHUNKS], b_dst[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int id = tid + i * kThreads8, row = id >> 3, c = id & 7;
        int gm = m0 + row;
        if (gm > p.M - 1) gm = p.M - 1;
        a_off[i] = gm * (int)p.lda + c * 16;
        a_dst[i] = row * kRowBytes + c * 16;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
        const int id = tid + i * kThreads8, row = id >> 3, c = id & 7;
        int gn = n0 + row;
        if (gn > p.N - 1) gn = p.N - 1;
        b_off[i] = gn * (int)p.ldb + c * 16;
        b_dst[i] = BM * kRowBytes + row * kRowBytes + c * 16;
    }
    u32x4 a_reg[A_CHUNKS], b_reg[B_CHUNKS];

#define GLA_LOAD_STEP(k0)                                                                     \
    do {                                                                                      \
        _Pragma("unroll") for (int i = 0; i < A_CHUNKS; ++i)                                  \
            a_reg[i] = *(const u32x4*)(p.a + (size_t)(unsigned)(a_off[i] + (k0)));            \
        _Pragma("unroll") for (int i = 0; i < B_CHUNKS; ++i)                                  \
            b_reg[i] = *(const u32x4*)(p.b + (size_t)(unsigned)(b_off[i] + (k0)));            \
    } while (0)
#define GLA_STORE_STEP(stage)                                                                 \
    do {                                                                                      \
        unsigned char* sbase = smem + (stage) * STAGE;                                        \
        _Pragma("unroll") for (int i = 0; i < A_CHUNKS; ++i) *(u32x4*)(sbase + a_dst[i]) = a_reg[i]; \
        _Pragma("unroll") for (int i = 0; i < B_CHUNKS; ++i) *(u32x4*)(sbase + b_dst[i]) = b_reg[i]; \
    } while (0)

    // ---- accumulators
    typedef typename std::conditional<INT8, int16_t_v, float16_t>::type acc_t;
    acc_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int r32 = lane & 31, kb = lane >> 5;
    const int a_row0 = (wm * WM + r32) * kRowBytes;
    const int b_row0 = BM * kRowBytes + (wn * 64 + r32) * kRowBytes;

    // ---- pipeline: LDS stage (k & 1) holds step k; registers hold step k+1
    const int steps = p.K / kBK;
    GLA_LOAD_STEP(0);
    GLA_STORE_STEP(0);
    __syncthreads();
#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
        const int cur = k & 1;
        if (k + 1 < steps) GLA_LOAD_STEP((k + 1) * kBK);
        const unsigned char* base = smem + cur * STAGE;
        if constexpr (!INT8) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {  // two MFMA K-steps of 64 bytes
                int8_t_v bf[TJ];
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const uint4* q = (const uint4*)(base + b_row0 + j * 32 * kRowBytes + h * 64 + kb * 32);
                    const uint4 lo = q[0], hi = q[1];
                    bf[j] = int8_t_v{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
                }
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const uint4* q = (const uint4*)(base + a_row0 + i * 32 * kRowBytes + h * 64 + kb * 32);
                    const uint4 lo = q[0], hi = q[1];
                    const int8_t_v af = int8_t_v{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
#pragma unroll
                    for (int j = 0; j < TJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, bf[j], acc[i][j], 0, 0, 0, 127, 0, 127);
                }
                __builtin_amdgcn_sched_barrier(0);  // bound the number of fragments in flight (register pressure)
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {  // four MFMA K-steps of 32 bytes
                int4_t bf[TJ];
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    const uint4 v = *(const uint4*)(base + b_row0 + j * 32 * kRowBytes + s * 32 + kb * 16);
                    bf[j] = int4_t{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                }
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const uint4 v = *(const uint4*)(base + a_row0 + i * 32 * kRowBytes + s * 32 + kb * 16);
                    const int4_t af = int4_t{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
#pragma unroll
                    for (int j = 0; j < TJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[j], acc[i][j], 0, 0, 0);
                }
            }
        }
        if (k + 1 < steps) GLA_STORE_STEP(cur ^ 1);  // that buffer was last read in step k-1
        __syncthreads();
    }
#undef GLA_LOAD_STEP
#undef GLA_STORE_STEP

    // ---- epilogue: lane holds column r32 of each 32-wide tile, rows 8*(e/4) + 4*kb + e%4
    float sb[TJ];
    bool n_ok[TJ];
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
        const int n = n0 + wn * 64 + j * 32 + r32;
        n_ok[j] = n < p.N;
        sb[j] = ((p.csm & 1) && n_ok[j]) ? load_as_float(p.scales, p.meta_dt, n) : 1.0f;
    }
    const bool row_scale = (p.csm & 2) != 0;
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

template <bool INT8, int BM>
int launch_bm(const Gemm8Args& a, hipStream_t stream) {
    const size_t smem = 2 * (size_t)(BM + kBN) * kRowBytes;
    static bool configured = false;  // per instantiation; the attribute is sticky per function
    auto kern = gemm_8bit_kernel<INT8, BM>;
    if (!configured) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_8bit: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n), dim3(kThreads8), smem, stream, a);
    return check_hip(hipGetLastError(), "gemm_8bit launch");
}

}  // namespace

bool gemm_8bit_eligible(const gla_matmul_args& p) {
    const bool fp8 = p.input_dtype == GLA_DT_FP8 && p.w_dtype == GLA_DT_FP8 && p.acc_dtype == GLA_DT_FP32;
    const bool i8 = p.input_dtype == GLA_DT_INT8 && p.w_dtype == GLA_DT_INT8;
    if (!fp8 && !i8) return false;
    if (p.elements_per_sample != 1 || p.W_nbits != 8 || p.W_group_mode != GLA_WGM_NONE) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.K % kBK != 0 || p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    if (i8 && p.acc_dtype != GLA_DT_INT32) return false;
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if (p.output_dtype == GLA_DT_INT32 && !(i8 && p.channel_scale_mode == GLA_CSM_NONE)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int launch_gemm_8bit(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype;
    const bool i8 = p.input_dtype == GLA_DT_INT8;
    a.tiles_n = ceil_div(p.N, kBN);
    int bm = p.tile_config > 0 ? p.tile_config : (p.M > 128 ? 256 : (p.M > 64 ? 128 : 64));
    if (bm != 64 && bm != 128 && bm != 256) bm = 256;
    if (!i8 && bm == 256) bm = 128;  // the fp8 256-row tile does not fit the register file yet
    a.tiles_m = ceil_div(p.M, bm);
    if (i8) {
        if (bm == 256) return launch_bm<true, 256>(a, stream);
        if (bm == 128) return launch_bm<true, 128>(a, stream);
        return launch_bm<true, 64>(a, stream);
    }
    if (bm == 256) return launch_bm<false, 256>(a, stream);
    if (bm == 128) return launch_bm<false, 128>(a, stream);
    return launch_bm<false, 64>(a, stream);
}

}  // namespace gla
