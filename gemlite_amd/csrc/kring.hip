// Skinny matmul (3..32 rows) for layers whose two operands are both narrow and K-contiguous:
//
//   MXFP4 x MXFP4   e2m1 nibble pairs, one e8m0 scale per 32 values on either side
//                   (v_mfma_scale_f32_16x16x128_f8f6f4, both block scales applied by the instruction)
//   fp8 x fp8       e4m3 bytes, per-token x per-channel scales in the epilogue (the same instruction, unit scales)
//   int8 x int8     exact int32 sums (v_mfma_i32_16x16x64_i8), scaled in the epilogue or stored as int32
//
// The decode-batch path of dynamically quantised A8W8 and A4W4 layers, between the streaming kernels (dot products
// on the vector unit, 1-2 rows) and the tiled GEMMs (64-row tiles, K split over workgroups, a finishing launch and,
// for MXFP4, a scale-regrouping launch in front).  Reference: gemlite/triton_kernels/gemm_splitK_kernels.py:300-523
// (8-bit operands) and :536-770 (`tl.dot_scaled` on e2m1 operands); epilogue scales :471-488 of gemm_kernels.py.
//
//  * Nothing is converted: a lane's 16 (fp8: 32) operand bytes of a weight row ARE its share of the MFMA's A operand,
//    the same bytes of an activation row its share of B, so one instruction multiplies 16 weight rows with 16
//    activation rows over 128 bytes of K.  XT = 1 or 2 tiles of 16 activation rows, RT = 1, 2 or 4 tiles of 16 weight
//    rows per wave.
//  * Every operand is copied global -> LDS by the load unit (global_load_lds) into a ring that is private to the
//    wave: a copy instruction moves 8 rows x 128 contiguous bytes, so the [rows, K] arrays are read in whole 128-byte
//    lines (an MFMA operand loaded straight into registers touches 16 rows x 64 bytes per instruction, and that
//    access pattern, not the arithmetic, bounded two earlier forms of this kernel: 13.0-13.8 us on an 8192^2 MXFP4
//    layer at 8 rows whatever else was varied, 9.5-11.1 with the same code reading 1 KiB contiguous per instruction
//    for timing; this form: 11.1).  Nothing waits in registers, and there is no barrier before the final sum of the
//    waves' accumulators through LDS in wave order (deterministic, no workspace, one launch).
//  * A tile of a turn (16 rows x 128 bytes) is 2 KiB, its 16-byte slots XOR-swizzled by row >> 1 so that the
//    operand reads (16 rows, one slot each) fall in different banks; MXFP4 tiles carry their 16 x 8 scale bytes.
//    The NW waves take the turns of K in order, NB turns per wave in flight; a wave waits on the vector-memory
//    counter only.
//  * MXFP4, 8 / 32 rows (us; tiled GEMM in brackets): 4096^2 4.7 / 6.5 (14.1 / 15.3), 8192^2 11.1 / 14.4 (17.8 / 19.9),
//    4096 x 14336 9.7 / 14.2 (18.9 / 21.0), 14336 x 4096 10.3 / 13.9 (16.1 / 18.6), 16384^2 34.0 / 40.8 (41.0 / 44.4).
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4r __attribute__((ext_vector_type(4)));
typedef float f32x4r __attribute__((ext_vector_type(4)));
typedef int i32x4r __attribute__((ext_vector_type(4)));
typedef int i32x8r __attribute__((ext_vector_type(8)));

enum { R_MX44 = 0, R_FP8 = 1, R_INT8 = 2 };

struct KRingArgs {
    const uint8_t* x;         // [M, K bytes or K/2 nibble pairs]
    const uint8_t* w;         // [N, the same]
    const uint8_t* bsx;       // MXFP4: activation block scales [ceil32(M), K/32] e8m0
    const uint8_t* bsw;       // MXFP4: weight block scales [N, K/32]
    const void* scales;       // 8-bit: per-channel scales [N] (channel_scale_mode bit 0)
    const void* scales_x;     // 8-bit: per-token scales [M] (bit 1)
    void* out;
    int M, N, Kb;             // Kb = operand bytes per row
    int64_t xsm, wsn, bsxm, bswn, sxm, osm;   // bytes (sxm, osm: elements)
    int csm, meta_dt, sx_dt, out_dt;
    const void* bias;
    int bias_dt;
};

// s_waitcnt vmcnt(N) only: vmcnt is bits 3:0 and 15:14, expcnt (6:4) and lgkmcnt (11:8) left at "no wait"
template <int N>
__device__ __forceinline__ void wait_vmcnt_r() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <int MODE, int RT, int XT, int NW, int NB>
__global__ __launch_bounds__(NW * 64) void kring_kernel(KRingArgs a) {
    constexpr bool BS = MODE == R_MX44;                 // block scales travel with the tiles
    constexpr int TILE = 2048 + (BS ? 256 : 0);
    constexpr int NT = RT + XT;
    constexpr int OPS = (2 + (BS ? 1 : 0)) * NT;        // copy instructions per turn
    typedef typename std::conditional<MODE == R_INT8, i32x4r, f32x4r>::type acc_t;
    static_assert((NB - 1) * OPS < 64, "outstanding copies must fit the vmcnt counter");
    extern __shared__ __align__(16) unsigned char ring[];  // [NW][NB][NT][TILE]
    __shared__ acc_t red[NW][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16 * RT;
    unsigned char* mine = ring + (size_t)wave * NB * NT * TILE;

    // copy plan of a turn: per tile two code instructions (rows 8j + lane / 8, slot lane % 8 <- piece slot ^ (row >> 1))
    // and, with block scales, one for the scale bytes (row (lane / 2) % 16, dword lane % 2; the upper half-wave
    // writes a duplicate)
    const uint8_t* csrc[NT][2];
    const uint8_t* ssrc[BS ? NT : 1];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const bool is_w = i < RT;
        auto row_ptr = [&](int row, bool scale) -> const uint8_t* {
            if (is_w) {
                int n = n0 + 16 * i + row;
                if (n > a.N - 1) n = a.N - 1;  // rows past the end repeat the last one; never stored
                return scale ? a.bsw + (int64_t)n * a.bswn : a.w + (int64_t)n * a.wsn;
            }
            int m = 16 * (i - RT) + row;
            if (m > a.M - 1) m = a.M - 1;
            return scale ? a.bsx + (int64_t)m * a.bsxm : a.x + (int64_t)m * a.xsm;
        };
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * j + (lane >> 3), slot = lane & 7;
            csrc[i][j] = row_ptr(row, false) + ((slot ^ (row >> 1)) & 7) * 16;
        }
        if constexpr (BS) ssrc[i] = row_ptr((lane >> 1) & 15, true) + (lane & 1) * 4;
    }
    auto issue = [&](int p, int slot) __attribute__((always_inline)) {
        unsigned char* base = mine + slot * (NT * TILE);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(csrc[i][j] + (int64_t)p * 128),
                                                 (__attribute__((address_space(3))) void*)(base + i * TILE + j * 1024), 16, 0, 0);
            if constexpr (BS)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ssrc[i] + (int64_t)p * 8),
                                                 (__attribute__((address_space(3))) void*)(base + i * TILE + 2048), 4, 0, 0);
        }
    };
    acc_t acc[RT][XT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) acc[t][xt] = acc_t{0, 0, 0, 0};
    const int code_off = r16 * 128, swz = r16 >> 1, scale_off = 2048 + r16 * 8;
    auto slot16 = [&](const unsigned char* tile, int piece) __attribute__((always_inline)) {
        return *(const u32x4r*)(tile + code_off + ((piece ^ swz) & 7) * 16);
    };
    auto multiply = [&](int slot) __attribute__((always_inline)) {
        const unsigned char* base = mine + slot * (NT * TILE);
        if constexpr (MODE == R_FP8) {
            // a turn is one MFMA: the lane's 32 bytes are slots 2 kq and 2 kq + 1 of its row
#pragma unroll
            for (int xt = 0; xt < XT; ++xt) {
                const unsigned char* xb = base + (RT + xt) * TILE;
                const u32x4r x0 = slot16(xb, 2 * kq), x1 = slot16(xb, 2 * kq + 1);
                const i32x8r b8 = {(int)x0[0], (int)x0[1], (int)x0[2], (int)x0[3], (int)x1[0], (int)x1[1], (int)x1[2], (int)x1[3]};
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const unsigned char* wb = base + t * TILE;
                    const u32x4r w0 = slot16(wb, 2 * kq), w1 = slot16(wb, 2 * kq + 1);
                    const i32x8r a8 = {(int)w0[0], (int)w0[1], (int)w0[2], (int)w0[3], (int)w1[0], (int)w1[1], (int)w1[2], (int)w1[3]};
                    acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 0, 0, 0, 127, 0, 127);
                }
            }
        } else {
            // two MFMAs a turn (MXFP4: 128 K-values each; int8: 64): the lane's 16 bytes are slot 4 u + kq
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int xt = 0; xt < XT; ++xt) {
                    const unsigned char* xb = base + (RT + xt) * TILE;
                    const u32x4r xv = slot16(xb, 4 * u + kq);
                    int ex = 0;
                    if constexpr (BS) ex = (int)((*(const uint32_t*)(xb + scale_off + 4 * u) >> (8 * kq)) & 0xffu);
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        const unsigned char* wb = base + t * TILE;
                        const u32x4r wv = slot16(wb, 4 * u + kq);
                        if constexpr (MODE == R_INT8) {
                            acc[t][xt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(i32x4r{(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3]},
                                                                               i32x4r{(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3]},
                                                                               acc[t][xt], 0, 0, 0);
                        } else {
                            const int ew = (int)((*(const uint32_t*)(wb + scale_off + 4 * u) >> (8 * kq)) & 0xffu);
                            const i32x8r a8 = {(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3], 0, 0, 0, 0};
                            const i32x8r b8 = {(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3], 0, 0, 0, 0};
                            acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 4, 4, 0, ew, 0, ex);
                        }
                    }
                }
            }
        }
    };
    const int turns = a.Kb / 128;
    const int iters = (turns + NW - 1) / NW;
    // a wave whose turn lies past the end copies the last one again (same count of copies for everybody) and skips the multiply
    auto turn_of = [&](int it) { const int p = it * NW + wave; return p < turns ? p : turns - 1; };
#pragma unroll
    for (int b = 0; b < NB - 1; ++b)
        if (b < iters) issue(turn_of(b), b);
    int slot = 0, islot = NB - 1;
    for (int it = 0; it < iters; ++it) {
        const int later = iters - 1 - it;  // turns issued after this one
        if (later >= NB - 1) {
            issue(turn_of(it + NB - 1), islot);
            islot = islot == NB - 1 ? 0 : islot + 1;
            wait_vmcnt_r<(NB - 1) * OPS>();
        } else if (NB > 2 && later == 1) {  // the ring drains: `later` turns may still be in flight
            wait_vmcnt_r<(NB > 2 ? 1 : 0) * OPS>();
        } else if (NB > 3 && later == 2) {
            wait_vmcnt_r<(NB > 3 ? 2 : 0) * OPS>();
        } else if (NB > 4 && later == 3) {
            wait_vmcnt_r<(NB > 4 ? 3 : 0) * OPS>();
        } else {
            wait_vmcnt_r<0>();
        }
        asm volatile("" ::: "memory");
        if (it * NW + wave < turns) multiply(slot);
        slot = slot == NB - 1 ? 0 : slot + 1;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);  // the copies of the next turn go to the slot these reads came from
    }
    // lane holds D[n0 + 16 t + 4 kq + e][m = 16 xt + r16]; the waves' sums are added in wave order, one tile at a time
    const bool col_scale = !BS && (a.csm & 1), row_scale = !BS && (a.csm & 2);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
            if (t || xt) __syncthreads();
            red[wave][lane] = acc[t][xt];
            __syncthreads();
            const int m = 16 * xt + r16;
            if (wave != 0 || m >= a.M) continue;
            acc_t D = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < NW; ++w) D += red[w][lane];
            const float sa = row_scale ? load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm) : 1.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n0 + 16 * t + 4 * kq + e;
                if (n >= a.N) continue;
                const int64_t o = (int64_t)m * a.osm + n;
                if constexpr (MODE == R_INT8) {
                    if (a.out_dt == GLA_DT_INT32) {
                        ((int32_t*)a.out)[o] = D[e];
                        continue;
                    }
                }
                float v = (float)D[e];
                if constexpr (!BS) v *= sa * (col_scale ? load_as_float(a.scales, a.meta_dt, n) : 1.0f);
                if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n);
                store_from_float(a.out, a.out_dt, o, v);
            }
        }
    }
}

template <int MODE, int RT, int XT, int NW, int NB>
int launch_ring(const KRingArgs& a, hipStream_t stream) {
    const size_t smem = (size_t)NW * NB * (RT + XT) * (2048 + (MODE == R_MX44 ? 256 : 0));
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = kring_kernel<MODE, RT, XT, NW, NB>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "kring: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(ceil_div(ceil_div(a.N, 16), RT)), dim3(NW * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "kring launch");
}

template <int MODE>
int launch_mode_ring(const KRingArgs& a, hipStream_t stream) {
    // rows of tiles per wave so that about one workgroup per CU comes out; fewer, deeper waves where a wave has
    // 4 weight tiles to an activation tile (MXFP4, 16384^2 at 8 rows: 34.3 us with 4 tiles x 4 waves x 3 turns in
    // flight, 38.4 with 2 x 8 x 2, 35.2 with 1 x 8 x 4; 8192^2: 15.5 / 11.2 / 12.6; 4096^2: 8.9 / 6.1 / 4.7)
    const int tiles = ceil_div(a.N, 16);
    if constexpr (MODE == R_MX44) {
        if (a.M <= 16) {
            if (tiles >= 880) return launch_ring<MODE, 4, 1, 4, 3>(a, stream);
            if (tiles >= 440) return launch_ring<MODE, 2, 1, 8, 2>(a, stream);
            return launch_ring<MODE, 1, 1, 8, 4>(a, stream);
        }
        if (tiles >= 880) return launch_ring<MODE, 4, 2, 4, 2>(a, stream);
        if (tiles >= 440) return launch_ring<MODE, 2, 2, 4, 4>(a, stream);
        return launch_ring<MODE, 1, 2, 8, 2>(a, stream);
    } else {
        // 8-bit operands: an activation tile is as many bytes as a weight tile, and one tile per wave with many waves
        // does best (fp8 at 8 rows, 8192^2: 17.3 us with 1 tile x 16 waves x 2 turns, 17.6 with 1 x 8 x 4, 21.1 with
        // 2 x 8 x 2; 16384^2: 58.6 / 60.0 / 66.1) unless K is short and N long (14336 x 4096: 21.1 / 21.8 against 18.8
        // with 4 x 4 x 3)
        if (a.M <= 16) {
            if (tiles >= 880 && a.Kb < 8192) return launch_ring<MODE, 4, 1, 4, 3>(a, stream);
            if (tiles >= 440) return launch_ring<MODE, 1, 1, 16, 2>(a, stream);
            return launch_ring<MODE, 1, 1, 8, 4>(a, stream);
        }
        if (tiles >= 440) return launch_ring<MODE, 2, 2, 8, 2>(a, stream);
        return launch_ring<MODE, 1, 2, 8, 2>(a, stream);
    }
}

int ring_mode(const gla_matmul_args& p) {
    if (p.input_dtype == GLA_DT_MXFP4) return R_MX44;
    if (p.input_dtype == GLA_DT_FP8 && p.w_dtype == GLA_DT_FP8) return R_FP8;
    if (p.input_dtype == GLA_DT_INT8 && p.w_dtype == GLA_DT_INT8) return R_INT8;
    return -1;
}

}  // namespace

bool kring_eligible(const gla_matmul_args& p) {
    const int mode = ring_mode(p);
    if (mode < 0 || p.x_quant_from != 0 || p.M < 1 || p.M > 32) return false;
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0 || ((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    if (mode == R_MX44) {
        if (p.group_size != 32 || p.channel_scale_mode != GLA_CSM_MX || !(p.W_nbits == 4 && p.elements_per_sample == 2)) return false;
        if (p.scales == nullptr || p.scales_x == nullptr || p.sx_dtype != GLA_DT_UINT8) return false;
        if (p.K % 256 != 0) return false;  // whole turns of 128 bytes
        if (p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3) || p.sx_stride_m % 4 != 0 || ((uintptr_t)p.scales_x & 3)) return false;
        if (p.meta_stride_g != 1 || p.sx_stride_g != 1) return false;
        return p.output_dtype == GLA_DT_FP32 || p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16;
    }
    // fp8 x fp8 and int8 x int8: what the tiled 8-bit GEMM takes, K in whole turns
    if (mode == R_FP8 && p.acc_dtype != GLA_DT_FP32) return false;
    if (mode == R_INT8 && p.acc_dtype != GLA_DT_INT32) return false;
    if (p.elements_per_sample != 1 || p.W_nbits != 8 || p.W_group_mode != GLA_WGM_NONE) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.K % 128 != 0) return false;
    if (p.output_dtype == GLA_DT_INT32) return mode == R_INT8 && p.channel_scale_mode == GLA_CSM_NONE;
    if (!(p.output_dtype == GLA_DT_FP32 || p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int launch_kring(const gla_matmul_args& p, hipStream_t stream) {
    if (!kring_eligible(p)) {
        set_error("kring: MXFP4 x MXFP4, fp8 x fp8 or int8 x int8 operands, K-contiguous with 16-byte aligned rows, up to 32 "
                  "rows, K a multiple of 256 (MXFP4) or 128");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    const int mode = ring_mode(p);
    KRingArgs a;
    a.x = (const uint8_t*)p.x; a.w = (const uint8_t*)p.w; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = mode == R_MX44 ? p.K / 2 : p.K;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m;
    a.bsx = mode == R_MX44 ? (const uint8_t*)p.scales_x : nullptr; a.bsw = mode == R_MX44 ? (const uint8_t*)p.scales : nullptr;
    a.bsxm = p.sx_stride_m; a.bswn = p.meta_stride_n;
    a.scales = p.scales; a.scales_x = p.scales_x; a.sxm = p.sx_stride_m;
    a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype; a.out_dt = p.output_dtype;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    if (mode == R_MX44) return launch_mode_ring<R_MX44>(a, stream);
    if (mode == R_FP8) return launch_mode_ring<R_FP8>(a, stream);
    return launch_mode_ring<R_INT8>(a, stream);
}

}  // namespace gla
