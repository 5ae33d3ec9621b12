// Skinny GEMM (3..16 rows) for weight-only micro-scaled layers: fp16 / bf16 activations x MXFP8 bytes or
// MXFP4 nibble pairs kept as the [K, N] view of an [N, K] array (K contiguous), one e8m0 scale per 32
// values along K (reference: gemlite/helper.py:384-420; the kernel it takes the place of:
// gemlite/triton_kernels/gemm_splitK_kernels.py:525-770 with 16-bit activations).
//
// Between the streaming kernel of mx_stream.hip (dot products on the vector unit: its cost grows with
// every row) and the tiled GEMM of gemm_kbytes.hip (64-row tiles staged through LDS, K split over
// workgroups, a finishing kernel) the weights are read once, straight into registers, and multiplied on
// the matrix cores:
//  * A wave owns RT tiles of 16 weight rows (output columns).  Lane (r, q) = (lane % 16, lane / 16)
//    loads 16 bytes of row r per tile and step, the four q's adjacent pieces, so a wave instruction
//    reads 16 rows x 64 contiguous bytes and consecutive steps of a wave continue those rows.  The 16
//    bytes lie inside one 32-value block: one scale byte per load.
//  * v_cvt_scalef32_pk_{f16,bf16}_{fp4,fp8} turns 8 codes and the block's scale into the four registers
//    of a 16-bit MFMA operand: the operand is the dequantised weight.  v_mfma_f32_16x16x32 multiplies
//    it with the activations of up to 16 rows, which a lane loads (through the vector cache, they are
//    small) for the same K positions once per step for all RT tiles.
//  * The 8 waves of a workgroup take the steps of K in turn, two adjacent steps at a time, and add their
//    accumulators through LDS in wave order; no workspace, no second kernel, deterministic.
//  * 16384^2 MXFP4: 45 us at 3 rows, 51 at 16 (a pure read in this access pattern: 30-34 us; the tiled GEMM:
//    52-62 us); MXFP8: 73-79 us.
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4s __attribute__((ext_vector_type(4)));
typedef float f32x4s __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8s __attribute__((ext_vector_type(8)));
typedef _Float16 half8s __attribute__((ext_vector_type(8)));

constexpr int kWavesS = 8;   // waves per workgroup, interleaved over K
constexpr int kStepB = 64;   // weight bytes per row and step

struct MxSkArgs {
    const uint16_t* x;
    const uint8_t* w;
    const uint8_t* scales;
    void* out;
    int M, N, K;
    int64_t xsm, wsn, osm, msn;
    int out_dt;
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

template <bool BF16>
__device__ __forceinline__ f32x4s mfma16s(const u32x4s& a, const u32x4s& b, f32x4s c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8s, a), __builtin_bit_cast(bf16x8s, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8s, a), __builtin_bit_cast(half8s, b), c, 0, 0, 0);
}

// 8 codes (W4: one dword; W8: two) times 2^(e - 127), e in the exponent field of `scale`
template <bool W4, bool BF16>
__device__ __forceinline__ u32x4s codes_to_operand_mx(uint32_t d0, uint32_t d1, float scale) {
    u32x4s o;
    if constexpr (W4) {
        if constexpr (BF16) {
            o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d0, scale, 0));
            o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d0, scale, 1));
            o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d0, scale, 2));
            o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(d0, scale, 3));
        } else {
            o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, scale, 0));
            o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, scale, 1));
            o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, scale, 2));
            o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, scale, 3));
        }
    } else {
        if constexpr (BF16) {
            o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, scale, false));
            o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d0, scale, true));
            o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, scale, false));
            o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(d1, scale, true));
        } else {
            o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, scale, false));
            o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d0, scale, true));
            o[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, scale, false));
            o[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(d1, scale, true));
        }
    }
    return o;
}

// W4: a step is 128 K-values (a lane's 16 bytes = 32 codes = block 4 step + q, four MFMAs of 8 codes);
// W8: 64 K-values (16 codes = half of block 2 step + q / 2, two MFMAs).
// K is walked in chunks of KC values = 2 steps per wave.  The activations of a chunk (16 rows) are shared by
// all waves of the workgroup through LDS, double-buffered: loaded into registers two chunks ahead, written
// to LDS one chunk ahead, one barrier per chunk.  (Loaded per lane from global memory instead, they are
// four times the weight bytes per instruction stream and the CU's load unit becomes the bound: 16384^2
// MXFP4 took 49 us at 2 rows and 59 us at 16.)  Weights are loaded one chunk ahead.
template <bool W4, bool BF16, int RT>
__global__ __launch_bounds__(kWavesS * 64) void mx_skinny_kernel(MxSkArgs a) {
    constexpr int XV = W4 ? 4 : 2;             // 16-byte activation pieces (= MFMAs per tile) per lane and step
    constexpr int STEPK = W4 ? 128 : 64;       // K-values per step
    constexpr int UN = 2;                      // steps per wave and chunk
    constexpr int KC = STEPK * UN * kWavesS;   // K-values per chunk: 2048 / 1024
    constexpr int ROWB = KC * 2 + 16;          // LDS row: a chunk of one activation row, padded so that the 16 rows
                                               // a quarter-wave reads lie in different banks
    constexpr int PIECES = KC / 8;             // 16-byte pieces per row and chunk
    constexpr int XS = 16 * PIECES / (kWavesS * 64);  // pieces a thread stages per chunk: 8 / 4
    extern __shared__ __align__(16) unsigned char xbuf[];  // [2][16][ROWB]
    __shared__ f32x4s red[kWavesS][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16 * RT;
    const uint8_t* wrow[RT];
    const uint8_t* srow[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        int n = n0 + 16 * t + r16;
        if (n > a.N - 1) n = a.N - 1;  // rows past the end repeat the last one; never stored
        wrow[t] = a.w + (int64_t)n * a.wsn + 16 * kq;
        srow[t] = a.scales + (int64_t)n * a.msn;
    }
    f32x4s acc[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[t] = f32x4s{0.0f, 0.0f, 0.0f, 0.0f};
    const int steps = a.K / STEPK;
    const int chunks = (a.K + KC - 1) / KC;

    // staging: piece id = i * 512 + tid -> (row, piece of the row)
    // only the M rows that exist are staged (lanes of further rows read row M - 1; their results are not stored)
    const uint16_t* xsrc[XS];
    int xcol[XS], xdst[XS];
    bool xlive[XS];
#pragma unroll
    for (int i = 0; i < XS; ++i) {
        const int id = i * (kWavesS * 64) + tid;
        const int row = id / PIECES, col = id % PIECES;
        xlive[i] = row < a.M;
        xsrc[i] = a.x + (int64_t)(xlive[i] ? row : 0) * a.xsm;
        xcol[i] = col * 8;
        xdst[i] = row * ROWB + col * 16;
    }
    u32x4s xs[XS];
    auto x_load = [&](int c) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            int k = c * KC + xcol[i];
            if (k > a.K - 8) k = a.K - 8;  // pieces past the end of K repeat the last one; never multiplied
            if (xlive[i]) xs[i] = *(const u32x4s*)(xsrc[i] + k);
        }
    };
    auto x_store = [&](int c) __attribute__((always_inline)) {
        unsigned char* base = xbuf + (c & 1) * (16 * ROWB);
#pragma unroll
        for (int i = 0; i < XS; ++i)
            if (xlive[i]) *(u32x4s*)(base + xdst[i]) = xs[i];
    };
    // A wave takes two adjacent steps of a chunk (2 wave, 2 wave + 1): the scale bytes of both are then 8 (W4)
    // or 4 (W8) consecutive bytes of the row, one load per tile and chunk.  (One byte load per tile and step
    // made the kernel a fifth slower: the CU's load unit spends as long on a byte per lane as on 16.)
    struct Batch {
        u32x4s wv[UN][RT];
        uint32_t sc[RT][W4 ? 2 : 1];
    };
    auto w_load = [&](Batch& b, int c) __attribute__((always_inline)) {
        // chunks have whole pairs of steps (K is a multiple of two steps); pairs past the end re-read the first
        int s0 = c * (UN * kWavesS) + UN * wave;
        if (s0 > steps - UN) s0 = 0;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const uint4 q = load_streaming_u4(wrow[t] + (int64_t)(s0 + u) * kStepB);
                b.wv[u][t] = u32x4s{q.x, q.y, q.z, q.w};
            }
            if constexpr (W4) {
                const uint2 w = *(const uint2*)(srow[t] + s0 * 4);
                b.sc[t][0] = w.x; b.sc[t][1] = w.y;
            } else {
                b.sc[t][0] = *(const uint32_t*)(srow[t] + s0 * 2);
            }
        }
    };
    const int xoff = (r16 < a.M ? r16 : a.M - 1) * ROWB + kq * (STEPK / 2);  // this lane's bytes of a step's activations inside an LDS row
    auto multiply = [&](const Batch& b, int c) __attribute__((always_inline)) {
        const unsigned char* base = xbuf + (c & 1) * (16 * ROWB) + xoff;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int sl = UN * wave + u;  // step inside the chunk
            if (c * (UN * kWavesS) + sl < steps) {
                u32x4s xv[XV];
#pragma unroll
                for (int j = 0; j < XV; ++j) xv[j] = *(const u32x4s*)(base + sl * (STEPK * 2) + 16 * j);
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    // this lane's block: W4 byte kq of the step's word, W8 byte 2 u + kq / 2 of the pair's
                    const uint32_t e8 = W4 ? (b.sc[t][u] >> (8 * kq)) & 0xffu : (b.sc[t][0] >> (8 * (2 * u + kq / 2))) & 0xffu;
                    const float scale = __builtin_bit_cast(float, e8 << 23);
#pragma unroll
                    for (int j = 0; j < XV; ++j) {
                        u32x4s op;
                        if constexpr (W4) op = codes_to_operand_mx<W4, BF16>(b.wv[u][t][j], 0u, scale);
                        else op = codes_to_operand_mx<W4, BF16>(b.wv[u][t][2 * j], b.wv[u][t][2 * j + 1], scale);
                        acc[t] = mfma16s<BF16>(op, xv[j], acc[t]);
                    }
                }
            }
        }
    };
    Batch b0, b1;
    x_load(0);
    w_load(b0, 0);
    x_store(0);
    if (chunks > 1) x_load(1);
    for (int c = 0; c < chunks; c += 2) {
        __syncthreads();  // chunk c is in LDS; everybody is done with the buffer chunk c + 1 goes to
        if (c + 1 < chunks) {
            x_store(c + 1);
            w_load(b1, c + 1);
        }
        if (c + 2 < chunks) x_load(c + 2);
        multiply(b0, c);
        if (c + 1 < chunks) {
            __syncthreads();
            if (c + 2 < chunks) {
                x_store(c + 2);
                w_load(b0, c + 2);
            }
            if (c + 3 < chunks) x_load(c + 3);
            multiply(b1, c + 1);
        }
    }
    // lane holds D[n0 + 16 t + 4 kq + e][m = r16]; the waves' sums are added in wave order, one tile at a time
    const int m = r16;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        if (t) __syncthreads();
        red[wave][lane] = acc[t];
        __syncthreads();
        if (wave != 0 || m >= a.M) continue;
        f32x4s D = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < kWavesS; ++w) D += red[w][lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = n0 + 16 * t + 4 * kq + e;
            if (n >= a.N) continue;
            float v = D[e];
            if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n);
            store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + n, v);
        }
    }
}

template <bool W4, bool BF16, int RT>
int launch_variant(const MxSkArgs& a, hipStream_t stream) {
    constexpr int KC = (W4 ? 128 : 64) * 2 * kWavesS;
    const size_t smem = 2 * 16 * (size_t)(KC * 2 + 16);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = mx_skinny_kernel<W4, BF16, RT>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "mx_skinny: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(ceil_div(ceil_div(a.N, 16), RT)), dim3(kWavesS * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "mx_skinny launch");
}

template <bool W4, bool BF16>
int launch_sk(const MxSkArgs& a, hipStream_t stream) {
    // as many row tiles per wave as still leave every CU a workgroup (16384^2 MXFP4, 8 rows: 51 / 56 / 70 us
    // with 4 / 2 / 1 tiles); MXFP8 reads twice the bytes per activation and does best with 2
    const int tiles = ceil_div(a.N, 16);
    if (tiles >= 4 * 256 && W4) return launch_variant<W4, BF16, 4>(a, stream);
    if (tiles >= 2 * 256) return launch_variant<W4, BF16, 2>(a, stream);
    return launch_variant<W4, BF16, 1>(a, stream);
}

}  // namespace

bool mx_skinny_eligible(const gla_matmul_args& p) {
    if (!(p.input_dtype == GLA_DT_MXFP16 || p.input_dtype == GLA_DT_MXBF16)) return false;
    if (p.M < 1 || p.M > 16 || p.group_size != 32 || p.channel_scale_mode != GLA_CSM_NONE || p.scales == nullptr) return false;
    const bool w4 = p.W_nbits == 4 && p.elements_per_sample == 2;
    const bool w8 = p.W_nbits == 8 && p.elements_per_sample == 1;
    if (!w4 && !w8) return false;
    if (p.K % (w4 ? 256 : 128) != 0) return false;  // whole pairs of steps
    if (p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3)) return false;  // a pair's scale bytes are read as 32-bit words
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.out_stride_n != 1 || p.meta_stride_g != 1) return false;
    if (p.x_stride_m % 8 != 0 || p.w_stride_n % 16 != 0 || ((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    switch (p.output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_MXFP16: case GLA_DT_MXBF16: break;
        default: return false;
    }
    return true;
}

int launch_mx_skinny(const gla_matmul_args& p, hipStream_t stream) {
    if (!mx_skinny_eligible(p)) {
        set_error("mx_skinny: weight-only MX operands, K-contiguous with 16-byte aligned rows, up to 16 rows, "
                  "K a multiple of 256 (MXFP4) or 128 (MXFP8)");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    MxSkArgs a;
    a.x = (const uint16_t*)p.x; a.w = (const uint8_t*)p.w; a.scales = (const uint8_t*)p.scales; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.msn = p.meta_stride_n;
    a.out_dt = p.output_dtype == GLA_DT_MXFP16 ? GLA_DT_FP16 : (p.output_dtype == GLA_DT_MXBF16 ? GLA_DT_BF16 : p.output_dtype);
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    const bool bf16 = p.input_dtype == GLA_DT_MXBF16;
    const bool w4 = p.elements_per_sample == 2;
    if (w4) return bf16 ? launch_sk<true, true>(a, stream) : launch_sk<true, false>(a, stream);
    return bf16 ? launch_sk<false, true>(a, stream) : launch_sk<false, false>(a, stream);
}

}  // namespace gla
