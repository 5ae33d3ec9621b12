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
// The second kernel of the file takes MXFP4 activations (codes + e8m0 bytes) on the same weights, 3..32 rows, and
// feeds both sides to the block-scaled MFMA unconverted.
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

// ---------------------------------------------------------------------------------------------------------
// MXFP4 x MXFP4 at 3..32 rows: the same walk over the weights, but nothing is converted.  A lane's 16 weight
// bytes (32 e2m1 codes of one 32-block) ARE its share of the A operand of v_mfma_scale_f32_16x16x128_f8f6f4,
// the block's e8m0 byte its scale; the B operand is the same 32-block of 16 activation rows (codes and e8m0
// bytes staged through LDS like the 16-bit activations above), so one instruction multiplies 16 weight rows
// with 16 activation rows over 128 K-values and applies both block scales (reference:
// gemlite/triton_kernels/gemm_splitK_kernels.py:536-770, `tl.dot_scaled` on e2m1 operands).  XT = 1 or 2 tiles of
// 16 activation rows.  Between the vector-unit streaming kernel (1-2 rows, 4 on small layers) and the tiled
// GEMM (64-row tiles through LDS, split K, a finishing launch and a scale-regrouping launch in front).
//  * 8 / 32 rows: 4096^2 5.1 / 6.5 us (tiled GEMM 14.1 / 15.3), 8192^2 13.0 / 16.0 (17.8 / 19.9), 14336 x 4096
//    11.3 / 14.5 (16.1 / 18.6), 16384^2 42.7 / 48.0 (41.0 / 44.4: the dispatcher keeps the GEMM there).
//  * The bound is the access pattern the [N, K/2] layout forces on an MFMA operand: a wave instruction reads 16
//    rows x 64 bytes.  The same kernel reading 1 KiB contiguous per instruction (weights regrouped by operand;
//    timing only, not built) took 28 / 35 us at 1 / 16 rows on 16384^2 and 9.5 / 11.1 on 8192^2.  Loading the
//    activations per lane from global memory instead of through LDS (no barrier in the K loop) gave the same
//    times up to 16 rows and 10-20 % worse ones at 32.
struct Mx4SkArgs {
    const uint8_t* x;         // [M, K/2] e2m1 pairs
    const uint8_t* sx;        // [ceil32(M), K/32] e8m0
    const uint8_t* w;         // [N, K/2]
    const uint8_t* scales;    // [N, K/32]
    void* out;
    int M, N, K;
    int64_t xsm, sxm, wsn, osm, msn;   // bytes (osm: elements)
    int out_dt;
    const void* bias;
    int bias_dt;
};

typedef int i32x8s __attribute__((ext_vector_type(8)));

template <int RT, int XT>
__global__ __launch_bounds__(kWavesS * 64) void mx4_skinny_kernel(Mx4SkArgs a) {
    constexpr int STEPK = 128, UN = 2;
    constexpr int KC = STEPK * UN * kWavesS;   // 2048 K-values per chunk
    constexpr int ROWB = KC / 2 + 16;          // LDS row of codes: 1 KiB + padding (the 16 rows of a quarter-wave in different banks)
    constexpr int SROW = KC / 32 + 4;          // LDS row of scale bytes: 64 + padding
    constexpr int ROWS = 16 * XT;
    constexpr int PIECES = KC / 2 / 16;        // 16-byte pieces per row and chunk: 64
    constexpr int XS = ROWS * PIECES / (kWavesS * 64);  // code pieces a thread stages per chunk: 2 XT
    extern __shared__ __align__(16) unsigned char xbuf[];  // [2][ROWS][ROWB] codes, then [2][ROWS][SROW] scales
    unsigned char* sbuf = xbuf + 2 * ROWS * ROWB;
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
    f32x4s acc[RT][XT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) acc[t][xt] = f32x4s{0.0f, 0.0f, 0.0f, 0.0f};
    const int steps = a.K / STEPK;
    const int chunks = (a.K + KC - 1) / KC;

    // staging of a chunk: code pieces id = i * 512 + tid -> (row, piece); the scale bytes of a row are 4 pieces,
    // taken by the first 4 ROWS threads.  Rows past M repeat row M - 1 (their results are not stored).
    const uint8_t* xsrc[XS];
    int xcol[XS], xdst[XS];
#pragma unroll
    for (int i = 0; i < XS; ++i) {
        const int id = i * (kWavesS * 64) + tid;
        const int row = id / PIECES, col = id % PIECES;
        xsrc[i] = a.x + (int64_t)(row < a.M ? row : a.M - 1) * a.xsm;
        xcol[i] = col * 16;
        xdst[i] = row * ROWB + col * 16;
    }
    const bool s_stager = tid < 4 * ROWS;
    const int s_row = tid >> 2, s_col = (tid & 3) * 16;
    const uint8_t* ssrc = a.sx + (int64_t)(s_stager && s_row < a.M ? s_row : a.M - 1) * a.sxm;
    u32x4s xs[XS], ss;
    auto x_load = [&](int c) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
            int kb = c * (KC / 2) + xcol[i];
            if (kb > a.K / 2 - 16) kb = a.K / 2 - 16;  // pieces past the end of K repeat the last one; never multiplied
            xs[i] = *(const u32x4s*)(xsrc[i] + kb);
        }
        if (s_stager) {
            // 16 scale bytes as four dwords (rows are only 4-byte aligned in general, and K/32 is a multiple of 8,
            // not of 16: a piece can end inside the row).  Dwords past the end repeat the last one; never multiplied.
            const int sb = c * (KC / 32) + s_col, last = a.K / 32 - 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int o = sb + 4 * j;
                ss[j] = *(const uint32_t*)(ssrc + (o < last ? o : last));
            }
        }
    };
    auto x_store = [&](int c) __attribute__((always_inline)) {
        unsigned char* base = xbuf + (c & 1) * (ROWS * ROWB);
#pragma unroll
        for (int i = 0; i < XS; ++i) *(u32x4s*)(base + xdst[i]) = xs[i];
        if (s_stager) {
            uint32_t* d = (uint32_t*)(sbuf + (c & 1) * (ROWS * SROW) + s_row * SROW + s_col);
            d[0] = ss[0]; d[1] = ss[1]; d[2] = ss[2]; d[3] = ss[3];
        }
    };
    struct Batch {
        u32x4s wv[UN][RT];
        uint32_t sc[RT][2];
    };
    auto w_load = [&](Batch& b, int c) __attribute__((always_inline)) {
        int s0 = c * (UN * kWavesS) + UN * wave;
        if (s0 > steps - UN) s0 = 0;  // pairs past the end re-read the first; never multiplied
#pragma unroll
        for (int t = 0; t < RT; ++t) {
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const uint4 q = load_streaming_u4(wrow[t] + (int64_t)(s0 + u) * kStepB);
                b.wv[u][t] = u32x4s{q.x, q.y, q.z, q.w};
            }
            const uint32_t* sp = (const uint32_t*)(srow[t] + s0 * 4);  // rows are 4-byte aligned in general
            b.sc[t][0] = sp[0]; b.sc[t][1] = sp[1];
        }
    };
    auto multiply = [&](const Batch& b, int c) __attribute__((always_inline)) {
        const unsigned char* cbase = xbuf + (c & 1) * (ROWS * ROWB) + r16 * ROWB + kq * 16;
        const unsigned char* sbase = sbuf + (c & 1) * (ROWS * SROW) + r16 * SROW;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int sl = UN * wave + u;  // step inside the chunk
            if (c * (UN * kWavesS) + sl < steps) {
#pragma unroll
                for (int xt = 0; xt < XT; ++xt) {
                    const u32x4s xv = *(const u32x4s*)(cbase + xt * 16 * ROWB + sl * (STEPK / 2));
                    const uint32_t sxw = *(const uint32_t*)(sbase + xt * 16 * SROW + sl * 4);
                    const int ex = (int)((sxw >> (8 * kq)) & 0xffu);
                    const i32x8s b8 = {(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3], 0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        const int ew = (int)((b.sc[t][u] >> (8 * kq)) & 0xffu);
                        const u32x4s wv = b.wv[u][t];
                        const i32x8s a8 = {(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3], 0, 0, 0, 0};
                        acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 4, 4, 0, ew, 0, ex);
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
    // lane holds D[n0 + 16 t + 4 kq + e][m = 16 xt + r16]; the waves' sums are added in wave order, one tile at a time
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
            if (t || xt) __syncthreads();
            red[wave][lane] = acc[t][xt];
            __syncthreads();
            const int m = 16 * xt + r16;
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
}

template <int RT, int XT>
int launch_variant4(const Mx4SkArgs& a, hipStream_t stream) {
    constexpr int KC = 128 * 2 * kWavesS;
    const size_t smem = 2 * 16 * XT * (size_t)(KC / 2 + 16) + 2 * 16 * XT * (size_t)(KC / 32 + 4);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = mx4_skinny_kernel<RT, XT>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "mx4_skinny: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(ceil_div(ceil_div(a.N, 16), RT)), dim3(kWavesS * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "mx4_skinny launch");
}

template <int XT>
int launch_sk4(const Mx4SkArgs& a, hipStream_t stream) {
    // as many row tiles per wave as still leave every CU a workgroup
    const int tiles = ceil_div(a.N, 16);
    if (tiles >= 4 * 256) return launch_variant4<4, XT>(a, stream);
    if (tiles >= 2 * 256) return launch_variant4<2, XT>(a, stream);
    return launch_variant4<1, XT>(a, stream);
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

// MXFP4 x MXFP4 (codes and e8m0 bytes on both sides), up to 32 rows
static bool mx4_skinny_ok(const gla_matmul_args& p) {
    if (p.input_dtype != GLA_DT_MXFP4 || p.x_quant_from != 0) return false;
    if (p.M < 1 || p.M > 32 || p.group_size != 32 || p.channel_scale_mode != GLA_CSM_MX) return false;
    if (p.scales == nullptr || p.scales_x == nullptr || p.sx_dtype != GLA_DT_UINT8) return false;
    if (!(p.W_nbits == 4 && p.elements_per_sample == 2)) return false;
    if (p.K % 256 != 0) return false;  // whole pairs of steps
    if (p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3) || p.sx_stride_m % 4 != 0 || ((uintptr_t)p.scales_x & 3)) return false;
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.out_stride_n != 1 || p.meta_stride_g != 1 || p.sx_stride_g != 1) return false;
    if (p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0 || ((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    return p.output_dtype == GLA_DT_FP32 || p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16;
}

bool mx_skinny_eligible(const gla_matmul_args& p) {
    if (p.input_dtype == GLA_DT_MXFP4) return mx4_skinny_ok(p);
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
    if (p.input_dtype == GLA_DT_MXFP4 && mx4_skinny_ok(p)) {
        Mx4SkArgs a;
        a.x = (const uint8_t*)p.x; a.sx = (const uint8_t*)p.scales_x; a.w = (const uint8_t*)p.w; a.scales = (const uint8_t*)p.scales;
        a.out = p.out; a.M = p.M; a.N = p.N; a.K = p.K;
        a.xsm = p.x_stride_m; a.sxm = p.sx_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.msn = p.meta_stride_n;
        a.out_dt = p.output_dtype; a.bias = p.bias; a.bias_dt = p.bias_dtype;
        return p.M <= 16 ? launch_sk4<1>(a, stream) : launch_sk4<2>(a, stream);
    }
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
