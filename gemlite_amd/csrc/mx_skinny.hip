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
// the block's e8m0 byte its scale; the B operand is the same 32-block of 16 activation rows, so one instruction
// multiplies 16 weight rows with 16 activation rows over 128 K-values and applies both block scales (reference:
// gemlite/triton_kernels/gemm_splitK_kernels.py:536-770, `tl.dot_scaled` on e2m1 operands).  XT = 1 or 2 tiles of
// 16 activation rows.  Between the vector-unit streaming kernel (1-2 rows) and the tiled GEMM (64-row tiles
// through LDS, split K, a finishing launch and a scale-regrouping launch in front).
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

// s_waitcnt vmcnt(N) only: vmcnt is bits 3:0 and 15:14, expcnt (6:4) and lgkmcnt (11:8) left at "no wait"
template <int N>
__device__ __forceinline__ void wait_vmcnt_sk() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Every operand is copied global -> LDS by the load unit (global_load_lds) into a ring that is private to the wave:
// a copy instruction moves 8 rows x 128 contiguous bytes (the codes of a pair of steps), so rows are read in whole
// 128-byte lines instead of the 16 x 64 bytes an MFMA operand load touches, nothing waits in registers, and there is
// no barrier before the final sum of the waves' accumulators.  A tile (16 weight rows, or 16 activation rows) of a
// pair is 2 KiB of codes, 16-byte slots XOR-swizzled by row >> 1 so that the operand reads (16 rows, one slot each)
// fall in different banks, plus its 16 x 8 scale bytes.  The NW waves take the pairs of K in turn, NB pairs per wave
// in flight.  K must be a multiple of 256.
//  * 8 / 32 rows (us; tiled GEMM in brackets): 4096^2 4.7 / 6.5 (14.1 / 15.3), 8192^2 11.2 / 14.5 (17.8 / 19.9),
//    4096 x 14336 9.8 / 14.3 (18.9 / 21.0), 14336 x 4096 10.8 / 14.7 (16.1 / 18.6), 16384^2 34.3 / 41.2 (41.0 / 44.4).
//  * Two earlier forms of this kernel loaded the weights per lane in operand order (16 rows x 64 bytes per wave
//    instruction), the activations through a shared LDS stage or per lane: 13.0-13.8 us on 8192^2 and 42.7-43.0 on
//    16384^2 at 8 rows whatever else was varied (rows per wave, steps in flight, 8 or 16 waves, K order rotated per
//    workgroup); the same code reading 1 KiB contiguous per instruction (timing only) took 9.5-11.1 and 28-35 us.
//    The access pattern was the bound; copies by whole lines recover most of it without a second weight layout.
template <int RT, int XT, int NW, int NB>
__global__ __launch_bounds__(NW * 64) void mx4_ring_kernel(Mx4SkArgs a) {
    constexpr int TILE = 2048 + 256;
    constexpr int NT = RT + XT;
    constexpr int OPS = 3 * NT;  // copy instructions per pair
    static_assert((NB - 1) * OPS < 64, "outstanding copies must fit the vmcnt counter");
    extern __shared__ __align__(16) unsigned char ring[];  // [NW][NB][NT][TILE]
    __shared__ f32x4s red[NW][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16 * RT;
    unsigned char* mine = ring + (size_t)wave * NB * NT * TILE;

    // copy plan of a pair: per tile two code instructions (rows 8j + lane / 8, slot lane % 8 <- piece slot ^ (row >> 1))
    // and one for the scale bytes (row (lane / 2) % 16, dword lane % 2; the upper half-wave writes a duplicate)
    const uint8_t* csrc[NT][2];
    const uint8_t* ssrc[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const bool is_w = i < RT;
        auto row_ptr = [&](int row, bool scale) -> const uint8_t* {
            if (is_w) {
                int n = n0 + 16 * i + row;
                if (n > a.N - 1) n = a.N - 1;  // rows past the end repeat the last one; never stored
                return scale ? a.scales + (int64_t)n * a.msn : a.w + (int64_t)n * a.wsn;
            }
            int m = 16 * (i - RT) + row;
            if (m > a.M - 1) m = a.M - 1;
            return scale ? a.sx + (int64_t)m * a.sxm : a.x + (int64_t)m * a.xsm;
        };
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * j + (lane >> 3), slot = lane & 7;
            csrc[i][j] = row_ptr(row, false) + ((slot ^ (row >> 1)) & 7) * 16;
        }
        ssrc[i] = row_ptr((lane >> 1) & 15, true) + (lane & 1) * 4;
    }
    auto issue = [&](int p, int slot) __attribute__((always_inline)) {
        unsigned char* base = mine + slot * (NT * TILE);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(csrc[i][j] + (int64_t)p * 128),
                                                 (__attribute__((address_space(3))) void*)(base + i * TILE + j * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ssrc[i] + (int64_t)p * 8),
                                             (__attribute__((address_space(3))) void*)(base + i * TILE + 2048), 4, 0, 0);
        }
    };
    f32x4s acc[RT][XT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) acc[t][xt] = f32x4s{0.0f, 0.0f, 0.0f, 0.0f};
    const int code_off = r16 * 128, swz = r16 >> 1, scale_off = 2048 + r16 * 8;
    auto multiply = [&](int slot) __attribute__((always_inline)) {
        const unsigned char* base = mine + slot * (NT * TILE);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int piece = (((4 * u + kq) ^ swz) & 7) * 16;
#pragma unroll
            for (int xt = 0; xt < XT; ++xt) {
                const unsigned char* xb = base + (RT + xt) * TILE;
                const u32x4s xv = *(const u32x4s*)(xb + code_off + piece);
                const int ex = (int)((*(const uint32_t*)(xb + scale_off + 4 * u) >> (8 * kq)) & 0xffu);
                const i32x8s b8 = {(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3], 0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const unsigned char* wb = base + t * TILE;
                    const u32x4s wv = *(const u32x4s*)(wb + code_off + piece);
                    const int ew = (int)((*(const uint32_t*)(wb + scale_off + 4 * u) >> (8 * kq)) & 0xffu);
                    const i32x8s a8 = {(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3], 0, 0, 0, 0};
                    acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 4, 4, 0, ew, 0, ex);
                }
            }
        }
    };
    const int pairs = a.K / 256;
    const int iters = (pairs + NW - 1) / NW;
    // a wave whose turn lies past the end copies the last pair again (same count of copies for everybody) and skips the multiply
    auto pair_of = [&](int it) { const int p = it * NW + wave; return p < pairs ? p : pairs - 1; };
#pragma unroll
    for (int b = 0; b < NB - 1; ++b)
        if (b < iters) issue(pair_of(b), b);
    int slot = 0, islot = NB - 1;
    for (int it = 0; it < iters; ++it) {
        const int later = iters - 1 - it;  // pairs issued after this one
        if (later >= NB - 1) {
            issue(pair_of(it + NB - 1), islot);
            islot = islot == NB - 1 ? 0 : islot + 1;
            wait_vmcnt_sk<(NB - 1) * OPS>();
        } else {
            // the ring drains: `later` pairs are still allowed in flight
            bool done = false;
#pragma unroll
            for (int k = NB - 2; k >= 1; --k) {
                if (!done && later == k) {
                    if (k == 1) wait_vmcnt_sk<1 * OPS < 64 ? 1 * OPS : 0>();
                    else if (k == 2) wait_vmcnt_sk<2 * OPS < 64 ? 2 * OPS : 0>();
                    else if (k == 3) wait_vmcnt_sk<3 * OPS < 64 ? 3 * OPS : 0>();
                    else wait_vmcnt_sk<0>();
                    done = true;
                }
            }
            if (!done) wait_vmcnt_sk<0>();
        }
        asm volatile("" ::: "memory");
        if (it * NW + wave < pairs) multiply(slot);
        slot = slot == NB - 1 ? 0 : slot + 1;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);  // the copies of the next turn go to the slot these reads came from
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
            for (int w = 0; w < NW; ++w) D += red[w][lane];
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

template <int RT, int XT, int NW, int NB>
int launch_ring4(const Mx4SkArgs& a, hipStream_t stream) {
    const size_t smem = (size_t)NW * NB * (RT + XT) * (2048 + 256);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = mx4_ring_kernel<RT, XT, NW, NB>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "mx4_ring: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(ceil_div(ceil_div(a.N, 16), RT)), dim3(NW * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "mx4_ring launch");
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
        // rows of tiles per wave so that about one workgroup per CU comes out; fewer, deeper waves where a wave has
        // 4 weight tiles to an activation tile (16384^2 at 8 rows: 34.3 us with 4 tiles x 4 waves x 3 pairs in flight,
        // 38.4 with 2 x 8 x 2, 35.2 with 1 x 8 x 4; 8192^2: 15.5 / 11.2 / 12.6; 4096^2: 8.9 / 6.1 / 4.7)
        const int tiles = ceil_div(p.N, 16);
        if (p.M <= 16) {
            if (tiles >= 880) return launch_ring4<4, 1, 4, 3>(a, stream);
            if (tiles >= 440) return launch_ring4<2, 1, 8, 2>(a, stream);
            return launch_ring4<1, 1, 8, 4>(a, stream);
        }
        if (tiles >= 880) return launch_ring4<4, 2, 4, 2>(a, stream);
        if (tiles >= 440) return launch_ring4<2, 2, 4, 4>(a, stream);
        return launch_ring4<1, 2, 8, 2>(a, stream);
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
