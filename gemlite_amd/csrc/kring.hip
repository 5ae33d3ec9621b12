// Skinny matmul (3..32 rows) for layers whose two operands are both narrow and K-contiguous:
//
//   MXFP4 x MXFP4   e2m1 nibble pairs, one e8m0 scale per 32 values on either side
//                   (v_mfma_scale_f32_16x16x128_f8f6f4, both block scales applied by the instruction)
//   fp8 x fp8       e4m3 bytes, per-token x per-channel scales in the epilogue (the same instruction, unit scales)
//   int8 x int8     exact int32 sums (v_mfma_i32_16x16x64_i8), scaled in the epilogue or stored as int32
//   fp8 x MXFP8      e4m3 bytes on both sides, e8m0 block scales on the weights and, by channel_scale_mode, either the
//                   same on the activations or one fp32 scale per token in the epilogue
//   fp8 x MXFP4      the mixed form of the instruction (A e2m1, B e4m3): 256 K-values a turn, the activations of a
//                   turn travelling as two tiles (4096^2 at 8 rows 5.2 us against 16.2 tiled, 16384^2 35.0 against 54.9)
//   16-bit x MXFP8 / MXFP4 (weight-only layers)
//                   the last two modes on activations written as a sum of e4m3 terms: a bf16 value is 8 significant
//                   bits = two e4m3 values of 4 (an fp16 value three), each term with its own e8m0 scale per 32-block, 16
//                   apart.  A small launch writes the terms as rows of their own (row T j + t of a 16-row tile = term
//                   t of the tile's j-th activation row), the matmul multiplies them like any fp8 rows - the products
//                   of the scaled MFMA are exact, so the sum of a row's terms is the product with the 16-bit value -
//                   and the epilogue adds the T accumulator columns of a row.  No weight is converted.  What the terms
//                   cannot hold is smaller than 2^-20 (fp16: 2^-24) of the block's largest magnitude.
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

enum { R_MX44 = 0, R_FP8 = 1, R_INT8 = 2, R_MX88 = 3, R_MX84 = 4 };

struct KRingArgs {
    const uint8_t* x;         // [M, bytes of K]
    const uint8_t* w;         // [N, bytes of K]
    const uint8_t* bsx;       // block-scaled activations: [ceil32(M), K/32] e8m0
    const uint8_t* bsw;       // block-scaled weights: [N, K/32] e8m0
    const void* scales;       // fp8 / int8: per-channel scales [N] (channel_scale_mode bit 0)
    const void* scales_x;     // per-token scales [M] (bit 1)
    void* out;
    int M, N, turns;          // turns = K / (K-values per turn)
    int fold, Mo;             // fold T > 1: activation row T j + t of a tile is term t of output row (16 / T) tile + j; Mo output rows
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

// What a turn of K is in each mode.  A tile is always 16 rows x 128 bytes; the fp8 activations under MXFP4 weights
// are 256 bytes per row and turn and travel as two tiles.
template <int MODE>
struct RingShape {
    static constexpr bool WBS = MODE == R_MX44 || MODE == R_MX88 || MODE == R_MX84;  // weights carry block scales
    static constexpr int XH = MODE == R_MX84 ? 2 : 1;                                // activation tiles per 16 rows and turn
    static constexpr int KT = (MODE == R_MX44 || MODE == R_MX84) ? 256 : 128;        // K-values per turn
    static constexpr int SB = KT / 32;                                               // scale bytes per row and turn
};

// XBS: the activations carry block scales too (always with MXFP4 activations; MXFP8 activations by channel_scale_mode)
template <int MODE, bool XBS, int RT, int XT, int NW, int NB>
__global__ __launch_bounds__(NW * 64) void kring_kernel(KRingArgs a) {
    using SH = RingShape<MODE>;
    constexpr bool WBS = SH::WBS;
    constexpr int XH = SH::XH, SB = SH::SB;
    constexpr int TILE = 2048 + (WBS ? 256 : 0);
    constexpr int NT = RT + XT * XH;
    constexpr int OPS = RT * (2 + (WBS ? 1 : 0)) + XT * XH * 2 + (XBS ? XT : 0);  // copy instructions per turn
    typedef typename std::conditional<MODE == R_INT8, i32x4r, f32x4r>::type acc_t;
    static_assert((NB - 1) * OPS < 64, "outstanding copies must fit the vmcnt counter");
    static_assert(!XBS || WBS, "block-scaled activations come with block-scaled weights");
    extern __shared__ __align__(16) unsigned char ring[];  // [NW][NB][NT][TILE]
    __shared__ acc_t red[NW][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16 * RT;
    unsigned char* mine = ring + (size_t)wave * NB * NT * TILE;

    // copy plan of a turn: per tile two code instructions (rows 8j + lane / 8, slot lane % 8 <- piece slot ^ (row >> 1))
    // and, with block scales, one for the tile's scale bytes: 8 per row (row (lane / 2) % 16, dword lane % 2) or 4
    // (row lane % 16); the rest of the wave writes duplicates behind them
    const uint8_t* csrc[NT][2];
    const uint8_t* ssrc[WBS ? NT : 1];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const bool is_w = i < RT;
        const int xt = is_w ? 0 : (i - RT) / XH, half = is_w ? 0 : (i - RT) % XH;
        auto row_ptr = [&](int row, bool scale) -> const uint8_t* {
            if (is_w) {
                int n = n0 + 16 * i + row;
                if (n > a.N - 1) n = a.N - 1;  // rows past the end repeat the last one; never stored
                return scale ? a.bsw + (int64_t)n * a.bswn : a.w + (int64_t)n * a.wsn;
            }
            int m = 16 * xt + row;
            if (m > a.M - 1) m = a.M - 1;
            return scale ? a.bsx + (int64_t)m * a.bsxm : a.x + (int64_t)m * a.xsm + half * 128;
        };
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * j + (lane >> 3), slot = lane & 7;
            csrc[i][j] = row_ptr(row, false) + ((slot ^ (row >> 1)) & 7) * 16;
        }
        if constexpr (WBS) {
            if (is_w || (XBS && half == 0))
                ssrc[i] = SB == 8 ? row_ptr((lane >> 1) & 15, true) + (lane & 1) * 4 : row_ptr(lane & 15, true);
            else
                ssrc[i] = nullptr;
        }
    }
    auto issue = [&](int p, int slot) __attribute__((always_inline)) {
        unsigned char* base = mine + slot * (NT * TILE);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const int adv = i < RT ? 128 : 128 * XH;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(csrc[i][j] + (int64_t)p * adv),
                                                 (__attribute__((address_space(3))) void*)(base + i * TILE + j * 1024), 16, 0, 0);
            if constexpr (WBS) {
                if (i < RT || (XBS && (i - RT) % XH == 0))
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ssrc[i] + (int64_t)p * SB),
                                                     (__attribute__((address_space(3))) void*)(base + i * TILE + 2048), 4, 0, 0);
            }
        }
    };
    acc_t acc[RT][XT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) acc[t][xt] = acc_t{0, 0, 0, 0};
    const int code_off = r16 * 128, swz = r16 >> 1, scale_off = 2048 + r16 * SB;
    auto slot16 = [&](const unsigned char* tile, int piece) __attribute__((always_inline)) {
        return *(const u32x4r*)(tile + code_off + ((piece ^ swz) & 7) * 16);
    };
    // the lane's 32 bytes of a row as an 8-register fp8 operand.  Registers 0-3 of the four lane groups together are
    // K-values 0..63 of the instruction, registers 4-7 K-values 64..127 (slots kq and 4 + kq), while the scale byte a
    // lane group hands in applies to 32-block kq.
    auto slot32 = [&](const unsigned char* tile) __attribute__((always_inline)) {
        const u32x4r lo = slot16(tile, kq), hi = slot16(tile, 4 + kq);
        return i32x8r{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    };
    // e8m0 byte of the lane's 32-block: byte kq of dword u of the row's scale bytes
    auto scale_byte = [&](const unsigned char* tile, int u) __attribute__((always_inline)) {
        return (int)((*(const uint32_t*)(tile + scale_off + 4 * u) >> (8 * kq)) & 0xffu);
    };
    auto multiply = [&](int slot) __attribute__((always_inline)) {
        const unsigned char* base = mine + slot * (NT * TILE);
        if constexpr (MODE == R_FP8 || MODE == R_MX88) {
            // a turn is one MFMA of 128 bytes of K
#pragma unroll
            for (int xt = 0; xt < XT; ++xt) {
                const unsigned char* xb = base + (RT + xt) * TILE;
                const i32x8r b8 = slot32(xb);
                int ex = 127;
                if constexpr (XBS) ex = scale_byte(xb, 0);
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const unsigned char* wb = base + t * TILE;
                    int ew = 127;
                    if constexpr (WBS) ew = scale_byte(wb, 0);
                    acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(slot32(wb), b8, acc[t][xt], 0, 0, 0, ew, 0, ex);
                }
            }
        } else {
            // two MFMAs a turn (MXFP4 weights: 128 K-values each; int8: 64): the lane's 16 bytes are slot 4 u + kq
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int xt = 0; xt < XT; ++xt) {
                    const unsigned char* xb = base + (RT + xt * XH) * TILE;  // (first) tile of these 16 rows: holds their scales
                    int ex = 127;
                    if constexpr (XBS) ex = scale_byte(xb, u);
                    u32x4r xv;
                    i32x8r b8;
                    if constexpr (MODE == R_MX84) {
                        b8 = slot32(xb + u * TILE);  // fp8 activations: half u of the turn is a tile of its own
                    } else {
                        xv = slot16(xb, 4 * u + kq);
                        b8 = i32x8r{(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3], 0, 0, 0, 0};
                    }
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        const unsigned char* wb = base + t * TILE;
                        const u32x4r wv = slot16(wb, 4 * u + kq);
                        if constexpr (MODE == R_INT8) {
                            acc[t][xt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(i32x4r{(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3]},
                                                                               i32x4r{(int)xv[0], (int)xv[1], (int)xv[2], (int)xv[3]},
                                                                               acc[t][xt], 0, 0, 0);
                        } else {
                            const int ew = scale_byte(wb, u);
                            const i32x8r a8 = {(int)wv[0], (int)wv[1], (int)wv[2], (int)wv[3], 0, 0, 0, 0};
                            // operand formats: 4 = e2m1, 0 = e4m3
                            if constexpr (MODE == R_MX84)
                                acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 4, 0, 0, ew, 0, ex);
                            else
                                acc[t][xt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[t][xt], 4, 4, 0, ew, 0, ex);
                        }
                    }
                }
            }
        }
    };
    const int turns = a.turns;
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
    const bool col_scale = a.csm <= GLA_CSM_BOTH && (a.csm & 1), row_scale = a.csm <= GLA_CSM_BOTH && (a.csm & 2);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
            if (t || xt) __syncthreads();
            red[wave][lane] = acc[t][xt];
            __syncthreads();
            if (wave != 0) continue;
            acc_t D = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < NW; ++w) D += red[w][lane];
            int m = 16 * xt + r16;
            if constexpr (MODE == R_MX88 || MODE == R_MX84) {
                if (a.fold > 1) {
                    // the terms of output row j are the accumulator columns T j .. T j + T - 1 of the same lane group
                    const int T = a.fold, per_tile = 16 / T;
                    const int src = 16 * kq + (r16 < per_tile ? T * r16 : 0);
                    acc_t S = {0, 0, 0, 0};
                    for (int t = 0; t < T; ++t)
#pragma unroll
                        for (int e = 0; e < 4; ++e) S[e] += __shfl(D[e], src + t, 64);
                    D = S;
                    m = r16 < per_tile ? per_tile * xt + r16 : a.Mo;
                }
            }
            if (m >= a.Mo) continue;
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
                if (row_scale || col_scale) v *= sa * (col_scale ? load_as_float(a.scales, a.meta_dt, n) : 1.0f);
                if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + load_as_float(a.bias, a.bias_dt, n);
                store_from_float(a.out, a.out_dt, o, v);
            }
        }
    }
}

// 16-bit activation rows as sums of T e4m3 terms with e8m0 block scales, in the row order the fold of the epilogue
// expects.  One thread per (tile, row slot j, 32-block): term t = RNE_e4m3(r / s_t), r <- r - term s_t (exact), s_t =
// 2^(floor(log2 amax) - 7 - 4 t), so the block's largest value lands in [128, 256).  Slots past M and the rows a tile
// cannot use (16 - T (16 / T)) are written as zeros with the identity scale: the matmul reads all of them.
template <bool BF16, int T>
__global__ __launch_bounds__(256) void split_e4m3_kernel(const uint16_t* __restrict__ x, int64_t xsm, int M, int K, int tiles,
                                                         uint8_t* __restrict__ y, uint8_t* __restrict__ sy) {
    constexpr int PER = 16 / T, SLOTS = PER + (16 % T ? 1 : 0);
    const int groups = K / 32;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)tiles * SLOTS * groups) return;
    const int g = (int)(id % groups), j = (int)((id / groups) % SLOTS), tile = (int)(id / groups / SLOTS);
    const int m = tile * PER + j;
    uint8_t* yrow = y + ((int64_t)tile * 16 + T * j) * K + g * 32;
    uint8_t* srow = sy + ((int64_t)tile * 16 + T * j) * groups + g;
    if (j >= PER || m >= M) {
        const int rows = j >= PER ? 16 % T : T;
        for (int t = 0; t < rows; ++t) {
            *(uint4*)(yrow + (int64_t)t * K) = make_uint4(0, 0, 0, 0);
            *(uint4*)(yrow + (int64_t)t * K + 16) = make_uint4(0, 0, 0, 0);
            srow[(int64_t)t * groups] = 127;
        }
        return;
    }
    float r[32];
    const uint4* src = (const uint4*)(x + (int64_t)m * xsm + g * 32);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint4 v = src[i];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if constexpr (BF16) {
                r[8 * i + 2 * k] = __builtin_bit_cast(float, w[k] << 16);
                r[8 * i + 2 * k + 1] = __builtin_bit_cast(float, w[k] & 0xffff0000u);
            } else {
                r[8 * i + 2 * k] = half_bits_to_float((uint16_t)(w[k] & 0xffffu));
                r[8 * i + 2 * k + 1] = half_bits_to_float((uint16_t)(w[k] >> 16));
            }
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(r[i]));
    // floor(log2 amax) from the exponent field (a block of zeros, or of values below 2^-126, keeps the smallest scale)
    const int e = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xffu) - 127;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        int se = e + 120 - 4 * t;  // biased exponent of s_t
        se = se < 0 ? 0 : (se > 254 ? 254 : se);
        const float s = __builtin_ldexpf(1.0f, se - 127);
        uint32_t out[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float q[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) q[k] = __builtin_ldexpf(r[4 * i + k], 127 - se);  // below 256 in magnitude
            const uint32_t w = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false) & 0xffffu;
            const uint32_t w2 = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], 0, false) & 0xffffu;
            out[i] = w | (w2 << 16);
            if (t + 1 < T) {
                r[4 * i + 0] = __builtin_fmaf(-__builtin_amdgcn_cvt_f32_fp8((int)out[i], 0), s, r[4 * i + 0]);
                r[4 * i + 1] = __builtin_fmaf(-__builtin_amdgcn_cvt_f32_fp8((int)out[i], 1), s, r[4 * i + 1]);
                r[4 * i + 2] = __builtin_fmaf(-__builtin_amdgcn_cvt_f32_fp8((int)out[i], 2), s, r[4 * i + 2]);
                r[4 * i + 3] = __builtin_fmaf(-__builtin_amdgcn_cvt_f32_fp8((int)out[i], 3), s, r[4 * i + 3]);
            }
        }
        *(uint4*)(yrow + (int64_t)t * K) = make_uint4(out[0], out[1], out[2], out[3]);
        *(uint4*)(yrow + (int64_t)t * K + 16) = make_uint4(out[4], out[5], out[6], out[7]);
        srow[(int64_t)t * groups] = (uint8_t)se;
    }
}

template <int MODE, bool XBS, int RT, int XT, int NW, int NB>
int launch_ring(const KRingArgs& a, hipStream_t stream) {
    using SH = RingShape<MODE>;
    const size_t smem = (size_t)NW * NB * (RT + XT * SH::XH) * (2048 + (SH::WBS ? 256 : 0));
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = kring_kernel<MODE, XBS, RT, XT, NW, NB>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "kring: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(ceil_div(ceil_div(a.N, 16), RT)), dim3(NW * 64), smem, stream, a);
    return check_hip(hipGetLastError(), "kring launch");
}

template <int MODE, bool XBS>
int launch_mode_ring(const KRingArgs& a, hipStream_t stream) {
    // rows of tiles per wave so that about one workgroup per CU comes out; fewer, deeper waves where a wave has
    // 4 weight tiles to an activation tile (MXFP4, 16384^2 at 8 rows: 34.3 us with 4 tiles x 4 waves x 3 turns in
    // flight, 38.4 with 2 x 8 x 2, 35.2 with 1 x 8 x 4; 8192^2: 15.5 / 11.2 / 12.6; 4096^2: 8.9 / 6.1 / 4.7)
    const int tiles = ceil_div(a.N, 16);
    if constexpr (MODE == R_MX44) {
        if (a.M <= 16) {
            if (tiles >= 880) return launch_ring<MODE, XBS, 4, 1, 4, 3>(a, stream);
            if (tiles >= 440) return launch_ring<MODE, XBS, 2, 1, 8, 2>(a, stream);
            return launch_ring<MODE, XBS, 1, 1, 8, 4>(a, stream);
        }
        if (tiles >= 880) return launch_ring<MODE, XBS, 4, 2, 4, 2>(a, stream);
        if (tiles >= 440) return launch_ring<MODE, XBS, 2, 2, 4, 4>(a, stream);
        return launch_ring<MODE, XBS, 1, 2, 8, 2>(a, stream);
    } else if constexpr (MODE == R_MX84) {
        // 16 activation rows are two tiles a turn here, 32 rows four: shallower rings
        if (a.M <= 16) {
            if (tiles >= 880) return launch_ring<MODE, XBS, 4, 1, 4, 2>(a, stream);
            if (tiles >= 440) return launch_ring<MODE, XBS, 2, 1, 8, 2>(a, stream);
            return launch_ring<MODE, XBS, 1, 1, 8, 2>(a, stream);
        }
        // (16-bit activations as e4m3 terms, 16 rows of bf16 = 32 fp8 rows, 16384^2: 58 us with 2 weight tiles per wave, 51 with 4)
        if (tiles >= 880) return launch_ring<MODE, XBS, 4, 2, 4, 2>(a, stream);
        if (tiles >= 440) return launch_ring<MODE, XBS, 2, 2, 4, 2>(a, stream);
        return launch_ring<MODE, XBS, 1, 2, 4, 3>(a, stream);
    } else {
        // 8-bit operands: an activation tile is as many bytes as a weight tile, and one tile per wave with many waves
        // does best (fp8 at 8 rows, 8192^2: 17.3 us with 1 tile x 16 waves x 2 turns, 17.6 with 1 x 8 x 4, 21.1 with
        // 2 x 8 x 2; 16384^2: 58.6 / 60.0 / 66.1) unless K is short and N long (14336 x 4096: 21.1 / 21.8 against 18.8
        // with 4 x 4 x 3)
        constexpr int D1 = RingShape<MODE>::WBS ? 3 : 4;  // ring depth that fits with one tile each and 8 waves
        if (a.M <= 16) {
            if (tiles >= 880 && a.turns < 64) return launch_ring<MODE, XBS, 4, 1, 4, 3>(a, stream);
            if (tiles >= 440) return launch_ring<MODE, XBS, 1, 1, 16, 2>(a, stream);
            return launch_ring<MODE, XBS, 1, 1, 8, D1>(a, stream);
        }
        if (tiles >= 440) return launch_ring<MODE, XBS, 2, 2, 8, 2>(a, stream);
        return launch_ring<MODE, XBS, 1, 2, 8, 2>(a, stream);
    }
}

int ring_mode(const gla_matmul_args& p) {
    if (p.input_dtype == GLA_DT_MXFP4) return R_MX44;
    if (p.input_dtype == GLA_DT_FP8 && p.w_dtype == GLA_DT_FP8) return R_FP8;
    if (p.input_dtype == GLA_DT_INT8 && p.w_dtype == GLA_DT_INT8) return R_INT8;
    if (p.input_dtype == GLA_DT_MXFP8) return (p.W_nbits == 4 && p.elements_per_sample == 2) ? R_MX84 : R_MX88;
    return -1;
}

// Weight-only MX layers: terms per 16-bit activation value (0: not such a call)
int split_terms(const gla_matmul_args& p) {
    return p.input_dtype == GLA_DT_MXBF16 ? 2 : (p.input_dtype == GLA_DT_MXFP16 ? 3 : 0);
}

struct SplitPlan {
    int T, tiles;         // terms; 16-row tiles of fp8 rows
    int64_t y_off, s_off, total;   // workspace offsets of the terms and their scale bytes, bytes in all
};

SplitPlan split_plan(const gla_matmul_args& p) {
    SplitPlan s;
    s.T = split_terms(p);
    s.tiles = ceil_div(p.M, 16 / s.T);
    s.y_off = kWsPrivateBytes;
    s.s_off = s.y_off + (int64_t)s.tiles * 16 * p.K;
    s.total = s.s_off + (int64_t)s.tiles * 16 * (p.K / 32);
    return s;
}

bool split_eligible(const gla_matmul_args& p) {
    const int T = split_terms(p);
    if (T == 0 || p.M < 1 || p.M > 2 * (16 / T) || p.x_quant_from != 0) return false;
    if (p.group_size != 32 || p.channel_scale_mode != GLA_CSM_NONE || p.scales == nullptr) return false;
    const bool w4 = p.W_nbits == 4 && p.elements_per_sample == 2;
    const bool w8 = p.W_nbits == 8 && p.elements_per_sample == 1;
    if (!w4 && !w8) return false;
    if (p.K % (w4 ? 256 : 128) != 0) return false;
    if (p.meta_stride_g != 1 || p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3)) return false;
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.x_stride_m % 8 != 0 || p.w_stride_n % 16 != 0 || ((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    switch (p.output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_MXFP16: case GLA_DT_MXBF16: return true;
        default: return false;
    }
}

int launch_split(const gla_matmul_args& p, hipStream_t stream) {
    const SplitPlan sp = split_plan(p);
    if (p.workspace == nullptr || (int64_t)p.workspace_bytes < sp.total) {
        set_error("kring: workspace of %lld bytes required (the activations' e4m3 terms go there), %llu given", (long long)sp.total,
                  (unsigned long long)p.workspace_bytes);
        return GLA_ERR_WORKSPACE_TOO_SMALL;
    }
    uint8_t* y = (uint8_t*)p.workspace + sp.y_off;
    uint8_t* sy = (uint8_t*)p.workspace + sp.s_off;
    const int slots = sp.T == 2 ? 8 : 6;
    const int64_t items = (int64_t)sp.tiles * slots * (p.K / 32);
    const dim3 grid((unsigned)((items + 255) / 256));
    if (sp.T == 2)
        hipLaunchKernelGGL((split_e4m3_kernel<true, 2>), grid, dim3(256), 0, stream, (const uint16_t*)p.x, p.x_stride_m, p.M, p.K, sp.tiles, y, sy);
    else
        hipLaunchKernelGGL((split_e4m3_kernel<false, 3>), grid, dim3(256), 0, stream, (const uint16_t*)p.x, p.x_stride_m, p.M, p.K, sp.tiles, y, sy);
    int rc = check_hip(hipGetLastError(), "kring: activation split launch");
    if (rc != GLA_OK) return rc;
    const bool w4 = p.elements_per_sample == 2;
    KRingArgs a;
    a.x = y; a.w = (const uint8_t*)p.w; a.out = p.out;
    a.M = sp.tiles * 16; a.N = p.N; a.Mo = p.M; a.fold = sp.T;
    a.turns = p.K / (w4 ? 256 : 128);
    a.xsm = p.K; a.wsn = p.w_stride_n; a.osm = p.out_stride_m;
    a.bsx = sy; a.bsw = (const uint8_t*)p.scales;
    a.bsxm = p.K / 32; a.bswn = p.meta_stride_n;
    a.scales = nullptr; a.scales_x = nullptr; a.sxm = 0;
    a.csm = GLA_CSM_MX; a.meta_dt = GLA_DT_UINT8; a.sx_dt = GLA_DT_UINT8;
    a.out_dt = p.output_dtype == GLA_DT_MXFP16 ? GLA_DT_FP16 : (p.output_dtype == GLA_DT_MXBF16 ? GLA_DT_BF16 : p.output_dtype);
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    return w4 ? launch_mode_ring<R_MX84, true>(a, stream) : launch_mode_ring<R_MX88, true>(a, stream);
}

}  // namespace

int64_t kring_workspace_bytes(const gla_matmul_args& p) { return split_terms(p) ? split_plan(p).total : 0; }

bool kring_eligible(const gla_matmul_args& p) {
    if (split_terms(p)) return split_eligible(p);
    const int mode = ring_mode(p);
    if (mode < 0 || p.x_quant_from != 0 || p.M < 1 || p.M > 32) return false;
    if (p.x_stride_k != 1 || p.w_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0 || ((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    const bool float_out = p.output_dtype == GLA_DT_FP32 || p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16;
    if (mode == R_MX44 || mode == R_MX88 || mode == R_MX84) {
        if (p.group_size != 32 || p.scales == nullptr || p.scales_x == nullptr || !float_out) return false;
        if (p.meta_stride_g != 1 || p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3)) return false;
        const bool xbs = p.channel_scale_mode == GLA_CSM_MX;
        if (xbs && (p.sx_dtype != GLA_DT_UINT8 || p.sx_stride_g != 1 || p.sx_stride_m % 4 != 0 || ((uintptr_t)p.scales_x & 3))) return false;
        if (mode == R_MX44) {
            if (!xbs || !(p.W_nbits == 4 && p.elements_per_sample == 2)) return false;
            return p.K % 256 == 0;  // whole turns of 128 bytes
        }
        // fp8 activations with block scales or one scale per token
        if (!xbs && p.channel_scale_mode != GLA_CSM_ACTIVATION) return false;
        if (mode == R_MX88) return p.W_nbits == 8 && p.elements_per_sample == 1 && p.w_dtype == GLA_DT_FP8 && p.K % 128 == 0;
        return p.K % 256 == 0;
    }
    // fp8 x fp8 and int8 x int8: what the tiled 8-bit GEMM takes, K in whole turns
    if (mode == R_FP8 && p.acc_dtype != GLA_DT_FP32) return false;
    if (mode == R_INT8 && p.acc_dtype != GLA_DT_INT32) return false;
    if (p.elements_per_sample != 1 || p.W_nbits != 8 || p.W_group_mode != GLA_WGM_NONE) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.K % 128 != 0) return false;
    if (p.output_dtype == GLA_DT_INT32) return mode == R_INT8 && p.channel_scale_mode == GLA_CSM_NONE;
    if (!float_out) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int launch_kring(const gla_matmul_args& p, hipStream_t stream) {
    if (!kring_eligible(p)) {
        set_error("kring: MXFP4 x MXFP4, fp8 x fp8, int8 x int8 or fp8 x MXFP8 / MXFP4 operands, K-contiguous with 16-byte "
                  "aligned rows, up to 32 rows (bf16 / fp16 on MX weights: 16 / 10), K a multiple of 256 (MXFP4 weights) or 128");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    if (split_terms(p)) return launch_split(p, stream);
    const int mode = ring_mode(p);
    const bool mx = mode == R_MX44 || mode == R_MX88 || mode == R_MX84;
    const bool xbs = mx && p.channel_scale_mode == GLA_CSM_MX;
    KRingArgs a;
    a.x = (const uint8_t*)p.x; a.w = (const uint8_t*)p.w; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Mo = p.M; a.fold = 1;
    a.turns = p.K / ((mode == R_MX44 || mode == R_MX84) ? 256 : 128);
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m;
    a.bsx = xbs ? (const uint8_t*)p.scales_x : nullptr; a.bsw = mx ? (const uint8_t*)p.scales : nullptr;
    a.bsxm = p.sx_stride_m; a.bswn = p.meta_stride_n;
    a.scales = p.scales; a.scales_x = p.scales_x; a.sxm = p.sx_stride_m;
    a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype; a.out_dt = p.output_dtype;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    switch (mode) {
        case R_MX44: return launch_mode_ring<R_MX44, true>(a, stream);
        case R_FP8: return launch_mode_ring<R_FP8, false>(a, stream);
        case R_INT8: return launch_mode_ring<R_INT8, false>(a, stream);
        case R_MX88: return xbs ? launch_mode_ring<R_MX88, true>(a, stream) : launch_mode_ring<R_MX88, false>(a, stream);
        default: return xbs ? launch_mode_ring<R_MX84, true>(a, stream) : launch_mode_ring<R_MX84, false>(a, stream);
    }
}

}  // namespace gla
