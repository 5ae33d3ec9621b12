// MFMA GEMM for fp16/bf16 activations x unpacked 8-bit weights kept as the [K, N] view of an [N, K]
// byte array (K contiguous): int8, uint8 or fp8-e4m3 codes with one scale per output channel.
// The prefill / mid-batch path (more than 16 rows) of weight-only A16W8 layers whose weights are
// not packed into 32-bit words; up to 16 rows the streaming kernels of gemv_kmajor.hip run.
// Also, from 3 rows up, weight-only MX layers: MXFP8 bytes or MXFP4 nibble pairs with one e8m0 scale
// per 32 values, applied by the conversion instruction (reference: gemlite/helper.py:384-420,
// gemlite/triton_kernels/gemm_kernels.py:509-737 with 16-bit activations).
//
// Takes the place of the reference's GEMM and split-K GEMM for one element per sample (reference:
// gemlite/triton_kernels/gemm_kernels.py:285-496, gemlite/triton_kernels/gemm_splitK_kernels.py:300-523;
// the processor that builds such layers: gemlite/helper.py:89-171).
//
//  * Workgroup tile BM x 256 with BM = 64, 128 or 256, K step 64; four wave columns of 64 and
//    two wave rows of BM/2 (one wave row of 64 at BM = 64), v_mfma_f32_32x32x16_{f16,bf16} tiles.
//  * Both operand tiles of a stage are copied global -> LDS by the load unit (global_load_lds) into
//    a ring of 3 or 4 stages, all in flight.  Activation rows are dense 128-byte rows with 16-byte
//    chunks XOR-swizzled by (row >> 1) & 7; weight rows are dense 64-byte rows swizzled by
//    (row >> 2) & 3.
//  * A lane's 8 weight bytes of a K-step become the four registers of a 16-bit MFMA operand in
//    registers, exactly (|code| <= 255 fits fp16 and bf16; fp8-e4m3 is a subset of both).  The
//    per-channel scale commutes with the K sum and is applied in the epilogue, whether the layer
//    asked for it before (W_group_mode 2) or after (channel_scale_mode 1) the sum.
//  * The weights are the row operand of the MFMA: an accumulator is the transposed output tile and
//    a lane stores four adjacent output columns of one row at once.
//  * The loop is software-pipelined as in gemm_wn.hip: LDS reads and conversion of K-step s+1 run
//    under the MFMAs of K-step s, and the barrier that publishes stage k+1 stands before the last
//    K-step of stage k.
//  * Few output tiles (small M): K is split over gridDim.y, fp32 partials go to the workspace and a
//    second kernel on the same stream sums them in order (deterministic).
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

// This file is compiled twice: as it is, and from gemm_kbytes_bias.hip with GLA_KB_BIAS set, which gives the same
// kernels with the bias added in the epilogue under other entry-point names.  A layer without a bias runs the
// epilogue without the extra loads, rounding and registers (a run-time test inside one kernel cost such layers 4-6 %),
// and the two halves compile side by side.
#ifndef GLA_KB_BIAS
#define GLA_KB_BIAS 0
#endif

namespace gla {

namespace {

constexpr bool kWithBias = GLA_KB_BIAS != 0;

typedef unsigned int u32x4b __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2b __attribute__((ext_vector_type(2)));
typedef float f32x2b __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2b __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8b __attribute__((ext_vector_type(8)));
typedef _Float16 half8b __attribute__((ext_vector_type(8)));

constexpr int kBKb = 64;     // K per pipeline stage
constexpr int kRowAb = 128;  // LDS row of the activation tile: 64 fp16/bf16 values
constexpr int kRowBb = 64;   // LDS row of the weight tile: 64 bytes
constexpr int kBNb = 256;
constexpr int kWavesNb = 4;
constexpr int64_t kWsReservedB = kWsPrivateBytes;  // the start of the workspace belongs to the GEMV family (common.hpp)
// Weight kinds beyond the element-type ids: micro-scaled weights of weight-only MX layers, fp8-e4m3 bytes or
// e2m1 nibble pairs with one e8m0 scale per 32 values along K.  The block scale is applied by the
// conversion instruction (v_cvt_scalef32_pk_*), so the 16-bit operand is the dequantised weight.
constexpr int kWMX8 = 100, kWMX4 = 101;

struct GemmKbArgs {
    const uint16_t* x;
    const uint8_t* w;
    const void* scales;
    const void* scales_x;
    void* out;
    int M, N, K;
    int64_t xsm, wsn, osm, msn, sxm;
    int col_scale;  // 0: none, 1: scales[n] once, 2: twice (dequantisation scale and channel scale both set)
    int row_scale;  // multiply by scales_x[m]
    int meta_dt, sx_dt, out_dt;
    int tiles_m, tiles_n;
    int S, sps;
    float* partials;
    const uint8_t* bscales;  // micro-scaled weights: e8m0 block scales [N, K/32], K contiguous
    int64_t bsn;             // ... bytes from one row's scales to the next
    const void* bias;        // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

__device__ __forceinline__ void tile_coords_kb(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
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

template <int N>
__device__ __forceinline__ void wait_vmcnt_kb() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// 8 codes (two dwords) -> the four registers of an 8-element 16-bit operand, K order kept
template <int WDT, bool BF16>
__device__ __forceinline__ u32x4b bytes_to_operand(uint32_t d0, uint32_t d1) {
    u32x4b o;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t d = h ? d1 : d0;
        if constexpr (WDT == GLA_DT_FP8) {
            const f32x2b lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)d, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)d, true);
            if constexpr (BF16) {
                o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2b));
                o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2b));
            } else {
                o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo.x, lo.y));
                o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(hi.x, hi.y));
            }
        } else if constexpr (BF16) {
            const uint32_t u = WDT == GLA_DT_INT8 ? d ^ 0x80808080u : d;
            const float off = WDT == GLA_DT_INT8 ? -128.0f : 0.0f;
            const f32x2b lo = {(float)(u & 0xffu) + off, (float)((u >> 8) & 0xffu) + off};
            const f32x2b hi = {(float)((u >> 16) & 0xffu) + off, (float)(u >> 24) + off};
            o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2b));
            o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2b));
        } else {
            // fp16: bytes into the mantissa of 1024.0, two per register, then minus 1024 (+128 for signed codes)
            const uint32_t u = WDT == GLA_DT_INT8 ? d ^ 0x80808080u : d;
            const half2_t off = WDT == GLA_DT_INT8 ? half2_t{(half_t)1152.0f, (half_t)1152.0f} : half2_t{(half_t)1024.0f, (half_t)1024.0f};
            const uint32_t t0 = __builtin_amdgcn_perm(u, u, 0x0c010c00u) | 0x64006400u;
            const uint32_t t1 = __builtin_amdgcn_perm(u, u, 0x0c030c02u) | 0x64006400u;
            o[2 * h] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, t0) - off);
            o[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, t1) - off);
        }
    }
    return o;
}

// micro-scaled weights: 8 codes (two dwords of fp8, one of fp4) times the block scale 2^(e - 127), whose e8m0
// byte sits in the exponent field of `scale` (which is all the conversion instruction reads of it)
template <int WDT, bool BF16>
__device__ __forceinline__ u32x4b mx_to_operand(uint32_t d0, uint32_t d1, float scale) {
    u32x4b o;
    if constexpr (WDT == kWMX8) {
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
    } else {
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
    }
    return o;
}

template <bool BF16>
__device__ __forceinline__ float16_t mfma32b(const u32x4b& a, const u32x4b& b, float16_t c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8b, a), __builtin_bit_cast(bf16x8b, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8b, a), __builtin_bit_cast(half8b, b), c, 0, 0, 0);
}

constexpr int ring_slots_kb(int bm) { return bm >= 256 ? 3 : 4; }
// weight bytes per row and stage: 64 codes are 64 bytes, or 32 for nibble pairs; micro-scaled weights add one
// 32-bit word of block scales per row (it covers 128 values, two stages)
constexpr int row_bytes_kb(int wdt) { return wdt == kWMX4 ? 32 : kRowBb; }
constexpr int slot_bytes_kb(int bm, int wdt = 0) {
    return bm * kRowAb + kBNb * row_bytes_kb(wdt) + (wdt == kWMX8 || wdt == kWMX4 ? kBNb * 4 : 0);
}

// WDT: GLA_DT_INT8, GLA_DT_UINT8, GLA_DT_FP8, kWMX8 or kWMX4; TI = 32-row MFMA tiles per wave (1, 2 or 4)
template <int WDT, bool BF16, int WAVES_M, int TI>
__global__ __launch_bounds__(WAVES_M * kWavesNb * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_kbytes_kernel(GemmKbArgs p) {
    constexpr int TJ = 2;
    constexpr int WM = 32 * TI;
    constexpr int BM = WAVES_M * WM;
    constexpr int NW = WAVES_M * kWavesNb;
    constexpr int RING = ring_slots_kb(BM);
    constexpr bool MXW = WDT == kWMX8 || WDT == kWMX4;
    constexpr bool FP4 = WDT == kWMX4;
    constexpr int ROWB = row_bytes_kb(WDT);
    constexpr int SLOT = slot_bytes_kb(BM, WDT);
    constexpr int B_OFF = BM * kRowAb;
    constexpr int S_OFF = B_OFF + kBNb * ROWB;  // micro-scaled weights: one scale word per weight row
    constexpr int A_JOBS = BM / 8;            // 16-byte copy instructions for the A tile (8 rows x 128 bytes each)
    constexpr int JOBS16 = A_JOBS + (FP4 ? kBNb / 32 : kBNb / 16);  // ... and the weight tile (16 rows x 64 bytes, or 32 rows x 32 bytes, each)
    constexpr int J16 = (JOBS16 + NW - 1) / NW;
    constexpr int J4 = MXW ? (kBNb / 64 + NW - 1) / NW : 0;  // 4-byte copies of scale words, 64 rows each
    constexpr int LPS = J16 + J4;             // copy instructions per wave per stage
    static_assert(RING * LPS < 64, "outstanding copies must fit the vmcnt counter");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / kWavesNb, wn = wave % kWavesNb;
    const int r32 = lane & 31, kb = lane >> 5;
    int tm, tn;
    tile_coords_kb(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBNb;

    // ---- copy plan: job q = wave + NW i of a stage (wave-uniform).  q < A_JOBS: rows 8q..8q+7 of the
    // activation tile, lane (row l/8, position l%8) fetches the chunk that belongs at that position of
    // the swizzled row; otherwise rows 16(q - A_JOBS).. of the weight tile, lane (row l/4, position l%4).
    // A source address is a wave-uniform base that advances per stage plus a 32-bit lane offset.
    unsigned off16[J16];
    int dst16[J16];
    bool is_a16[J16];
#pragma unroll
    for (int i = 0; i < J16; ++i) {
        int q = wave + NW * i;
        if (q > JOBS16 - 1) q = JOBS16 - 1;  // surplus jobs repeat the last one: same data, same place
        is_a16[i] = q < A_JOBS;
        if (is_a16[i]) {
            const int row = q * 8 + (lane >> 3);
            const int chunk = (lane & 7) ^ ((row >> 1) & 7);
            int gm = m0 + row;
            if (gm > p.M - 1) gm = p.M - 1;
            off16[i] = (unsigned)(gm * (int)p.xsm + chunk * 8) * 2u;
            dst16[i] = q * 8 * kRowAb;
        } else if constexpr (FP4) {
            // 32 rows of two 16-byte chunks: lane (chunk l/32, row l%32), so that the job's LDS image is
            // [chunk][row] and the 32 lanes of a half-wave later read 32 consecutive 16-byte slots
            int gn = n0 + (q - A_JOBS) * 32 + (lane & 31);
            if (gn > p.N - 1) gn = p.N - 1;
            off16[i] = (unsigned)(gn * (int)p.wsn + (lane >> 5) * 16);
            dst16[i] = B_OFF + (q - A_JOBS) * 1024;
        } else {
            const int row = (q - A_JOBS) * 16 + (lane >> 2);
            const int chunk = (lane & 3) ^ ((row >> 2) & 3);
            int gn = n0 + row;
            if (gn > p.N - 1) gn = p.N - 1;
            off16[i] = (unsigned)(gn * (int)p.wsn + chunk * 16);
            dst16[i] = B_OFF + (q - A_JOBS) * 16 * kRowBb;
        }
    }
    // micro-scaled weights: job q copies the scale word (4 blocks of 32 values = two stages) of 64 weight rows
    unsigned off4[MXW ? J4 : 1];
    int dst4[MXW ? J4 : 1];
    if constexpr (MXW) {
#pragma unroll
        for (int i = 0; i < J4; ++i) {
            int q = wave + NW * i;
            if (q > kBNb / 64 - 1) q = kBNb / 64 - 1;
            int gn = n0 + q * 64 + lane;
            if (gn > p.N - 1) gn = p.N - 1;
            off4[i] = (unsigned)(gn * (int)p.bsn);
            dst4[i] = S_OFF + q * 256;
        }
    }
    const int total_steps = p.K / kBKb;
    const int k_first = blockIdx.y * p.sps;
    const int steps = (total_steps - k_first) < p.sps ? (total_steps - k_first) : p.sps;
    const int kk_last = k_first + steps - 1;
    // past the end of the split the last stage is copied again so that every step issues the same number of copies
    int ik = k_first;
    auto issue_next = [&](int slot) __attribute__((always_inline)) {
        const int kk = ik < kk_last ? ik : kk_last;
        ++ik;
        unsigned char* base = smem + slot * SLOT;
        const unsigned char* xk = (const unsigned char*)p.x + (int64_t)kk * (kBKb * 2);
        const unsigned char* wk = p.w + (int64_t)kk * ROWB;
#pragma unroll
        for (int i = 0; i < J16; ++i) {
            const unsigned char* src = (is_a16[i] ? xk : wk) + off16[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + dst16[i]), 16, 0, 0);
        }
        if constexpr (MXW) {
            const unsigned char* sk = p.bscales + (int64_t)(kk >> 1) * 4;
#pragma unroll
            for (int i = 0; i < J4; ++i)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sk + off4[i]),
                                                 (__attribute__((address_space(3))) void*)(base + dst4[i]), 4, 0, 0);
        }
    };

    float16_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int swa = (r32 >> 1) & 7, swb = (r32 >> 2) & 3;  // chunk swizzles of this lane's rows (tile offsets are multiples of 32)
    const int a_row0 = (wm * WM + r32) * kRowAb;
    const int b_row0 = FP4 ? B_OFF + wn * TJ * 1024 + r32 * 16 + 4 * kb   // [job = 32 rows][chunk][row] image
                           : B_OFF + (wn * 32 * TJ + r32) * kRowBb + 8 * kb;
    const int s_row0 = S_OFF + (wn * 32 * TJ + r32) * 4;
    uint32_t sword[MXW ? TJ : 1];  // scale words of the stage whose K-steps are being converted

    struct Raw {
        u32x4b a[TI];   // activation chunk of the lane's row in each row tile
        u32x2b w[TJ];   // 8 weight bytes of the lane's column in each column tile
    };
    struct Ops {
        u32x4b af[TI], bq[TJ];
    };
    auto read_raw = [&](const unsigned char* base, int s, Raw& r) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) r.a[i] = *(const u32x4b*)(base + a_row0 + i * 32 * kRowAb + (((2 * s + kb) ^ swa) << 4));
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            if constexpr (FP4) {  // K-step s: bytes 8 s .. 8 s + 7 of the row = chunk s / 2, half s % 2; 4 of them per lane
                r.w[j].x = *(const uint32_t*)(base + b_row0 + j * 1024 + (s >> 1) * 512 + (s & 1) * 8);
                r.w[j].y = 0;
            } else {
                r.w[j] = *(const u32x2b*)(base + b_row0 + j * 32 * kRowBb + ((s ^ swb) << 4));
            }
        }
        if constexpr (MXW) {
            if (s == 0) {
#pragma unroll
                for (int j = 0; j < TJ; ++j) sword[j] = *(const uint32_t*)(base + s_row0 + j * 128);
            }
        }
    };
    // (s, par: the K-step just read and the parity of its stage, which pick the block's byte of the scale word)
    auto unpack = [&](const Raw& r, Ops& o, int s, int par) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) o.af[i] = r.a[i];
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            if constexpr (MXW) {
                const uint32_t e = (sword[j] >> (8 * (2 * par + (s >> 1)))) & 0xffu;
                o.bq[j] = mx_to_operand<WDT, BF16>(r.w[j].x, r.w[j].y, __builtin_bit_cast(float, e << 23));
            } else {
                o.bq[j] = bytes_to_operand<WDT, BF16>(r.w[j].x, r.w[j].y);
            }
        }
    };

    // ---- pipeline (see the header): RING stages in flight, bare barriers, explicit waits
#pragma unroll
    for (int u = 0; u < RING; ++u) issue_next(u);
    Raw raw;
    Ops ops[2];
    wait_vmcnt_kb<(RING - 1) * LPS>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_raw(smem, 0, raw);
    unpack(raw, ops[0], 0, k_first & 1);

    constexpr int NMF = TI * TJ;
    constexpr int NVA = 16 * TJ;  // VALU instructions of a conversion, roughly
    int slot = 0;
#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
        const unsigned char* base = smem + slot * SLOT;
        const int next = slot == RING - 1 ? 0 : slot + 1;
        const unsigned char* nbase = smem + next * SLOT;
        const int par = (k_first + k) & 1;
        auto kstep = [&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value;
            if constexpr (s == 3) {
                // stage k+1 has landed once at most the copies of the RING - 2 stages after it are outstanding
                wait_vmcnt_kb<(RING - 2) * LPS>();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                issue_next(slot);  // stage k + RING; every wave is done reading stage k
                __builtin_amdgcn_sched_barrier(0);
                read_raw(nbase, 0, raw);
            } else {
                read_raw(base, s + 1, raw);
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int i = 0; i < TI; ++i) acc[i][j] = mfma32b<BF16>(ops[s & 1].bq[j], ops[s & 1].af[i], acc[i][j]);
            unpack(raw, ops[(s + 1) & 1], s == 3 ? 0 : s + 1, s == 3 ? par ^ 1 : par);
            __builtin_amdgcn_sched_group_barrier(0x100, TI + TJ, 0);  // the LDS reads first
#pragma unroll
            for (int q = 0; q < NMF; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (NVA + NMF - 1) / NMF, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        kstep(std::integral_constant<int, 0>{});
        kstep(std::integral_constant<int, 1>{});
        kstep(std::integral_constant<int, 2>{});
        kstep(std::integral_constant<int, 3>{});
        slot = next;
    }

    // ---- epilogue: the lane holds output row r32 of tile i and, in elements 4g .. 4g+3 of tile j, the
    // four adjacent columns n_wave + 32 j + 8 g + 4 kb .. + 3
    const int n_wave = n0 + wn * 32 * TJ + 4 * kb;
    if (p.S > 1) {  // partial tile; the reduction kernel finishes
        float* part = p.partials + (size_t)blockIdx.y * p.M * p.N;
        const bool wide = (p.N & 3) == 0;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int m = m0 + wm * WM + i * 32 + r32;
            if (m >= p.M) continue;
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n_wave + j * 32 + 8 * g;
                    float* dst = part + (size_t)m * p.N + n;
                    if (wide && n + 3 < p.N) {
                        *(float4_t*)dst = float4_t{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (n + t < p.N) dst[t] = acc[i][j][4 * g + t];
                    }
                }
        }
        return;
    }
    float sb[TJ][16];
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int n = n_wave + j * 32 + 8 * (e / 4) + (e % 4);
            float s = 1.0f;
            if (p.col_scale && n < p.N) {
                s = load_as_float(p.scales, p.meta_dt, (int64_t)n * p.msn);
                if (p.col_scale == 2) s *= s;
            }
            sb[j][e] = s;
        }
    auto emit = [&](auto dt_tag) __attribute__((always_inline)) {
        constexpr int DT = decltype(dt_tag)::value;
        constexpr int ES = DT == GLA_DT_FP32 ? 4 : 2;
        const bool wide = (p.osm & 3) == 0 && (((uintptr_t)p.out) & (4 * ES - 1)) == 0;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int m = m0 + wm * WM + i * 32 + r32;
            if (m >= p.M) continue;
            const float sa = p.row_scale ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n_wave + j * 32 + 8 * g;
                    const int64_t o = (int64_t)m * p.osm + n;
                    float v[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] = acc[i][j][4 * g + t] * (sa * sb[j][4 * g + t]);
                    if constexpr (kWithBias) {  // `out += bias` on the output already rounded to its type
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (n + t < p.N) v[t] = round_to_dtype(DT, v[t]) + load_as_float(p.bias, p.bias_dt, n + t);
                    }
                    if (wide && n + 3 < p.N) {
                        if constexpr (DT == GLA_DT_FP32) {
                            *(float4_t*)((float*)p.out + o) = float4_t{v[0], v[1], v[2], v[3]};
                        } else if constexpr (DT == GLA_DT_FP16) {
                            *(u32x2b*)((uint16_t*)p.out + o) = u32x2b{pack_half2(v[0], v[1]),
                                                                       pack_half2(v[2], v[3])};
                        } else {
                            *(u32x2b*)((uint16_t*)p.out + o) = u32x2b{pack_bf16x2(v[0], v[1]),
                                                                       pack_bf16x2(v[2], v[3])};
                        }
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (n + t < p.N) store_typed<DT>(p.out, o + t, v[t]);
                    }
                }
        }
    };
    if (p.out_dt == GLA_DT_FP16) emit(std::integral_constant<int, GLA_DT_FP16>{});
    else if (p.out_dt == GLA_DT_BF16) emit(std::integral_constant<int, GLA_DT_BF16>{});
    else emit(std::integral_constant<int, GLA_DT_FP32>{});
}

// Sum the K splits in order, apply the scales and store: one thread per output element.
__global__ __launch_bounds__(256) void splitk_finish_kb_kernel(GemmKbArgs p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx % p.N);
    const size_t slab = (size_t)p.M * p.N;
    float v = 0.0f;
    for (int s = 0; s < p.S; ++s) v += p.partials[s * slab + idx];
    float sc = p.row_scale ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
    if (p.col_scale) {
        const float s = load_as_float(p.scales, p.meta_dt, (int64_t)n * p.msn);
        sc *= p.col_scale == 2 ? s * s : s;
    }
    v *= sc;
    if (p.bias != nullptr) v = round_to_dtype(p.out_dt, v) + load_as_float(p.bias, p.bias_dt, n);
    store_from_float(p.out, p.out_dt, (int64_t)m * p.osm + n, v);
}

template <int WDT, bool BF16, int WAVES_M, int TI>
int launch_kb(const GemmKbArgs& a, hipStream_t stream) {
    constexpr int BM = WAVES_M * 32 * TI;
    const size_t smem = (size_t)ring_slots_kb(BM) * slot_bytes_kb(BM, WDT);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = gemm_kbytes_kernel<WDT, BF16, WAVES_M, TI>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_kbytes: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n, a.S), dim3(WAVES_M * kWavesNb * 64), smem, stream, a);
    int rc = check_hip(hipGetLastError(), "gemm_kbytes launch");
    if (rc == GLA_OK && a.S > 1) {
        const int64_t items = (int64_t)a.M * a.N;
        hipLaunchKernelGGL(splitk_finish_kb_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, a);
        rc = check_hip(hipGetLastError(), "gemm_kbytes split-K reduction launch");
    }
    return rc;
}

template <int WDT, bool BF16>
int launch_kb_m(const GemmKbArgs& a, int bm, hipStream_t stream) {
    // four wave columns of 64.  A second wave row repeats the byte -> fp16/bf16 conversion, which
    // bounds the 64-row tile: one row of four waves there (measured: -17 % time at 16384^2, M <= 64;
    // at 128 rows the two arrangements time the same)
    if (bm == 256) return launch_kb<WDT, BF16, 2, 4>(a, stream);
    if (bm == 128) return launch_kb<WDT, BF16, 2, 2>(a, stream);
    return launch_kb<WDT, BF16, 1, 2>(a, stream);
}

// tile_config encoding: BM (64, 128 or 256; other = chosen here) + 1000 * K splits (0 = chosen here)
struct KbPlan {
    int bm, tiles_m, tiles_n, S, sps;
};

KbPlan kb_plan(const gla_matmul_args& p) {
    KbPlan g;
    const int cfg = p.tile_config > 0 ? p.tile_config : 0;
    const int bm_asked = cfg % 1000;
    const int total_steps = p.K / kBKb;
    // per-stage cost of a workgroup (64 K-values) by tile height, us, the chip full: the byte -> 16-bit conversion
    // makes the short tiles cheaper per stage than their share of the MFMA work
    static const int bms[3] = {64, 128, 256};
    static const float cost[3] = {0.95f, 1.48f, 1.8f};
    const TilePick pick = pick_tile_and_split(p.M, p.N, kBNb, total_steps, 8, 32, bms, cost, 3,
                                              (bm_asked == 64 || bm_asked == 128 || bm_asked == 256) ? bm_asked : 0, cfg / 1000);
    g.bm = pick.bm;
    g.tiles_m = ceil_div(p.M, g.bm);
    g.tiles_n = ceil_div(p.N, kBNb);
    int want = pick.S;
    if (want > total_steps) want = total_steps;
    if (want < 1) want = 1;
    g.sps = ceil_div(total_steps, want);
    g.S = ceil_div(total_steps, g.sps);
    return g;
}

}  // namespace

#if !GLA_KB_BIAS
bool gemm_kbytes_eligible(const gla_matmul_args& p) {
    if (p.W_nbits != 8 || p.elements_per_sample != 1) return false;
    if (!(p.w_dtype == GLA_DT_INT8 || p.w_dtype == GLA_DT_UINT8 || p.w_dtype == GLA_DT_FP8)) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16) || p.acc_dtype != GLA_DT_FP32) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    // no zero point here: the dequantisation is w or w * s with one scale per channel
    if (!(p.W_group_mode == GLA_WGM_NONE || (p.W_group_mode == GLA_WGM_SCALE && p.group_size == p.K))) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.K % kBKb != 0 || p.w_stride_n % 16 != 0 || p.x_stride_m % 8 != 0) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    // lane offsets inside the activation and weight arrays are 32-bit
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 30) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if ((p.W_group_mode == GLA_WGM_SCALE || (p.channel_scale_mode & 1)) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int64_t gemm_kbytes_workspace_bytes(const gla_matmul_args& p) {
    const KbPlan g = kb_plan(p);
    return g.S > 1 ? kWsReservedB + (int64_t)g.S * p.M * p.N * 4 : 0;
}

// ---- weight-only MX layers above 2 rows: fp16 / bf16 activations x MXFP8 / MXFP4 weights ------------
// (reference: gemlite/triton_kernels/gemm_kernels.py:509-737 with 16-bit activations and unit activation
// scales, gemlite/helper.py:199-237.)  The conversion instruction applies the block scale, so the operand is
// the dequantised weight in the activations' type: exact in bf16; in fp16 as far as code x 2^(e-127) is a
// finite normal fp16 number, which weights of trained layers are.
bool gemm_kbytes_mx_eligible(const gla_matmul_args& p) {
    if (!(p.input_dtype == GLA_DT_MXFP16 || p.input_dtype == GLA_DT_MXBF16)) return false;
    if (p.M <= 2 || p.group_size != 32 || p.channel_scale_mode != GLA_CSM_NONE || p.scales == nullptr) return false;
    const bool fp4 = p.elements_per_sample == 2 && p.W_nbits == 4;
    const bool fp8 = p.elements_per_sample == 1 && p.W_nbits == 8 && p.w_dtype == GLA_DT_FP8;
    if (!fp4 && !fp8) return false;
    switch (p.output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_MXFP16: case GLA_DT_MXBF16: break;
        default: return false;
    }
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1 || p.meta_stride_g != 1) return false;
    if (p.K % 128 != 0 || p.w_stride_n % 16 != 0 || p.x_stride_m % 8 != 0 || p.meta_stride_n % 4 != 0) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15) || ((uintptr_t)p.scales & 3)) return false;
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 30) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if ((int64_t)p.N * p.meta_stride_n >= (1ll << 31)) return false;
    return true;
}

int64_t gemm_kbytes_mx_workspace_bytes(const gla_matmul_args& p) { return gemm_kbytes_workspace_bytes(p); }
#endif

#if GLA_KB_BIAS
int launch_gemm_kbytes_mx_bias(const gla_matmul_args& p, hipStream_t stream) {
#else
int launch_gemm_kbytes_mx(const gla_matmul_args& p, hipStream_t stream) {
#endif
    if (!gemm_kbytes_mx_eligible(p)) {
        set_error("gemm_kbytes_mx: operands not eligible (K-contiguous MXFP8 / MXFP4 weights, K %% 128 == 0, more than 2 rows)");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    GemmKbArgs a;
    a.x = (const uint16_t*)p.x; a.w = (const uint8_t*)p.w; a.scales = nullptr; a.scales_x = nullptr; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.msn = 0; a.sxm = 0;
    a.col_scale = 0; a.row_scale = 0;
    a.bscales = (const uint8_t*)p.scales; a.bsn = p.meta_stride_n;
    a.bias = kWithBias ? p.bias : nullptr; a.bias_dt = p.bias_dtype;
    if (kWithBias && p.bias == nullptr) {
        set_error("gemm_kbytes_mx: the bias variant was called without a bias");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype == GLA_DT_MXFP16 ? GLA_DT_FP16 : (p.output_dtype == GLA_DT_MXBF16 ? GLA_DT_BF16 : p.output_dtype);
    const KbPlan g = kb_plan(p);
    a.tiles_m = g.tiles_m; a.tiles_n = g.tiles_n; a.S = g.S; a.sps = g.sps;
    a.partials = nullptr;
    if (g.S > 1) {
        const int64_t need = gemm_kbytes_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemm_kbytes_mx: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.partials = (float*)((char*)p.workspace + kWsReservedB);
    }
    const bool bf16 = p.input_dtype == GLA_DT_MXBF16;
    if (p.elements_per_sample == 2)
        return bf16 ? launch_kb_m<kWMX4, true>(a, g.bm, stream) : launch_kb_m<kWMX4, false>(a, g.bm, stream);
    return bf16 ? launch_kb_m<kWMX8, true>(a, g.bm, stream) : launch_kb_m<kWMX8, false>(a, g.bm, stream);
}

#if GLA_KB_BIAS
int launch_gemm_kbytes_bias(const gla_matmul_args& p, hipStream_t stream) {
#else
int launch_gemm_kbytes(const gla_matmul_args& p, hipStream_t stream) {
#endif
    GemmKbArgs a;
    a.x = (const uint16_t*)p.x; a.w = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.K = p.K;
    a.xsm = p.x_stride_m; a.wsn = p.w_stride_n; a.osm = p.out_stride_m; a.msn = p.meta_stride_n; a.sxm = p.sx_stride_m;
    a.col_scale = (p.W_group_mode == GLA_WGM_SCALE ? 1 : 0) + ((p.channel_scale_mode & 1) ? 1 : 0);
    a.row_scale = (p.channel_scale_mode & 2) ? 1 : 0;
    a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype; a.out_dt = p.output_dtype;
    a.bscales = nullptr; a.bsn = 0;
    a.bias = kWithBias ? p.bias : nullptr; a.bias_dt = p.bias_dtype;
    if (kWithBias && p.bias == nullptr) {
        set_error("gemm_kbytes: the bias variant was called without a bias");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    const KbPlan g = kb_plan(p);
    a.tiles_m = g.tiles_m; a.tiles_n = g.tiles_n; a.S = g.S; a.sps = g.sps;
    a.partials = nullptr;
    if (g.S > 1) {
        const int64_t need = gemm_kbytes_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemm_kbytes: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.partials = (float*)((char*)p.workspace + kWsReservedB);
    }
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.w_dtype) {
        case GLA_DT_INT8: return bf16 ? launch_kb_m<GLA_DT_INT8, true>(a, g.bm, stream) : launch_kb_m<GLA_DT_INT8, false>(a, g.bm, stream);
        case GLA_DT_UINT8: return bf16 ? launch_kb_m<GLA_DT_UINT8, true>(a, g.bm, stream) : launch_kb_m<GLA_DT_UINT8, false>(a, g.bm, stream);
        default: return bf16 ? launch_kb_m<GLA_DT_FP8, true>(a, g.bm, stream) : launch_kb_m<GLA_DT_FP8, false>(a, g.bm, stream);
    }
}

}  // namespace gla
