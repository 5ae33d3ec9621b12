// MFMA GEMM for K-contiguous narrow operands: out[M,N] = x[M,K] * w[N,K]^T with
//   fp8-e4m3 x fp8-e4m3 -> fp32      (v_mfma_f32_32x32x64_f8f6f4, unit block scales)
//   int8 x int8 -> int32             (v_mfma_i32_32x32x32_i8, exact)
//   MXFP4 x MXFP4 -> fp32            (v_mfma_scale_f32_32x32x64_f8f6f4 with one e8m0 scale per
//                                     32 K-values on either operand; MXFP8 likewise)
//   fp8 / int8 with fp32 scales per 128 x 128 weight block and per (activation row, 128 values):
//                                     the sum over each 128 values of K is folded, scaled, into a
//                                     second fp32 accumulator (channel_scale_mode 5,
//                                     reference: gemlite/triton_kernels/gemm_kernels.py:441-450)
// and a per-row / per-column scale epilogue.  The prefill path of dynamically quantised A8W8
// and A4W4 layers.
//
// Takes the place of the reference's GEMM kernels for unpacked 8-bit weights and for the
// micro-scaled formats (reference: gemlite/triton_kernels/gemm_kernels.py:285-496 and :509-737,
// epilogue :471-488, tl.dot_scaled :696).
//
//  * Workgroup tile BM x 256, pipeline stage of 64 bytes of K per row (64 fp8/int8 values or 128
//    fp4 values); 8 waves in a 2 x 4 grid, wave tile (BM/2) x 64 of 32x32 MFMA tiles; the
//    accumulators stay in registers for the whole K loop.
//  * Operand tiles (and the MXFP4 block scales) are copied global -> LDS by the load unit itself
//    (global_load_lds) into a ring of 4 stages, all in flight: a stage's slot is refilled as soon as
//    every wave has read its fragments into registers, which happens one step before they are
//    multiplied (fragments are double-buffered in registers), so LDS latency and the barrier are
//    hidden behind the MFMAs and the loop waits only for the oldest copy.  The LDS
//    image is dense; 16-byte chunk c of row r is placed at chunk position c ^ ((r >> 2) & 3),
//    chosen on the global side of the copy, so that the 16 lanes of one LDS read phase hit 16
//    distinct bank groups.
//  * Workgroups are renumbered so that each of the 8 XCDs (one L2 each) works on its own band
//    of output tiles, and tiles inside a band are visited in groups that share operand panels.
//  * The weights are the row operand of every MFMA: an accumulator is the transposed output tile,
//    so a lane holds four adjacent output columns of one row and stores them at once.
//  * MXFP4 with tiles of 128 rows or more: a small kernel first regroups both scale arrays by
//    pipeline stage in the workspace (dst[stage][row], one 32-bit word each), so that a tile's
//    scales are one contiguous run per stage instead of one cache line per row.
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

enum Mode { kFP8 = 0, kINT8 = 1, kMXFP4 = 2, kMXFP8 = 3, kMXFP8T = 4, kBQF8 = 5, kBQI8 = 6, kMX84 = 7, kMX84T = 8, kH16 = 9, kB16 = 10, kINT8R = 11 };
// kINT8R: int8 x int8 whose K is not a multiple of 64 (a K-step past the end multiplies zeroed operands: a select per
// operand register and K-step, 33 vector instructions per stage in front of the MFMAs that the other layers do without)
// kH16 / kB16: fp16 x fp16 / bf16 x bf16 (unquantised layers, W_nbits = 16): the byte geometry of the int8 mode (two
// K-steps of 32 bytes per stage, here 16 values each) on v_mfma_f32_32x32x16; built in a translation unit of its own
// kMXFP8T: MXFP8 weights whose activations carry no block scales (their per-token scale is applied in the
// epilogue), so no registers are spent on activation scale words and the 256-row tile fits
// kMX84 / kMX84T: fp8 activations (with MXFP8 micro-scales / per token) x MXFP4 weights: the mixed form of the
// scaled MFMA; a stage's weight tile has rows of 32 bytes (64 e2m1 values)
// kBQF8 / kBQI8: fp8 / int8 with one fp32 scale per 128 x 128 weight block and per (activation row, 128 values):
// the sum over two stages (128 values) goes to a second, fp32 accumulator scaled by both

constexpr int kRowB8 = 64;  // bytes per LDS row = bytes of K per pipeline stage
constexpr int kBN = 256;
constexpr int kWavesM = 2;  // wave rows; wave columns WN (4 or 2) are a template parameter

struct Gemm8Args {
    const uint8_t* a;      // [M, Kb] bytes
    const uint8_t* b;      // [N, Kb] bytes
    const void* scales;    // weight scales: [N] (channel) or [N, K/32] e8m0 (MXFP4)
    const void* scales_x;  // activation scales: [M] or [M_pad, K/32] e8m0
    void* out;
    int M, N, Kb;          // Kb = bytes of K per row
    int64_t lda, ldb, osm, sxm, msn;
    int64_t sx_stage, sw_stage;  // micro-scaled: bytes from one scale word of a row to the next one's
    const void* ascales;         // micro-scaled: activation block scales (row stride asxm bytes); scales_x is the epilogue's
    int64_t asxm;
    int csm, meta_dt, sx_dt, out_dt;
    int tiles_m, tiles_n;
    int S;     // K splits (gridDim.y)
    int sps;   // pipeline stages per split
    void* partials;  // [S][M][N] 32-bit accumulators when S > 1
    const void* bias;  // [N] or NULL: added to the result rounded to the output type (float outputs)
    int bias_dt;
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

// s_waitcnt vmcnt(N) only: vmcnt is bits 3:0 and 15:14, expcnt (6:4) and lgkmcnt (11:8) left at "no wait"
template <int N>
__device__ __forceinline__ void wait_vmcnt8() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

constexpr int kRing8 = 4;  // LDS ring of pipeline stages, all of them in flight
constexpr int slot_bytes8(int mode, int bm) {
    const bool w4 = mode == kMX84 || mode == kMX84T;
    return bm * kRowB8 + kBN * (w4 ? 32 : kRowB8) + (mode == kFP8 || mode == kINT8 || mode == kINT8R || mode == kH16 || mode == kB16 ? 0 : (bm + kBN) * 4);
}

// WN = wave columns (4): 8 waves, wave tile (BM/2) x 64, up to 128 accumulator registers per lane.
// (A 2-column variant with 4 waves of 128 x 128 and accumulators in AGPRs reads a third less from
// LDS per MFMA but, with one wave per SIMD and fragments read in the step that multiplies them,
// measured slower.  LDS bandwidth is not what limits these loops: 128-bit reads sustain well over
// 200 bytes per clock and CU, the loop needs about 35.  With random operands the board's power
// limit is: the clock falls to about 1.55 GHz under these kernels.)
// BIAS: the epilogue adds p.bias.  A separate instantiation: the extra rounding and the bias loads cost the
// 256-row tile 10-35 % when they are compiled into the one kernel and merely switched off at run time.
template <int MODE, int BM, int WN, bool BIAS = false>
__global__ __launch_bounds__(kWavesM * WN * 64) void gemm_8bit_kernel(Gemm8Args p) {
    constexpr int WM = BM / kWavesM;  // wave tile rows
    constexpr int TI = WM / 32;       // 32-row MFMA tiles per wave along M
    constexpr int WNC = kBN / WN;     // wave tile columns
    constexpr int TJ = WNC / 32;      // 32-column MFMA tiles per wave along N
    constexpr bool W4 = MODE == kMX84 || MODE == kMX84T;    // MXFP4 weights under fp8 activations
    constexpr bool M8 = MODE == kMXFP8 || MODE == kMXFP8T || W4;
    constexpr bool TOKEN = MODE == kMXFP8T || MODE == kMX84T;  // no activation block scales
    constexpr bool BQ = MODE == kBQF8 || MODE == kBQI8;     // fp32 block scales, applied by the vector unit
    constexpr bool F8 = MODE == kFP8 || MODE == kBQF8;      // plain fp8 operands, one 64-byte K-step per stage
    constexpr bool I8 = MODE == kINT8 || MODE == kINT8R || MODE == kBQI8;
    constexpr bool RAGGED = MODE == kINT8R;                 // K ends inside a stage
    constexpr bool H16 = MODE == kH16 || MODE == kB16;      // 16-bit float operands, two K-steps of 16 values per stage
    constexpr bool MX = MODE == kMXFP4 || M8 || BQ;         // block scales ride along with every stage
    // MXFP8 and the fp32 block scales: a 32-bit scale word of a row covers 128 values = two stages; MXFP4: one stage
    constexpr int SSH = (M8 || BQ) ? 1 : 0;
    constexpr int NW = kWavesM * WN;
    constexpr int RING = kRing8;
    constexpr int SLOT = slot_bytes8(MODE, BM);
    constexpr int ROWW = W4 ? 32 : kRowB8;    // bytes of a weight row per stage
    constexpr int B_OFF = BM * kRowB8, S_OFF = BM * kRowB8 + kBN * ROWW;
    constexpr int A_JOBS = BM / 16;           // 16-byte copy instructions for the A tile (16 rows each)
    constexpr int JOBS16 = A_JOBS + (W4 ? kBN / 32 : kBN / 16); // ... and the B tile (W4: 32 rows of two chunks each)
    constexpr int J16 = (JOBS16 + NW - 1) / NW;
    constexpr int A_JOBS4 = TOKEN ? 0 : BM / 64;
    constexpr int JOBS4 = A_JOBS4 + kBN / 64; // micro-scaled: 4-byte copies of block scales, 64 rows each
    constexpr int J4 = MX ? (JOBS4 + NW - 1) / NW : 0;
    constexpr int LPS = J16 + J4;             // copy instructions per wave per stage
    static_assert(RING * LPS < 64, "outstanding copies must fit the vmcnt counter");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    // The wave index as a scalar: what depends on it alone (which operand a copy job serves, and with it
    // the choice between two kernel arguments) is then decided by scalar selects.  Left in a vector
    // register, such a choice becomes a load of the chosen argument inside the K loop, and the wait for
    // it drains every copy in flight.
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBN;

    // ---- copy plan.  Everything a stage needs reaches LDS through global_load_lds, so the K loop
    // holds no loads into registers and the only waits on the vector-memory counter are the
    // explicit ones below.  Job q = wave + NW i (wave-uniform) moves 16 rows x 64 bytes of one tile:
    // lane (row l/4, position l%4) fetches the 16-byte chunk that belongs at that position of the
    // swizzled row (chunk c of row r sits at position c ^ ((r >> 2) & 3)).  A source address is a
    // wave-uniform base that advances per stage plus a 32-bit lane offset.
    unsigned off16[J16];
    int chunk16[J16], dst16[J16];
    bool is_a16[J16];
#pragma unroll
    for (int i = 0; i < J16; ++i) {
        int q = wave + NW * i;
        if (q > JOBS16 - 1) q = JOBS16 - 1;  // surplus jobs repeat the last one: same data, same place
        is_a16[i] = q < A_JOBS;
        const int row = (is_a16[i] ? q : q - A_JOBS) * 16 + (lane >> 2);
        chunk16[i] = ((lane & 3) ^ ((row >> 2) & 3)) * 16;
        if (W4 && !is_a16[i]) {
            // 32 weight rows of two 16-byte chunks: lane (chunk l/32, row l%32); the job's LDS image is
            // [chunk][row], so a half-wave later reads 32 consecutive 16-byte slots
            int gn = n0 + (q - A_JOBS) * 32 + (lane & 31);
            if (gn > p.N - 1) gn = p.N - 1;
            chunk16[i] = (lane >> 5) * 16;
            off16[i] = (unsigned)(gn * (int)p.ldb);
            dst16[i] = B_OFF + (q - A_JOBS) * 1024;
        } else if (is_a16[i]) {
            int gm = m0 + row;
            if (gm > p.M - 1) gm = p.M - 1;
            off16[i] = (unsigned)(gm * (int)p.lda);
            dst16[i] = q * 16 * kRowB8;
        } else {
            int gn = n0 + row;
            if (gn > p.N - 1) gn = p.N - 1;
            off16[i] = (unsigned)(gn * (int)p.ldb);
            dst16[i] = B_OFF + (q - A_JOBS) * 16 * kRowB8;
        }
    }
    // MXFP4: job q copies the 4 scale bytes (4 blocks of 32 values) of 64 rows, one row per lane
    unsigned off4[MX ? J4 : 1];
    int dst4[MX ? J4 : 1];
    bool is_a4[MX ? J4 : 1];
    if constexpr (MX) {
#pragma unroll
        for (int i = 0; i < J4; ++i) {
            int q = wave + NW * i;
            if (q > JOBS4 - 1) q = JOBS4 - 1;
            is_a4[i] = q < A_JOBS4;
            if (is_a4[i]) {
                int gm = m0 + q * 64 + lane;
                if (gm > p.M - 1) gm = p.M - 1;
                off4[i] = (unsigned)(gm * (int)p.asxm);
            } else {
                int gn = n0 + (q - A_JOBS4) * 64 + lane;
                if (gn > p.N - 1) gn = p.N - 1;
                off4[i] = (unsigned)((BQ ? gn / 128 : gn) * (int)p.msn);  // BQ: every column copies its block's word
            }
            // the LDS image keeps room for the activation scales of BM rows whether they are copied or not
            dst4[i] = S_OFF + (is_a4[i] ? q : q - A_JOBS4 + BM / 64) * 256;
        }
    }

    const int total_steps = (p.Kb + kRowB8 - 1) / kRowB8;
    const int k_first = blockIdx.y * p.sps;  // first stage of this split
    const int steps = (total_steps - k_first) < p.sps ? (total_steps - k_first) : p.sps;
    // A row's last stage may hold fewer than 64 bytes: chunks past the end re-read chunk 0 of the
    // stage (always inside the row) and are never multiplied.  Stages past the end of K copy the
    // last one again so that every step issues the same number of copies.
    // copy c (0 <= c < LPS) of stage k into ring slot `slot`
    // The operand a job copies from, chosen once, here, between two argument values held in scalar
    // registers.  (Written as a choice between p.a and p.b at the point of use, the compiler selects
    // between the arguments' addresses and loads the chosen one inside the K loop.)
    const uint8_t *arg_a = p.a, *arg_b = p.b;
    asm volatile("" : "+s"(arg_a), "+s"(arg_b));
    const uint8_t* src16[J16];
#pragma unroll
    for (int i = 0; i < J16; ++i) src16[i] = is_a16[i] ? arg_a : arg_b;
    const uint8_t* src4[MX ? J4 : 1];
    int64_t stage4[MX ? J4 : 1];
    if constexpr (MX) {
        const uint8_t *arg_sx = (const uint8_t*)p.ascales, *arg_sw = (const uint8_t*)p.scales;
        int64_t arg_xs = p.sx_stage, arg_ws = p.sw_stage;
        asm volatile("" : "+s"(arg_sx), "+s"(arg_sw), "+s"(arg_xs), "+s"(arg_ws));
#pragma unroll
        for (int i = 0; i < J4; ++i) {
            src4[i] = is_a4[i] ? arg_sx : arg_sw;
            stage4[i] = is_a4[i] ? arg_xs : arg_ws;
        }
    }
    auto issue_one = [&](int k, int slot, int c) __attribute__((always_inline)) {
        const int kk = k_first + (k > steps - 1 ? steps - 1 : k);  // absolute stage
        unsigned char* base = smem + slot * SLOT;
        if (c < J16) {
            const int limit = p.Kb - kk * kRowB8;
            const uint8_t* src = src16[c] + kk * (is_a16[c] ? kRowB8 : ROWW) + (off16[c] + (unsigned)(chunk16[c] < limit ? chunk16[c] : 0));
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + dst16[c]), 16, 0, 0);
        } else if constexpr (MX) {
            const int i = c - J16;
            const uint8_t* sk = src4[i] + (kk >> SSH) * stage4[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sk + off4[i]),
                                             (__attribute__((address_space(3))) void*)(base + dst4[i]), 4, 0, 0);
        }
    };
    auto issue = [&](int k, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < LPS; ++c) issue_one(k, slot, c);
    };

    // ---- accumulators
    typedef typename std::conditional<I8, int16_t_v, float16_t>::type acc_t;
    acc_t acc[TI][TJ];
    float16_t folded[BQ ? TI : 1][BQ ? TJ : 1];  // BQ: the scaled sum over the 128-blocks done so far
    if constexpr (BQ) {
#pragma unroll
        for (int i = 0; i < TI; ++i)
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) folded[i][j][e] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int r32 = lane & 31, kb = lane >> 5;
    const int sw = (r32 >> 2) & 3;  // chunk swizzle of this lane's rows (tile offsets are multiples of 32)
    // the two 16-byte chunks of a 64-byte row this lane feeds to the MFMAs of a stage:
    // fp8 (one K-step of 64 bytes): chunks 2kb, 2kb+1; int8 / fp4 (two K-steps of 32 bytes): chunks kb, 2+kb
    const int c0 = ((F8 ? 2 * kb : kb) ^ sw) << 4;
    const int c1 = ((F8 ? 2 * kb + 1 : 2 + kb) ^ sw) << 4;
    const int a_row0 = (wm * WM + r32) * kRowB8;
    // W4: [32-row job][chunk][row] image, the half-wave's chunk kb is K-block kb of the stage
    const int b_row0 = W4 ? B_OFF + (wn * TJ) * 1024 + kb * 512 + r32 * 16 : B_OFF + (wn * WNC + r32) * kRowB8;
    const int sa_row0 = S_OFF + (wm * WM + r32) * 4;
    const int sb_row0 = S_OFF + (BM + wn * WNC + r32) * 4;

    // Operand fragments are double-buffered in registers: while the MFMAs of stage k run on one
    // set, the LDS reads of stage k+1 fill the other, so neither LDS latency nor the barrier
    // leaves the matrix pipe idle.
    // fp8: the two chunks form the eight-register operand of one MFMA; int8 / fp4: one chunk per K-step
    typedef union {
        int8_t_v v8;
        u32x4 c[2];
    } frag_t;
    frag_t fa[2][TI], fb[2][TJ];
    unsigned fsa[2][MX && !TOKEN ? TI : 1], fsb[2][MX ? TJ : 1];
    // LDS read r of a stage's NRD: chunk reads of the weight tiles, then of the activation tiles,
    // then (MXFP4) the scale words
    constexpr int NRD = (TI + TJ) * 2 + (MX ? (TOKEN ? TJ : TI + TJ) : 0);
    // (`par`: parity of the absolute stage being read, which picks the half of an MXFP8 scale word)
    auto load_one = [&](int slot, auto buf_tag, int r, int par) __attribute__((always_inline)) {
        constexpr int B = decltype(buf_tag)::value;
        const unsigned char* base = smem + slot * SLOT;
        if (r < 2 * TJ) {
            if constexpr (W4) {
                if (r % 2 == 0) fb[B][r / 2].c[0] = *(const u32x4*)(base + b_row0 + (r / 2) * 1024);
            } else {
                fb[B][r / 2].c[r % 2] = *(const u32x4*)(base + b_row0 + (r / 2) * 32 * kRowB8 + (r % 2 ? c1 : c0));
            }
        } else if (r < 2 * (TI + TJ)) {
            const int q = r - 2 * TJ;
            fa[B][q / 2].c[q % 2] = *(const u32x4*)(base + a_row0 + (q / 2) * 32 * kRowB8 + (q % 2 ? c1 : c0));
        } else if constexpr (MX) {
            // MXFP4: half-wave kb multiplies blocks kb and 2 + kb of the stage: shift them into bytes 0 and 2.
            // MXFP8: it multiplies with the scale of block kb of the stage, byte 2 par + kb of the word.
            const int q = r - 2 * (TI + TJ) + (TOKEN ? TI : 0);   // TOKEN: weight scale words only
            const int sh = BQ ? 0 : (M8 ? 8 * (2 * par + kb) : 8 * kb);  // BQ: the word is the fp32 scale
            if (q < TI) {
                if constexpr (!TOKEN) fsa[B][q] = *(const unsigned*)(base + sa_row0 + q * 128) >> sh;
            } else {
                fsb[B][q - TI] = *(const unsigned*)(base + sb_row0 + (q - TI) * 128) >> sh;
            }
        }
    };
    // The same for one K-step (h = 0, 1) of a stage, into fragment buffer 0: read r of TI + TJ chunk reads
    // and, after them, of the TI + TJ scale words, which go to scale buffer SB
    auto load_half = [&](int slot, int h, auto scale_tag, int r) __attribute__((always_inline)) {
        constexpr int SB = decltype(scale_tag)::value;
        const unsigned char* base = smem + slot * SLOT;
        if (r < TJ) {
            fb[0][r].c[h] = *(const u32x4*)(base + b_row0 + r * 32 * kRowB8 + (h ? c1 : c0));
        } else if (r < TI + TJ) {
            fa[0][r - TJ].c[h] = *(const u32x4*)(base + a_row0 + (r - TJ) * 32 * kRowB8 + (h ? c1 : c0));
        } else if constexpr (MX) {
            const int q = r - (TI + TJ);
            if (q < TI) fsa[SB][q] = *(const unsigned*)(base + sa_row0 + q * 128) >> (8 * kb);
            else fsb[SB][q - TI] = *(const unsigned*)(base + sb_row0 + (q - TI) * 128) >> (8 * kb);
        }
    };
    auto load_frags = [&](int slot, auto buf_tag, int par) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < NRD; ++r) load_one(slot, buf_tag, r, par);
    };
    // MFMA q of a stage's NM.  fp8: one K-step of 64 bytes per tile pair; int8 / fp4: two K-steps of 32
    constexpr int NM = TI * TJ * (F8 || M8 ? 1 : 2);
    auto multiply_one = [&](int limit, auto buf_tag, auto scale_tag, int q) __attribute__((always_inline)) {
        constexpr int B = decltype(buf_tag)::value;    // fragment buffer
        constexpr int SB = decltype(scale_tag)::value; // scale buffer (MXFP4)
        const int s2 = q / (TI * TJ), i = (q % (TI * TJ)) / TJ, j = q % TJ;
        // BQ: the first MFMA of a 128-block (even stage = register buffer 0, first K-step) starts from zero
        // instead of the accumulator, which spares the vector unit clearing it after every fold
        constexpr bool FRESH_STAGE = BQ && B == 0;
        if constexpr (F8) {
            acc_t cin = acc[i][j];
            if constexpr (FRESH_STAGE) {
#pragma unroll
                for (int e = 0; e < 16; ++e) cin[e] = 0;
            }
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[B][j].v8, fa[B][i].v8, cin, 0, 0, 0, 127, 0, 127);
        } else if constexpr (W4) {
            // mixed formats: e2m1 weights (the first four operand registers, K-block kb in half-wave kb) x e4m3
            // activations (chunk pair (kb, 2 + kb) as for MXFP8); each half-wave's scale byte is that of block kb
            const int4_t b4 = int4_t{(int)fb[B][j].c[0].x, (int)fb[B][j].c[0].y, (int)fb[B][j].c[0].z, (int)fb[B][j].c[0].w};
            const int8_t_v b8 = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
            if constexpr (TOKEN)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, fa[B][i].v8, acc[i][j], 4, 0, 0, (int)fsb[SB][j], 0, 127);
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, fa[B][i].v8, acc[i][j], 4, 0, 0, (int)fsb[SB][j], 0,
                                                                            (int)fsa[SB][i]);
        } else if constexpr (TOKEN) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[B][j].v8, fa[B][i].v8, acc[i][j], 0, 0, 0,
                                                                        (int)fsb[SB][j], 0, 127);
        } else if constexpr (MODE == kMXFP8) {
            // registers 0-3 of both half-waves are block 0 of the stage, registers 4-7 block 1, and the
            // half-wave's scale is that of block kb: the chunk pair (kb, 2 + kb) as one operand
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[B][j].v8, fa[B][i].v8, acc[i][j], 0, 0, 0,
                                                                        (int)fsb[SB][j], 0, (int)fsa[SB][i]);
        } else {
            // a K-step past the end of a ragged K multiplies zeros (no branch: the accumulators
            // must not live across control flow)
            const bool valid = !RAGGED || s2 * 32 < limit;
            u32x4 af = fa[B][i].c[s2];
            if (!valid) af = u32x4{0, 0, 0, 0};
            const u32x4 bf = fb[B][j].c[s2];
            if constexpr (I8) {
                acc_t cin = acc[i][j];
                if (FRESH_STAGE && s2 == 0) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) cin[e] = 0;
                }
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(int4_t{(int)bf.x, (int)bf.y, (int)bf.z, (int)bf.w},
                                                                  int4_t{(int)af.x, (int)af.y, (int)af.z, (int)af.w}, cin, 0, 0, 0);
            } else if constexpr (H16) {
                if constexpr (MODE == kB16)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf), __builtin_bit_cast(bf16x8_t, af), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, bf), __builtin_bit_cast(half8_t, af), acc[i][j], 0, 0, 0);
            } else {
                // fp4 operands occupy the first four of the eight operand registers; the rest is not read
                const int4_t a4 = int4_t{(int)af.x, (int)af.y, (int)af.z, (int)af.w};
                const int4_t b4 = int4_t{(int)bf.x, (int)bf.y, (int)bf.z, (int)bf.w};
                const int8_t_v a8 = __builtin_shufflevector(a4, a4, 0, 1, 2, 3, -1, -1, -1, -1);
                const int8_t_v b8 = __builtin_shufflevector(b4, b4, 0, 1, 2, 3, -1, -1, -1, -1);
                if (s2 & 1)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, a8, acc[i][j], 4, 4, 2, (int)fsb[SB][j], 2, (int)fsa[SB][i]);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b8, a8, acc[i][j], 4, 4, 0, (int)fsb[SB][j], 0, (int)fsa[SB][i]);
            }
        }
    };

    // ---- pipeline.  Copies complete in issue order.  Barriers are bare on purpose (a __syncthreads()
    // carries a release fence, which for copies into LDS means draining the counter and with it the
    // pipeline); the empty asm statements pin LDS accesses to their side of a barrier.
    // Operand fragments are read one step ahead of the MFMAs that use them, so that LDS latency is
    // hidden although the barrier keeps all waves of the workgroup in the same phase:
    //  * whole stages (two register buffers): RING stages in flight; step k reads stage k+1 and
    //    multiplies stage k, whose slot is refilled;
    //  * HALF (MXFP4 with the 256-row tile, which has no registers for a second buffer): the two
    //    K-steps of a stage are the two buffers.  RING - 1 stages in flight; step k multiplies K-step 0
    //    of stage k while reading its K-step 1, then multiplies that while reading K-step 0 of stage
    //    k+1, and refills the slot of stage k-1.  The scale words of a stage serve both K-steps and
    //    alternate between two buffers.
    constexpr bool HALF = MODE == kMXFP4 && BM == 256;
    constexpr int AHEAD = HALF ? RING - 1 : RING;
    typedef std::integral_constant<int, 0> tag0;
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) issue(u, u);
    wait_vmcnt8<(AHEAD - 1) * LPS>();  // stage 0 has landed (this wave's part)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();      // ... and everybody else's
    asm volatile("" ::: "memory");
    if constexpr (HALF) {
#pragma unroll
        for (int r = 0; r < 2 * (TI + TJ); ++r) load_half(0, 0, tag0{}, r);
    } else {
        load_frags(0, tag0{}, k_first & 1);
    }

    // BQ: tile t = i * TJ + j has summed a whole 128-block (an even and an odd stage; splits start on even
    // stages, so the odd ones are those multiplied from register buffer 1, whose scale words are the block's):
    // add it, scaled, to the fp32 result (the next block's first MFMA starts from zero)
    auto fold_one = [&](int t) __attribute__((always_inline)) {
        if constexpr (BQ) {
            const int i = t / TJ, j = t % TJ;
            const float sc = __builtin_bit_cast(float, fsa[1][i]) * __builtin_bit_cast(float, fsb[1][j]);
#pragma unroll
            for (int e = 0; e < 16; ++e) folded[i][j][e] = __builtin_fmaf((float)acc[i][j][e], sc, folded[i][j][e]);
        }
    };
    int slot = 0;  // ring slot of the stage being multiplied
    auto step = [&](int k, auto buf_tag) __attribute__((always_inline)) {
        constexpr int B = decltype(buf_tag)::value;
        typedef std::integral_constant<int, B ^ 1> other;
        // stage k+1, read in this step, has landed once at most the copies of the stages issued after
        // it are outstanding; after the barrier the slot refilled below is no longer read by anyone
        wait_vmcnt8<(AHEAD - 2) * LPS>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // The step is cut into NM slices of one MFMA, a share of the copies and a share of
        // the LDS reads, with the scheduler fenced between slices.  Left alone, the compiler issues the
        // copies in one burst right after the barrier, where every wave of the workgroup queues at
        // the one address unit of the CU (16 clocks per 16-byte-per-lane instruction) before its first
        // MFMA, and the matrix pipe idles for that long in every step.
        const int limit = p.Kb - (k_first + k) * kRowB8;
        const int next = slot == RING - 1 ? 0 : slot + 1;
        // (the reads go with the first slices only, so that the last of them has returned when the
        // MFMAs that follow need it)
        if constexpr (!HALF) {
            constexpr int RS = NM > 2 ? NM * 3 / 4 : NM;  // slices that carry reads
#pragma unroll
            for (int q = 0; q < NM; ++q) {
                multiply_one(limit, buf_tag, buf_tag, q);
#pragma unroll
                for (int c = q * LPS / NM; c < (q + 1) * LPS / NM; ++c) issue_one(k + RING, slot, c);
#pragma unroll
                for (int r = q * NRD / RS; r < (q + 1) * NRD / RS && r < NRD; ++r) load_one(next, other{}, r, (k_first + k + 1) & 1);
                // a finished tile is folded one slice after its last MFMA, in the shadow of the next one
                if constexpr (BQ && B == 1) {
                    if (q > NM - TI * TJ) fold_one(q - (NM - TI * TJ) - 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (BQ && B == 1) fold_one(TI * TJ - 1);
        } else {
            const int refill = slot == 0 ? RING - 1 : slot - 1;
            constexpr int H = NM / 2, HS = H / 2, R1 = TI + TJ, R2 = 2 * (TI + TJ);
#pragma unroll
            for (int q = 0; q < NM; ++q) {
                multiply_one(limit, tag0{}, buf_tag, q);
#pragma unroll
                for (int c = q * LPS / NM; c < (q + 1) * LPS / NM; ++c) issue_one(k + RING - 1, refill, c);
                if (q < H) {
#pragma unroll
                    for (int r = q * R1 / HS; r < (q + 1) * R1 / HS && r < R1; ++r) load_half(slot, 1, buf_tag, r);
                } else {
#pragma unroll
                    for (int r = (q - H) * R2 / HS; r < (q - H + 1) * R2 / HS && r < R2; ++r) load_half(next, 0, other{}, r);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        slot = next;
    };
#pragma unroll 1
    for (int k = 0; k < steps; k += 2) {  // two steps per trip: the register buffers alternate
        step(k, std::integral_constant<int, 0>{});
        if (k + 1 < steps) step(k + 1, std::integral_constant<int, 1>{});
    }

    // ---- epilogue.  The weight fragment is the row operand of every MFMA, so a tile's accumulator is
    // the transposed output tile: the lane holds output row r32 (of the tile) and, in elements
    // 4g .. 4g+3, the four adjacent output columns 8g + 4kb .. + 3, which leave in one store.
    const int n_wave = n0 + wn * WNC + 4 * kb;
    if (p.S > 1) {  // partial tile, raw 32-bit accumulators; the reduction kernel finishes
        typedef typename std::conditional<MODE == kINT8 || MODE == kINT8R, int32_t, float>::type raw_t;  // BQ: the scaled fp32 sums
        typedef raw_t raw4_t __attribute__((ext_vector_type(4)));
        raw_t* part = (raw_t*)p.partials + (size_t)blockIdx.y * p.M * p.N;
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
                    raw_t* dst = part + (size_t)m * p.N + n;
                    raw_t v[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        if constexpr (BQ) v[t] = folded[i][j][4 * g + t];
                        else v[t] = acc[i][j][4 * g + t];
                    }
                    if (wide && n + 3 < p.N) {
                        *(raw4_t*)dst = raw4_t{v[0], v[1], v[2], v[3]};
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (n + t < p.N) dst[t] = v[t];
                    }
                }
        }
        return;
    }
    const bool col_scale = !MX && (p.csm & 1);
    const bool row_scale = MODE != kMXFP4 && !BQ && (p.csm & 2);
    auto value = [&](int i, int j, int e) __attribute__((always_inline)) -> float {
        if constexpr (BQ) return folded[i][j][e];
        else return (float)acc[i][j][e];
    };
    // The element type is tested once per vector, outside the loops, so that a lane's 16 * TJ loads
    // are issued back to back and waited for together.
    auto load_cols = [&](float (&dst)[TJ][16], const void* base, int dt, float fill) __attribute__((always_inline)) {
        auto each = [&](auto get) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int n = n_wave + j * 32 + 8 * (e / 4) + (e % 4);
                    dst[j][e] = n < p.N ? get(n) : fill;
                }
        };
        if (dt == GLA_DT_FP32) each([&](int n) { return ((const float*)base)[n]; });
        else if (dt == GLA_DT_BF16) each([&](int n) { return bf16_bits_to_float(((const uint16_t*)base)[n]); });
        else if (dt == GLA_DT_FP16) each([&](int n) { return (float)((const half_t*)base)[n]; });
        else each([&](int n) { return load_as_float(base, dt, n); });
    };
    float sb[TJ][16];
    if (col_scale) {
        load_cols(sb, p.scales, p.meta_dt, 1.0f);
    } else {
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) sb[j][e] = 1.0f;
    }
    // Bias: out = cast(cast(v) + bias[n]) like the reference's `out += bias` on the rounded output
    // (reference: gemlite/core.py:271-272).
    float bb[BIAS ? TJ : 1][16];
    if constexpr (BIAS) load_cols(bb, p.bias, p.bias_dt, 0.0f);
    auto biased = [&](auto dt_tag, float v, int j, int e) __attribute__((always_inline)) -> float {
        if constexpr (BIAS) return round_to_dtype(decltype(dt_tag)::value, v) + bb[j][e];
        else return v;
    };
    auto emit = [&](auto dt_tag) {
        constexpr int DT = decltype(dt_tag)::value;
        constexpr int ES = (DT == GLA_DT_FP16 || DT == GLA_DT_BF16) ? 2 : 4;
        // four elements leave as one 8- or 16-byte store when every such group of the tensor is aligned
        const bool wide = (p.osm & 3) == 0 && (((uintptr_t)p.out) & (4 * ES - 1)) == 0;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int m = m0 + wm * WM + i * 32 + r32;
            if (m >= p.M) continue;
            const float sa = row_scale ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int n = n_wave + j * 32 + 8 * g;
                    const int64_t o = (int64_t)m * p.osm + n;
                    if (wide && n + 3 < p.N) {
                        if constexpr (DT == GLA_DT_INT32) {
                            *(int4_t*)((int32_t*)p.out + o) = int4_t{(int)acc[i][j][4 * g], (int)acc[i][j][4 * g + 1],
                                                                     (int)acc[i][j][4 * g + 2], (int)acc[i][j][4 * g + 3]};
                        } else {
                            float v[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t) v[t] = biased(dt_tag, value(i, j, 4 * g + t) * (sa * sb[j][4 * g + t]), j, 4 * g + t);
                            if constexpr (DT == GLA_DT_FP32) {
                                *(float4_t*)((float*)p.out + o) = float4_t{v[0], v[1], v[2], v[3]};
                            } else {
                                uint32_t lo, hi;
                                if constexpr (DT == GLA_DT_FP16) {
                                    lo = pack_half2(v[0], v[1]);
                                    hi = pack_half2(v[2], v[3]);
                                } else {
                                    lo = pack_bf16x2(v[0], v[1]);
                                    hi = pack_bf16x2(v[2], v[3]);
                                }
                                *(u32x2*)((uint16_t*)p.out + o) = u32x2{lo, hi};
                            }
                        }
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            if (n + t >= p.N) continue;
                            if constexpr (DT == GLA_DT_INT32) ((int32_t*)p.out)[o + t] = (int32_t)acc[i][j][4 * g + t];
                            else store_typed<DT>(p.out, o + t, biased(dt_tag, value(i, j, 4 * g + t) * (sa * sb[j][4 * g + t]), j, 4 * g + t));
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

__device__ __forceinline__ float with_bias(const Gemm8Args& p, int n, float v) {
    if (p.bias == nullptr) return v;
    return round_to_dtype(p.out_dt, v) + load_as_float(p.bias, p.bias_dt, n);
}

// Sum the K splits in order (exactly, for integer accumulators), apply the channel scales and store.
template <bool INT>
__global__ __launch_bounds__(256) void splitk_finish8_kernel(Gemm8Args p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx % p.N);
    const size_t slab = (size_t)p.M * p.N;
    const int64_t o = (int64_t)m * p.osm + n;
    float scale = 1.0f;
    if (p.csm & 1) scale *= load_as_float(p.scales, p.meta_dt, n);
    if (p.csm & 2) scale *= load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm);
    if constexpr (INT) {
        int32_t v = 0;
        for (int s = 0; s < p.S; ++s) v += ((const int32_t*)p.partials)[s * slab + idx];
        if (p.out_dt == GLA_DT_INT32) ((int32_t*)p.out)[o] = v;
        else store_from_float(p.out, p.out_dt, o, with_bias(p, n, (float)v * scale));
    } else {
        float v = 0.0f;
        for (int s = 0; s < p.S; ++s) v += ((const float*)p.partials)[s * slab + idx];
        store_from_float(p.out, p.out_dt, o, with_bias(p, n, v * scale));
    }
}

template <int MODE, int BM, int WN, bool BIAS = false>
int launch_bm(const Gemm8Args& a, hipStream_t stream) {
    if constexpr (!BIAS) {
        // with a bias and an unsplit K the epilogue adds it (a split K leaves it to the finishing kernel)
        if (a.bias != nullptr && a.S == 1 && a.out_dt != GLA_DT_INT32) return launch_bm<MODE, BM, WN, true>(a, stream);
    }
    const size_t smem = (size_t)kRing8 * slot_bytes8(MODE, BM);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = gemm_8bit_kernel<MODE, BM, WN, BIAS>;
    if (once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_8bit: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n, a.S), dim3(kWavesM * WN * 64), smem, stream, a);
    int rc = check_hip(hipGetLastError(), "gemm_8bit launch");
    if (rc == GLA_OK && a.S > 1) {
        const int64_t items = (int64_t)a.M * a.N;
        Gemm8Args f = a;
        if (MODE == kMXFP4 || MODE == kBQF8 || MODE == kBQI8) f.csm = 0;  // block scales were applied in the main kernel
        hipLaunchKernelGGL((splitk_finish8_kernel<MODE == kINT8 || MODE == kINT8R>), dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                           stream, f);
        rc = check_hip(hipGetLastError(), "gemm_8bit split-K reduction launch");
    }
    return rc;
}

template <int MODE>
int launch_mode(const Gemm8Args& a, int bm, hipStream_t stream) {
    if (bm == 256) return launch_bm<MODE, 256, 4>(a, stream);
    if (bm == 128) return launch_bm<MODE, 128, 4>(a, stream);
    return launch_bm<MODE, 64, 4>(a, stream);
}

// tile_config encoding: BM (64, 128 or 256; other = chosen here) + 1000 * K splits (0 = chosen here)
struct Plan8 {
    int bm, tiles_m, tiles_n, S, sps;
};

// MXFP4 scales by pipeline stage.  In the caller's layout ([rows, K/32] bytes, K fastest) the four
// scale bytes a row contributes to a stage lie one row stride apart from the next row's, so the
// copy of a tile's scales touches one cache line per row and moves sixteen times the bytes it uses.
// This kernel regroups them as dst[stage][row] (one 32-bit word each), which a tile copies as
// consecutive words.  64 x 64 words per workgroup through LDS, both sides coalesced.
// blockIdx.z picks the array (0: activations, 1: weights), so that one launch regroups both.
__global__ __launch_bounds__(256) void mx_scales_by_stage_kernel(const uint8_t* src_x, int rows_x, int64_t row_stride_x, uint32_t* dst_x,
                                                                 const uint8_t* src_w, int rows_w, int64_t row_stride_w, uint32_t* dst_w,
                                                                 int stages) {
    __shared__ uint32_t tile[64][65];
    const uint8_t* src = blockIdx.z ? src_w : src_x;
    const int rows = blockIdx.z ? rows_w : rows_x;
    const int64_t row_stride = blockIdx.z ? row_stride_w : row_stride_x;
    uint32_t* dst = blockIdx.z ? dst_w : dst_x;
    const int r0 = blockIdx.x * 64, s0 = blockIdx.y * 64, t = threadIdx.x;
    if (r0 >= rows) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = r0 + (t >> 6) + 4 * i, st = s0 + (t & 63);
        if (r < rows && st < stages) tile[(t >> 6) + 4 * i][t & 63] = *(const uint32_t*)(src + (int64_t)r * row_stride + (int64_t)st * 4);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = r0 + (t & 63), st = s0 + (t >> 6) + 4 * i;
        if (r < rows && st < stages) dst[(int64_t)st * rows + r] = tile[t & 63][(t >> 6) + 4 * i];
    }
}

constexpr int64_t kWsReserved8 = kWsPrivateBytes;  // the start of the workspace belongs to the GEMV family (common.hpp)

Plan8 plan8(int M, int N, int Kb, int tile_config) {
    Plan8 g;
    const int cfg = tile_config > 0 ? tile_config : 0;
    const int bm_asked = cfg % 1000;
    const int total_steps = ceil_div(Kb, kRowB8);
    // per-stage cost of a workgroup (64 bytes of K) by tile height, us, the chip full
    static const int bms[3] = {64, 128, 256};
    static const float cost[3] = {0.53f, 0.66f, 0.85f};
    const TilePick pick = pick_tile_and_split(M, N, kBN, total_steps, 8, 16, bms, cost, 3,
                                              (bm_asked == 64 || bm_asked == 128 || bm_asked == 256) ? bm_asked : 0, cfg / 1000);
    g.bm = pick.bm;
    g.tiles_m = ceil_div(M, g.bm);
    g.tiles_n = ceil_div(N, kBN);
    int want = pick.S;
    if (want > total_steps) want = total_steps;
    if (want < 1) want = 1;
    g.sps = ceil_div(total_steps, want);
    g.S = ceil_div(total_steps, g.sps);
    return g;
}

int attach_plan(const gla_matmul_args& p, const Plan8& g, Gemm8Args& a) {
    a.tiles_m = g.tiles_m; a.tiles_n = g.tiles_n; a.S = g.S; a.sps = g.sps; a.partials = nullptr;
    if (g.S > 1) {
        const int64_t need = kWsReserved8 + (int64_t)g.S * p.M * p.N * 4;
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemm_8bit: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.partials = (char*)p.workspace + kWsReserved8;
    }
    return GLA_OK;
}

}  // namespace

#ifndef GLA_G8_16BIT
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
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if (p.output_dtype == GLA_DT_INT32 && !(i8 && p.channel_scale_mode == GLA_CSM_NONE)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int launch_gemm_8bit(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = 0; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype; a.sx_stage = 0; a.sw_stage = 0; a.ascales = nullptr; a.asxm = 0;
    const Plan8 g = plan8(p.M, p.N, a.Kb, p.tile_config);
    const int rc = attach_plan(p, g, a);
    if (rc != GLA_OK) return rc;
    if (p.input_dtype == GLA_DT_INT8) return a.Kb % kRowB8 ? launch_mode<kINT8R>(a, g.bm, stream) : launch_mode<kINT8>(a, g.bm, stream);
    return launch_mode<kFP8>(a, g.bm, stream);
}

static int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// ---- 128 x 128 block-quantised fp8 / int8 (channel_scale_mode 5) from 2 rows up ----------------
// (reference: gemlite/triton_kernels/gemm_kernels.py:396-400, :441-450.)  Tiles of 64 or 128 rows: the
// second accumulator leaves no registers for the 256-row tile.  K splits hold whole 128-blocks (an even
// number of stages) and their partials are the scaled fp32 sums, which the reduction kernel only adds.
static Plan8 plan_blockq(const gla_matmul_args& p) {
    const int cfg = p.tile_config > 0 ? p.tile_config : 0;
    const int bm_asked = (cfg % 1000 == 64 || cfg % 1000 == 128) ? cfg % 1000 : 0;
    // the same cost model as plan8() over the two tile heights there are (the fold makes a stage dearer)
    static const int bms[2] = {64, 128};
    static const float cost[2] = {0.77f, 0.96f};
    const TilePick pick = pick_tile_and_split(p.M, p.N, kBN, ceil_div(p.K, kRowB8), 8, 16, bms, cost, 2, bm_asked, cfg / 1000);
    Plan8 g = plan8(p.M, p.N, p.K, pick.S * 1000 + pick.bm);
    if (g.S > 1 && (g.sps & 1)) {
        g.sps += 1;
        g.S = ceil_div(ceil_div(p.K, kRowB8), g.sps);
    }
    return g;
}

bool gemm_blockq_eligible(const gla_matmul_args& p) {
    // The streaming kernel keeps the first rows: 2 everywhere (4096^2 11 against 15 us, 16384^2 63-65 against 74;
    // within 7 % either way on 8192^2 and 4096 x 14336), 3 on layers of 20 MB or less and of 200 MB or more (4096^2
    // 13-14.5 against 15-16; 16384^2 62-68 against 74; 8192^2 24-27 against 22)
    const int64_t wbytes = (int64_t)p.N * p.K;
    const int stream_rows = (wbytes <= 20000000 || wbytes >= 200000000) ? 3 : 2;
    if (!blockq_stream_eligible(p) || p.M <= stream_rows || p.out_stride_n != 1) return false;
    if (p.meta_stride_n < 0 || p.meta_stride_g < 0 || p.sx_stride_m < 0 || p.sx_stride_g < 0) return false;
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if ((int64_t)p.M * p.sx_stride_m * 4 >= (1ll << 31) || (int64_t)(p.N / 128 + 1) * p.meta_stride_n * 4 >= (1ll << 31)) return false;
    return true;
}

int64_t gemm_blockq_workspace_bytes(const gla_matmul_args& p) {
    const Plan8 g = plan_blockq(p);
    return g.S > 1 ? kWsReserved8 + align256((int64_t)g.S * p.M * p.N * 4) : 0;
}

int launch_gemm_blockq(const gla_matmul_args& p, hipStream_t stream) {
    if (!gemm_blockq_eligible(p)) {
        set_error("gemm_blockq: operands not eligible (see blockq_stream; more than 1 row, unit output column stride)");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    Gemm8Args a;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    // block scales travel with the stages like micro-scales: byte strides per row / per 128-block of K
    a.scales = p.scales; a.msn = p.meta_stride_n * 4; a.sw_stage = p.meta_stride_g * 4;
    a.ascales = p.scales_x; a.asxm = p.sx_stride_m * 4; a.sx_stage = p.sx_stride_g * 4;
    a.scales_x = nullptr; a.sxm = 0; a.csm = 0;  // nothing left for the epilogue
    a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype; a.out_dt = p.output_dtype;
    const Plan8 g = plan_blockq(p);
    const int rc = attach_plan(p, g, a);
    if (rc != GLA_OK) return rc;
    if (p.input_dtype == GLA_DT_INT8)
        return g.bm == 128 ? launch_bm<kBQI8, 128, 4>(a, stream) : launch_bm<kBQI8, 64, 4>(a, stream);
    return g.bm == 128 ? launch_bm<kBQF8, 128, 4>(a, stream) : launch_bm<kBQF8, 64, 4>(a, stream);
}

// MXFP4 scales regrouped by stage pay off once the GEMM itself takes much longer than regrouping
// the weight scales (a pass over N x K/32 bytes): from the 128-row tile on.
static bool mx_scales_staged(const gla_matmul_args& p, const Plan8& g) { return g.bm >= 128; }

int64_t gemm_8bit_workspace_bytes(const gla_matmul_args& p) {
    const bool mx = p.input_dtype == GLA_DT_MXFP4;
    const Plan8 g = plan8(p.M, p.N, mx ? p.K / 2 : p.K, p.tile_config);
    int64_t need = g.S > 1 ? kWsReserved8 + align256((int64_t)g.S * p.M * p.N * 4) : 0;
    if (mx && mx_scales_staged(p, g)) {
        if (need == 0) need = kWsReserved8;
        need += align256((int64_t)(p.K / 128) * p.M * 4) + align256((int64_t)(p.K / 128) * p.N * 4);
    }
    return need;
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
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if ((int64_t)p.M * p.sx_stride_m >= (1ll << 31) || (int64_t)p.N * p.meta_stride_n >= (1ll << 31)) return false;
    return true;
}

int launch_gemm_mxfp4(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K / 2; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = p.meta_stride_n; a.csm = 0; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype;
    a.sx_stage = 4; a.sw_stage = 4; a.ascales = p.scales_x; a.asxm = p.sx_stride_m;
    const Plan8 g = plan8(p.M, p.N, a.Kb, p.tile_config);
    const int rc = attach_plan(p, g, a);
    if (rc != GLA_OK) return rc;
    // with room in the workspace, both scale arrays are regrouped by stage first (same stream)
    if (mx_scales_staged(p, g) && p.workspace != nullptr && (int64_t)p.workspace_bytes >= gemm_8bit_workspace_bytes(p)) {
        const int stages = p.K / 128;
        const int64_t part = g.S > 1 ? align256((int64_t)g.S * p.M * p.N * 4) : 0;
        uint32_t* sx = (uint32_t*)((char*)p.workspace + kWsReserved8 + part);
        uint32_t* sw = (uint32_t*)((char*)sx + align256((int64_t)stages * p.M * 4));
        const int row_blocks = ceil_div(p.M > p.N ? p.M : p.N, 64);
        hipLaunchKernelGGL(mx_scales_by_stage_kernel, dim3(row_blocks, ceil_div(stages, 64), 2), dim3(256), 0, stream,
                           (const uint8_t*)p.scales_x, p.M, (int64_t)p.sx_stride_m, sx,
                           (const uint8_t*)p.scales, p.N, (int64_t)p.meta_stride_n, sw, stages);
        a.ascales = sx; a.asxm = 4; a.sx_stage = (int64_t)p.M * 4;
        a.scales = sw; a.msn = 4; a.sw_stage = (int64_t)p.N * 4;
    }
    return launch_mode<kMXFP4>(a, g.bm, stream);
}

// MXFP8 weights (fp8-e4m3 codes, one e8m0 scale per 32 values, [N, K/32] with unit stride along K) x
// fp8 activations that carry either the same kind of block scales (channel_scale_mode 4) or one fp32
// scale per row applied after the K sum (channel_scale_mode 2, the reference processor's default:
// gemlite/helper.py:876-923).
bool gemm_mxfp8_eligible(const gla_matmul_args& p) {
    if (p.input_dtype != GLA_DT_MXFP8) return false;
    if (!(p.channel_scale_mode == GLA_CSM_MX || p.channel_scale_mode == GLA_CSM_ACTIVATION)) return false;
    const bool w8 = p.W_nbits == 8 && p.elements_per_sample == 1 && p.w_dtype == GLA_DT_FP8;
    const bool w4 = p.W_nbits == 4 && p.elements_per_sample == 2;  // MXFP4 weights: the mixed fp8 x fp4 MFMA
    if (!(w8 || w4) || p.group_size != 32) return false;
    if (p.scales == nullptr || p.scales_x == nullptr) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    if (p.meta_stride_g != 1 || p.meta_stride_n % 4 != 0 || ((uintptr_t)p.scales & 3)) return false;
    if (p.channel_scale_mode == GLA_CSM_MX && (p.sx_stride_g != 1 || p.sx_stride_m % 4 != 0 || ((uintptr_t)p.scales_x & 3)))
        return false;
    if (p.K % 128 != 0 || p.x_stride_m % 16 != 0 || p.w_stride_n % 16 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)p.N * p.w_stride_n >= (1ll << 31)) return false;
    if ((int64_t)p.M * p.sx_stride_m >= (1ll << 31) || (int64_t)p.N * p.meta_stride_n >= (1ll << 31)) return false;
    return true;
}

// with block scales on both sides the 256-row tile has no registers for the scale words next to two
// fragment buffers of 8-register operands
// Left to choose, short batches on very large MXFP4 layers take the 128-row tile too: it reads the scales regrouped
// by stage (a launch of its own), the 64-row tile reads them where the caller keeps them (weights rotated, M=8:
// 16384^2 MXFP4 weights 54 against 64 us, MXFP8 weights 87 against 84; 8192^2 28 against 24 and 33 against 27;
// 4096^2 20 against 15.5 and 20 against 15).
static Plan8 plan_mxfp8(const gla_matmul_args& p) {
    Plan8 g = plan8(p.M, p.N, p.K, p.tile_config);
    const int asked = p.tile_config > 0 ? p.tile_config % 1000 : 0;
    const bool chosen_here = !(asked == 64 || asked == 128 || asked == 256);
    const bool large_fp4 = p.elements_per_sample == 2 && (int64_t)p.N * p.K >= 100000000;
    if ((g.bm == 256 && p.channel_scale_mode == GLA_CSM_MX) || (g.bm == 64 && chosen_here && large_fp4)) {
        const int cfg = (p.tile_config > 0 ? p.tile_config / 1000 : 0) * 1000 + 128;
        g = plan8(p.M, p.N, p.K, cfg);
    }
    return g;
}

int64_t gemm_mxfp8_workspace_bytes(const gla_matmul_args& p) {
    const Plan8 g = plan_mxfp8(p);
    int64_t need = g.S > 1 ? kWsReserved8 + align256((int64_t)g.S * p.M * p.N * 4) : 0;
    if (g.bm >= 128) {
        if (need == 0) need = kWsReserved8;
        need += align256((int64_t)(p.K / 128) * p.M * 4) + align256((int64_t)(p.K / 128) * p.N * 4);
    }
    return need;
}

int launch_gemm_mxfp8(const gla_matmul_args& p, hipStream_t stream) {
    Gemm8Args a;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    const bool act_blocks = p.channel_scale_mode == GLA_CSM_MX;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K; a.lda = p.x_stride_m; a.ldb = p.w_stride_n; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = p.meta_stride_n; a.sw_stage = 4;
    a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype; a.out_dt = p.output_dtype;
    a.csm = act_blocks ? 0 : 2;  // per-token scale in the epilogue
    // without activation block scales the copy jobs for them re-read the first weight scale word (never used)
    a.ascales = act_blocks ? p.scales_x : p.scales;
    a.asxm = act_blocks ? p.sx_stride_m : 0;
    a.sx_stage = act_blocks ? 4 : 0;
    const Plan8 g = plan_mxfp8(p);
    const int rc = attach_plan(p, g, a);
    if (rc != GLA_OK) return rc;
    if (g.bm >= 128 && p.workspace != nullptr && (int64_t)p.workspace_bytes >= gemm_mxfp8_workspace_bytes(p)) {
        const int words = p.K / 128;
        const int64_t part = g.S > 1 ? align256((int64_t)g.S * p.M * p.N * 4) : 0;
        uint32_t* sx = (uint32_t*)((char*)p.workspace + kWsReserved8 + part);
        uint32_t* sw = (uint32_t*)((char*)sx + align256((int64_t)words * p.M * 4));
        const int rows_x = act_blocks ? p.M : 0;
        const int row_blocks = ceil_div(rows_x > p.N ? rows_x : p.N, 64);
        hipLaunchKernelGGL(mx_scales_by_stage_kernel, dim3(row_blocks, ceil_div(words, 64), 2), dim3(256), 0, stream,
                           (const uint8_t*)p.scales_x, rows_x, (int64_t)p.sx_stride_m, sx,
                           (const uint8_t*)p.scales, p.N, (int64_t)p.meta_stride_n, sw, words);
        a.scales = sw; a.msn = 4; a.sw_stage = (int64_t)p.N * 4;
        if (act_blocks) { a.ascales = sx; a.asxm = 4; a.sx_stage = (int64_t)p.M * 4; }
        else { a.ascales = sw; }
    }
    if (p.elements_per_sample == 2) return act_blocks ? launch_mode<kMX84>(a, g.bm, stream) : launch_mode<kMX84T>(a, g.bm, stream);
    return act_blocks ? launch_mode<kMXFP8>(a, g.bm, stream) : launch_mode<kMXFP8T>(a, g.bm, stream);
}

#else  // GLA_G8_16BIT

// ---- unquantised layers: fp16 x fp16 / bf16 x bf16, weights [N, K] with K contiguous (W_nbits = 16) ----------------
// (reference: the same `tl.dot` GEMM with the unpacking switched off, gemlite/triton_kernels/gemm_kernels.py:285-496)
bool gemm_16bit_eligible(const gla_matmul_args& p) {
    const bool h = p.input_dtype == GLA_DT_FP16 && p.w_dtype == GLA_DT_FP16, b = p.input_dtype == GLA_DT_BF16 && p.w_dtype == GLA_DT_BF16;
    if (!h && !b) return false;
    if (p.elements_per_sample != 1 || p.W_nbits != 16 || p.W_group_mode != GLA_WGM_NONE || p.acc_dtype != GLA_DT_FP32) return false;
    if (p.channel_scale_mode < GLA_CSM_NONE || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (p.w_stride_k != 1 || p.x_stride_k != 1 || p.out_stride_n != 1) return false;
    // rows of whole 16-byte chunks, K in whole stages of 32 values
    if (p.K % 32 != 0 || p.x_stride_m % 8 != 0 || p.w_stride_n % 8 != 0) return false;
    if (((uintptr_t)p.x & 15) || ((uintptr_t)p.w & 15)) return false;
    if ((int64_t)p.M * p.x_stride_m * 2 >= (1ll << 31) || (int64_t)p.N * p.w_stride_n * 2 >= (1ll << 31)) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int64_t gemm_16bit_workspace_bytes(const gla_matmul_args& p) {
    const Plan8 g = plan8(p.M, p.N, p.K * 2, p.tile_config);
    return g.S > 1 ? kWsReserved8 + (int64_t)g.S * p.M * p.N * 4 : 0;
}

int launch_gemm_16bit(const gla_matmul_args& p, hipStream_t stream) {
    if (!gemm_16bit_eligible(p)) {
        set_error("gemm_16bit: fp16 x fp16 or bf16 x bf16, both K-contiguous with 16-byte aligned rows, K a multiple of 32");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    Gemm8Args a;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.a = (const uint8_t*)p.x; a.b = (const uint8_t*)p.w; a.scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N; a.Kb = p.K * 2; a.lda = p.x_stride_m * 2; a.ldb = p.w_stride_n * 2; a.osm = p.out_stride_m;
    a.sxm = p.sx_stride_m; a.msn = 0; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.sx_dt = p.sx_dtype;
    a.out_dt = p.output_dtype; a.sx_stage = 0; a.sw_stage = 0; a.ascales = nullptr; a.asxm = 0;
    const Plan8 g = plan8(p.M, p.N, a.Kb, p.tile_config);
    const int rc = attach_plan(p, g, a);
    if (rc != GLA_OK) return rc;
    if (p.input_dtype == GLA_DT_BF16) return launch_mode<kB16>(a, g.bm, stream);
    return launch_mode<kH16>(a, g.bm, stream);
}

#endif

}  // namespace gla
