// MFMA GEMM for fp16/bf16 activations x 32-bit packed low-bit weights stored [K/e, N], N fastest:
// out[M,N] = x[M,K] * dequant(W)[K,N], dequantisation fused into the B-operand path.  The prefill
// and mid-batch path of A16W4 / A16W8 / A16W2 layers.
//
// Takes the place of the reference's GPTQ-style GEMM and of its split-K GEMM (reference:
// gemlite/triton_kernels/gemm_kernels.py:285-496,
// gemlite/triton_kernels/gemm_splitK_kernels.py:300-523; dequant
// gemlite/triton_kernels/utils.py:73-105).
//
//  * Workgroup tile BM x 256 with BM = 32, 64, 128 or 256, K step 64, v_mfma_f32_32x32x16 tiles.
//    Four wave columns of 64 at every height: BM <= 128 is one wave row of BM x 64 wave tiles
//    (4 waves), BM = 256 two wave rows of 128 x 64 (8 waves).  Every wave unpacks the weights of
//    its own columns, so wave rows repeat that work and wave columns divide it; the unpacking,
//    not the MFMA, bounds the short tiles.
//  * Every operand of a stage (activation tile, packed weight words, scales, zeros) is copied
//    global -> LDS by the load unit (global_load_lds) into a ring of 3 or 4 stages; the K loop
//    loads nothing into registers from global memory and waits on the vector-memory counter only
//    where it says so.  Activation rows are dense 128-byte rows whose 16-byte chunks are
//    XOR-swizzled by (row >> 1) & 7.  A weight copy job moves 128 columns x both K-halves' word
//    rows, 16 bytes (4 adjacent columns) per lane; with column tiles interleaved ({TJ r + j}) a
//    lane reads the words of all its column tiles in one LDS access.
//  * Unpacking: one v_perm replicates the byte (pair of bytes) that holds two adjacent codes into
//    both 16-bit halves, a masked OR puts each code into the mantissa of a power of two whose
//    last-place unit matches the code's bit position (1024 + q, 256 + q, 64 + q, 16 + q), and
//    (t - offset) * s + z' runs in packed fp16.  Adjacent codes land in adjacent K-slots, so
//    the activation fragment is used as it lies in memory.  bf16 activations: codes paired (j, j+4)
//    in the mantissa of 128.0, fp32 fma, one packed round-to-nearest-even conversion (byte codes:
//    direct byte-to-float conversion); the activation fragment is reordered to match (v_perm).
//    2-bit codes on bf16: the four dequantised values of a column and group are made once per group and a
//    code pair picks its two with one byte permute (4 instructions per pair instead of 7; identical bits).
//  * The weights are the row operand of the MFMA: an accumulator is the transposed output tile and
//    a lane holds 4 TJ adjacent output columns of one row, stored 16 bytes at a time.
//  * When the output has too few tiles to fill the chip (small M), K is split over gridDim.y:
//    every split writes an fp32 partial tile to the workspace and a second small kernel on the
//    same stream sums the splits in order, applies the channel scales and stores the output
//    (deterministic, no float atomics, output need not be zeroed).
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"
#include "wn_dequant.hpp"

namespace gla {

namespace {

constexpr int kBKw = 64;    // K per pipeline stage
constexpr int kRowW = 128;  // LDS row: 64 fp16/bf16 values
constexpr int kBNw = 256;   // workgroup tile columns: 256 / (32 TJ) wave columns of TJ 32-column MFMA tiles
constexpr int64_t kWsReserved = kWsPrivateBytes;  // the start of the workspace belongs to the GEMV family (common.hpp)

struct GemmWnArgs {
    const uint16_t* x;
    const uint32_t* w;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    int M, N, K;
    int gs;  // K-values per quantisation group (K when ungrouped)
    int64_t xsm, wsk, osm, msg, sxm;
    int wgm, csm, meta_dt, z_dt, z_scalar, out_dt, sx_dt;
    int tiles_m, tiles_n;
    int S;    // K splits (gridDim.y)
    int sps;  // pipeline stages per split
    float* partials;  // [S][M][N] when S > 1
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
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

template <bool BF16>
__device__ __forceinline__ float16_t mfma32(const u32x4& a, const u32x4& b, float16_t c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}

// s_waitcnt vmcnt(N) only: vmcnt is bits 3:0 and 15:14, expcnt (6:4) and lgkmcnt (11:8) left at "no wait"
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// LDS ring of pipeline stages: as many as fit with two workgroups per CU where the tile is small.
constexpr int ring_slots(int bm) { return bm >= 128 ? 3 : 4; }
// One ring slot: A tile, weight words of both wave columns, scales and zeros of the 256 columns.
constexpr int slot_bytes(int bits, int bm) { return bm * kRowW + 2 * (bits == 8 ? 8 : 4) * 1024 + 1024; }

// BITS in {2, 4, 8}; WAVES_M in {1, 2, 4}; TI = 32-row MFMA tiles per wave (1, 2 or 4); TJ = 32-column
// tiles per wave (4 or 2; the launcher uses 2 throughout).  Every wave dequantises the weights of
// its own columns, so the work of unpacking is repeated WAVES_M times per workgroup and divided by
// the number of wave columns.
template <int BITS, bool BF16, int WAVES_M, int TI, int TJ>
__global__ __launch_bounds__(WAVES_M * (8 / TJ) * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_wn_kernel(GemmWnArgs p) {
    static_assert(TJ == 4 || TJ == 2, "wave tile of 128 or 64 columns");
    constexpr int E = 32 / BITS;
    constexpr int WM = 32 * TI;
    constexpr int BM = WAVES_M * WM;
    constexpr int WN = 8 / TJ;               // wave columns
    constexpr int NW = WAVES_M * WN;         // waves
    constexpr int WL = (BITS == 8) ? 8 : 4;  // 128-bit weight loads per lane per stage
    constexpr int RING = ring_slots(BM);
    constexpr int SLOT = slot_bytes(BITS, BM);
    constexpr int W_OFF = BM * kRowW, S_OFF = W_OFF + 2 * WL * 1024, Z_OFF = S_OFF + 512;
    constexpr int A_JOBS = BM / 8;           // 16-byte copy instructions for the A tile (8 rows each)
    constexpr int JOBS16 = A_JOBS + 2 * WL;  // ... and for the weight words (one per load per wave column)
    constexpr int J16 = (JOBS16 + NW - 1) / NW;  // per wave
    constexpr int J4 = (4 + NW - 1) / NW;        // 4-byte copy instructions per wave: scales / zeros x 2 wave columns
    constexpr int LPS = J16 + J4;                // copy instructions per wave per stage
    constexpr uint32_t kPairMask = ((1u << BITS) - 1u) * 0x00010001u;
    constexpr uint32_t kMagic = BF16 ? 0x43004300u : 0x64006400u;
    // fp16 (and bf16 with byte codes) unpack adjacent codes into adjacent K-slots, so the activation
    // chunks are used as they lie; the other bf16 cases pair code j with j + 4 (j + 8) and reorder
    // the activation chunk to match
    constexpr bool NATURAL = !BF16 || BITS == 8;
    static_assert(RING * LPS < 64, "outstanding copies must fit the vmcnt counter");

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int r32 = lane & 31, kb = lane >> 5;
    int tm, tn;
    tile_coords_wn(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * kBNw;
    // the wave's columns start at n_wave; as B operand of tile j the lane handles column n_wave + TJ r32 + j
    const int n_wave = n0 + wn * 32 * TJ;

    const bool grouped = p.wgm >= GLA_WGM_SCALE || (p.wgm == GLA_WGM_SHIFT && !p.z_scalar);
    const bool has_s = p.wgm >= GLA_WGM_SCALE;
    const bool has_zt = (p.wgm == GLA_WGM_SHIFT || p.wgm >= GLA_WGM_SHIFT_SCALE) && !p.z_scalar;
    const float z_const = ((p.wgm == GLA_WGM_SHIFT || p.wgm >= GLA_WGM_SHIFT_SCALE) && p.z_scalar)
                              ? load_as_float(p.zeros, p.z_dt, 0) : 0.0f;

    // ---- copy plan.  Every operand of a stage reaches LDS through global_load_lds: nothing in the
    // K loop loads into registers from global memory, so the only waits on the vector-memory
    // counter are the explicit ones below.  Job q = wave + NW i of a stage (wave-uniform):
    //   q < A_JOBS          rows 8q..8q+7 of the A tile; lane (row l/8, position l%8) fetches the
    //                       chunk that belongs at that position of the swizzled row;
    //   otherwise           load u of wave column c: every lane fetches its own 16 bytes (4 adjacent
    //                       columns of one word row) into a slot only it and its peers in the other
    //                       wave rows read back.
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
            dst16[i] = q * 8 * kRowW;
        } else {
            const int c = (q - A_JOBS) / WL, u = (q - A_JOBS) % WL;
            int col = n0 + c * 128 + r32 * 4;
            if (col > p.N - 4) col = p.N - 4;
            int row;
            if constexpr (BITS == 8) row = 4 * (u / 2) + 2 * kb + (u % 2);  // K-step u/2: rows 4s + 2kb + {0,1}
            else if constexpr (BITS == 4) row = 2 * u + kb;                 // K-step u: row 2s + kb
            else row = u;                                                   // K-step u: row s (both K-halves read it)
            off16[i] = (unsigned)(col + row * (int)p.wsk) * 4u;
            dst16[i] = W_OFF + (c * WL + u) * 1024;
        }
    }
    // scales / zeros: job (kind, c) copies the 128 values of wave column c, one dword (2 columns) per lane
    unsigned off4[J4];
    int dst4[J4];
    bool is_z4[J4];
#pragma unroll
    for (int i = 0; i < J4; ++i) {
        int q = wave + NW * i;
        if (q > 3) q = 3;
        is_z4[i] = q >= 2;
        const int c = q & 1;
        int col = n0 + c * 128 + 2 * lane;
        if (col > p.N - 2) col = p.N - 2;
        const bool present = is_z4[i] ? has_zt : has_s;
        off4[i] = present ? (unsigned)col * 2u : 0u;  // absent: every lane reads the first dword of the weights
        dst4[i] = (is_z4[i] ? Z_OFF : S_OFF) + c * 256;
    }
    const unsigned char* s_base = has_s ? (const unsigned char*)p.scales : (const unsigned char*)p.w;
    const unsigned char* z_base = has_zt ? (const unsigned char*)p.zeros : (const unsigned char*)p.w;
    const int64_t s_stride = has_s ? p.msg * 2 : 0, z_stride = has_zt ? p.msg * 2 : 0;  // bytes per group
    const int64_t w_stage = (int64_t)(kBKw / E) * p.wsk * 4;                              // bytes per stage

    auto issue = [&](int kk, int g, int slot) __attribute__((always_inline)) {
        unsigned char* base = smem + slot * SLOT;
        const unsigned char* xk = (const unsigned char*)p.x + (int64_t)kk * (kBKw * 2);
        const unsigned char* wk = (const unsigned char*)p.w + kk * w_stage;
#pragma unroll
        for (int i = 0; i < J16; ++i) {
            const unsigned char* src = (is_a16[i] ? xk : wk) + off16[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + dst16[i]), 16, 0, 0);
        }
        const unsigned char* sk = s_base + g * s_stride;
        const unsigned char* zk = z_base + g * z_stride;
#pragma unroll
        for (int i = 0; i < J4; ++i) {
            const unsigned char* src = (is_z4[i] ? zk : sk) + off4[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                             (__attribute__((address_space(3))) void*)(base + dst4[i]), 4, 0, 0);
        }
    };

    // ---- dequant constants: branch-free; absent scales / zeros are masked to 0 and replaced by
    // constants, and the zero-point term of every dequant mode is z * (c1 + c2 * s)
    const bool meta_bf16 = p.meta_dt == GLA_DT_BF16;
    const uint32_t s_mask = has_s ? 0xffffu : 0u, z_mask = has_zt ? 0xffffu : 0u;
    const float s_add = has_s ? 0.0f : 1.0f, z_add = has_zt ? 0.0f : z_const;
    const float c1 = p.wgm == GLA_WGM_SHIFT ? -1.0f : (p.wgm == GLA_WGM_FMA ? 1.0f : 0.0f);
    const float c2 = p.wgm == GLA_WGM_SHIFT_SCALE ? -1.0f : 0.0f;
    ColMeta<BF16> meta[TJ];
    auto convert_meta = [&](const unsigned char* sp, const unsigned char* zp) __attribute__((always_inline)) {
        uint32_t raw_s[TJ / 2], raw_z[TJ / 2];
        if constexpr (TJ == 4) {
            const u32x2 a = *(const u32x2*)sp, b = *(const u32x2*)zp;
            raw_s[0] = a.x; raw_s[1] = a.y; raw_z[0] = b.x; raw_z[1] = b.y;
        } else {
            raw_s[0] = *(const uint32_t*)sp; raw_z[0] = *(const uint32_t*)zp;
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
            const uint32_t sv = (raw_s[j / 2] >> (16 * (j & 1))) & s_mask;
            const uint32_t zv = (raw_z[j / 2] >> (16 * (j & 1))) & z_mask;
            const float s_h = half_bits_to_float((uint16_t)sv), s_b = __builtin_bit_cast(float, sv << 16);
            const float z_h = half_bits_to_float((uint16_t)zv), z_b = __builtin_bit_cast(float, zv << 16);
            const float s = (meta_bf16 ? s_b : s_h) + s_add;
            const float z = (meta_bf16 ? z_b : z_h) + z_add;
            meta[j] = make_meta<BF16, (BITS == 8 ? 0 : 128)>(s, z * __builtin_fmaf(c2, s, c1));
            if constexpr (BF16 && BITS == 2) {
                // a 2-bit code has four values per column and group: dequantise them once (same arithmetic as
                // dequant_pair: (128 + q) s + (z' - 128 s) in fp32, one round-to-nearest-even conversion) ...
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                const f32x2 w01 = {__builtin_fmaf(128.0f, meta[j].s, meta[j].z), __builtin_fmaf(129.0f, meta[j].s, meta[j].z)};
                const f32x2 w23 = {__builtin_fmaf(130.0f, meta[j].s, meta[j].z), __builtin_fmaf(131.0f, meta[j].s, meta[j].z)};
                meta[j].lut01 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w01, bf16x2_t));
                meta[j].lut23 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w23, bf16x2_t));
            }
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
    // natural-order unpacking (fp16): mask and magic of a code pair that shares a byte
    uint32_t nat_mask0 = BITS == 4 ? 0x00F0000Fu : 0x000C0003u, nat_magic0 = BITS == 4 ? 0x54006400u : 0x5C006400u;
    uint32_t nat_mask1 = 0x00C00030u, nat_magic1 = 0x4C005400u;
    asm volatile("" : "+s"(nat_mask0), "+v"(nat_magic0), "+s"(nat_mask1), "+v"(nat_magic1));
    // 2-bit: the lane's eight codes are bytes 2kb and 2kb + 1 of the word
    const uint32_t sel2_lo = 0x0c000c00u | ((2 * kb) << 16) | (2 * kb), sel2_hi = 0x0c000c00u | ((2 * kb + 1) << 16) | (2 * kb + 1);

    const int sw = (r32 >> 1) & 7;  // chunk swizzle of this lane's rows (tile offsets are multiples of 32)
    const int a_row0 = (wm * WM + r32) * kRowW;
    // weight words: a copy job holds 128 columns x the word rows of both K-halves, 16 bytes (4 columns) per copying lane
    const int w_lane = TJ == 4 ? W_OFF + wn * WL * 1024 + lane * 16
                               : W_OFF + (wn >> 1) * WL * 1024 + (kb * 32 + (wn & 1) * 16 + (r32 >> 1)) * 16 + (r32 & 1) * 8;
    const int m_lane = wn * 64 * TJ + r32 * 2 * TJ;
    const int total_steps = p.K / kBKw;
    const int k_first = blockIdx.y * p.sps;  // first stage of this split
    const int steps = (total_steps - k_first) < p.sps ? (total_steps - k_first) : p.sps;
    const int kk_last = k_first + steps - 1;
    const int spg = p.gs / kBKw;  // stages per group, >= 1 (checked on the host)
    const int g_last = grouped ? kk_last / spg : 0;

    // stage to copy next and its quantisation group, advanced without a division; past the end of
    // the split the last stage is copied again so that every step issues the same number of copies
    int ik = k_first, ig = grouped ? k_first / spg : 0, ic = grouped ? k_first % spg : 0;
    auto issue_next = [&](int slot) __attribute__((always_inline)) {
        issue(ik < kk_last ? ik : kk_last, ig < g_last ? ig : g_last, slot);
        ++ik;
        ++ic;
        if (ic == spg) {
            ic = 0;
            ++ig;
        }
    };

    // ---- pipeline.  RING stages are in flight.  The loop is software-pipelined twice over:
    //  * inside a stage, while the MFMAs of K-step s run, the LDS reads of K-step s+1 return and its
    //    operands are unpacked, one MFMA to every few VALU instructions (left to itself the compiler
    //    unpacks, then multiplies; the waves of a workgroup run in phase, so matrix pipe and VALU
    //    would take turns);
    //  * across stages, the barrier that publishes stage k+1 stands before the last K-step of
    //    stage k, whose MFMAs then cover the conversion of stage k+1's scales and zeros and the
    //    unpacking of its first K-step.  By then every wave has read all it needs of stage k, so
    //    the copies of stage k+RING go to that slot right after the barrier.
    // Copies complete in issue order.  The barrier is bare on purpose: __syncthreads() carries a
    // release fence, which for copies into LDS means draining the whole counter and with it the
    // pipeline.  The empty asm statements keep the compiler from moving LDS accesses across it.
    struct Raw {
        u32x4 a[TI];                       // activation chunk(s) of the lane's row in each row tile
        uint32_t w[BITS == 8 ? 2 : 1][TJ]; // weight words of the lane's column in each column tile
    };
    struct Ops {
        u32x4 af[TI], bq[TJ];
    };
    auto read_raw = [&](const unsigned char* base, int s, Raw& r) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const unsigned char* row = base + a_row0 + i * 32 * kRowW;
            if constexpr (BITS == 2 && !NATURAL) {
                // a word holds 16 K-values; half kb unpacks slots (j, j + 8), j = 4kb .. 4kb+3
                const u32x2 lo = *(const u32x2*)(row + (((2 * s) ^ sw) << 4) + 8 * kb);
                const u32x2 hi = *(const u32x2*)(row + (((2 * s + 1) ^ sw) << 4) + 8 * kb);
                r.a[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
            } else {
                r.a[i] = *(const u32x4*)(row + (((2 * s + kb) ^ sw) << 4));
            }
        }
        auto load_words = [&](int v, int u) __attribute__((always_inline)) {
            if constexpr (TJ == 4) {
                const u32x4 t = *(const u32x4*)(base + w_lane + u * 1024);
                r.w[v][0] = t.x; r.w[v][1] = t.y; r.w[v][2] = t.z; r.w[v][3] = t.w;
            } else {
                const u32x2 t = *(const u32x2*)(base + w_lane + u * 1024);
                r.w[v][0] = t.x; r.w[v][1] = t.y;
            }
        };
        if constexpr (BITS == 8) {
            load_words(0, 2 * s);
            load_words(1, 2 * s + 1);
        } else {
            load_words(0, s);
        }
    };
    auto unpack = [&](const Raw& r, Ops& o) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const u32x4 v = r.a[i];
            if constexpr (NATURAL) o.af[i] = v;
            else o.af[i] = pair_order(v.x, v.y, v.z, v.w);  // slots (j, j + 4), or (j, j + 8) for 2-bit codes
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t t;
                if constexpr (BITS == 8 && BF16) {
                    // 128 + q is not exact in bf16 above 127: convert bytes 2(q%2) and 2(q%2) + 1 of the
                    // word to fp32 directly, scale there and pack once
                    const uint32_t w = r.w[q / 2][j];
                    typedef float f32x2 __attribute__((ext_vector_type(2)));
                    const f32x2 f = {__builtin_fmaf((float)((w >> ((q % 2) * 16)) & 0xffu), meta[j].s, meta[j].z),
                                     __builtin_fmaf((float)((w >> ((q % 2) * 16 + 8)) & 0xffu), meta[j].s, meta[j].z)};
                    o.bq[j][q] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
                } else if constexpr (NATURAL) {
                    // fp16: register q gets the adjacent codes 2q and 2q+1 of the lane's eight, which
                    // share a byte (4-, 2-bit) or are adjacent bytes: one v_perm puts that byte (those
                    // bytes) into both halves, the mask keeps one code per half where it lies, and each
                    // half's magic exponent is the one whose unit in the last place matches the code's
                    // position: 1024 + q for bits 0.., 256 + q for bits 2.., 64 + q for bits 4.., 16 + q for bits 6..
                    if constexpr (BITS == 8) {
                        const uint32_t u = __builtin_amdgcn_perm(r.w[q / 2][j], r.w[q / 2][j], q % 2 ? 0x0c030c02u : 0x0c010c00u);
                        t = u | 0x64006400u;
                        o.bq[j][q] = dequant_pair<BF16>(t, meta[j]);
                    } else if constexpr (BITS == 4) {
                        const uint32_t u = __builtin_amdgcn_perm(r.w[0][j], r.w[0][j], 0x0c000c00u | (q << 16) | q);
                        t = (u & nat_mask0) | nat_magic0;
                        o.bq[j][q] = dequant_pair<BF16>(t, meta[j], 1024.0f, 64.0f);
                    } else {
                        const uint32_t u = __builtin_amdgcn_perm(r.w[0][j], r.w[0][j], q / 2 ? sel2_hi : sel2_lo);
                        if (q % 2 == 0) {
                            t = (u & nat_mask0) | nat_magic0;
                            o.bq[j][q] = dequant_pair<BF16>(t, meta[j], 1024.0f, 256.0f);
                        } else {
                            t = (u & nat_mask1) | nat_magic1;
                            o.bq[j][q] = dequant_pair<BF16>(t, meta[j], 64.0f, 16.0f);
                        }
                    }
                } else {
                    if constexpr (BITS == 4) {
                        t = ((r.w[0][j] >> (q * 4)) & pair_mask) | magic;
                        o.bq[j][q] = dequant_pair<BF16>(t, meta[j]);
                    } else {
                        // ... and pick them per code pair with one byte permute: selector bytes (2q, 2q + 1) of each
                        // code, made from the pair (q_lo, q_hi << 16) by one 24-bit multiply-add
                        t = (r.w[0][j] >> ((4 * kb + q) * 2)) & pair_mask;
                        const uint32_t sel = __umul24(t, 0x0202u) + 0x01000100u;
                        o.bq[j][q] = __builtin_amdgcn_perm(meta[j].lut23, meta[j].lut01, sel);
                    }
                }
            }
        }
    };
#pragma unroll
    for (int u = 0; u < RING; ++u) issue_next(u);
    Raw raw;
    Ops ops[2];
    wait_vmcnt<(RING - 1) * LPS>();  // stage 0 has landed (this wave's part)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();    // ... and everybody else's
    asm volatile("" ::: "memory");
    convert_meta(smem + S_OFF + m_lane, smem + Z_OFF + m_lane);
    read_raw(smem, 0, raw);
    unpack(raw, ops[0]);

    constexpr int NMF = TI * TJ;                                     // MFMAs of a K-step
    constexpr int NVA = (NATURAL ? 0 : 4 * TI) + 16 * TJ;            // VALU instructions of an unpacking, roughly
    constexpr int NRD = TI * (BITS == 2 && !NATURAL ? 2 : 1) + (BITS == 8 ? 2 : 1);  // LDS reads of a K-step
    int slot = 0;  // ring slot of the stage being multiplied
#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
        const unsigned char* base = smem + slot * SLOT;
        const int next = slot == RING - 1 ? 0 : slot + 1;
        const unsigned char* nbase = smem + next * SLOT;
        auto kstep = [&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value;
            if constexpr (s == 3) {
                // stage k+1 has landed once at most the copies of the RING - 2 stages after it are outstanding
                wait_vmcnt<(RING - 2) * LPS>();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                issue_next(slot);  // stage k + RING
                __builtin_amdgcn_sched_barrier(0);
                read_raw(nbase, 0, raw);
            } else {
                read_raw(base, s + 1, raw);
            }
#pragma unroll
            for (int j = 0; j < TJ; ++j)
#pragma unroll
                for (int i = 0; i < TI; ++i) acc[i][j] = mfma32<BF16>(ops[s & 1].bq[j], ops[s & 1].af[i], acc[i][j]);  // weights are the row operand
            if constexpr (s == 3) convert_meta(nbase + S_OFF + m_lane, nbase + Z_OFF + m_lane);
            unpack(raw, ops[(s + 1) & 1]);
            __builtin_amdgcn_sched_group_barrier(0x100, NRD + (s == 3 ? 2 : 0), 0);  // the LDS reads first
#pragma unroll
            for (int q = 0; q < NMF; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (NVA + (s == 3 ? 16 * TJ : 0) + NMF - 1) / NMF, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        kstep(std::integral_constant<int, 0>{});
        kstep(std::integral_constant<int, 1>{});
        kstep(std::integral_constant<int, 2>{});
        kstep(std::integral_constant<int, 3>{});
        slot = next;
    }

    // ---- epilogue.  With the weights as row operand an accumulator is the transposed output tile:
    // the lane holds output row r32 of tile i and, in elements 4g .. 4g+3 of tile j, the columns
    // n_wave + TJ (8g + 4kb + t) + j, t = 0..3.  Over t and j these are 4 TJ adjacent columns.
    constexpr int RUN = 4 * TJ;
    if (p.S > 1) {  // partial tile; the reduction kernel finishes
        float* part = p.partials + (size_t)blockIdx.y * p.M * p.N;
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int m = m0 + wm * WM + i * 32 + r32;
            if (m >= p.M) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = n_wave + TJ * (8 * g + 4 * kb);
#pragma unroll
                for (int c = 0; c < RUN; c += 4) {  // N % 4 == 0: a group of four columns is all-in or all-out
                    if (col + c + 3 >= p.N) continue;
                    float v[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) v[q] = acc[i][(c + q) % TJ][4 * g + (c + q) / TJ];
                    *(float4_t*)(part + (size_t)m * p.N + col + c) = float4_t{v[0], v[1], v[2], v[3]};
                }
            }
        }
        return;
    }
    const bool row_scale = (p.csm & 2) != 0;
    auto emit = [&](auto dt_tag) __attribute__((always_inline)) {
        constexpr int DT = decltype(dt_tag)::value;
        constexpr int ES = DT == GLA_DT_FP32 ? 4 : 2;
        // 16-byte stores when every group of 16 / ES elements of the tensor that starts at a multiple of that is aligned
        const bool wide = (((uintptr_t)p.out) & 15) == 0 && ((p.osm * ES) & 15) == 0;
        float sa[TI];
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int m = m0 + wm * WM + i * 32 + r32;
            sa[i] = (row_scale && m < p.M) ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = n_wave + TJ * (8 * g + 4 * kb);
            float sb[RUN];
#pragma unroll
            for (int c = 0; c < RUN; ++c) sb[c] = ((p.csm & 1) && col + c < p.N) ? load_as_float(p.scales, p.meta_dt, col + c) : 1.0f;
            float bv[RUN];
#pragma unroll
            for (int c = 0; c < RUN; ++c) bv[c] = (p.bias != nullptr && col + c < p.N) ? load_as_float(p.bias, p.bias_dt, col + c) : 0.0f;
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                const int m = m0 + wm * WM + i * 32 + r32;
                if (m >= p.M) continue;
                float v[RUN];
#pragma unroll
                for (int c = 0; c < RUN; ++c) v[c] = acc[i][c % TJ][4 * g + c / TJ] * (sa[i] * sb[c]);
                if (p.bias != nullptr) {  // `out += bias` on the rounded output
#pragma unroll
                    for (int c = 0; c < RUN; ++c) v[c] = round_to_dtype(DT, v[c]) + bv[c];
                }
                const int64_t o = (int64_t)m * p.osm + col;
                constexpr int PER = 16 / ES;  // elements per 16-byte store
#pragma unroll
                for (int c = 0; c < RUN; c += PER) {
                    if (wide && col + c + PER - 1 < p.N) {
                        if constexpr (DT == GLA_DT_FP32) {
                            *(float4_t*)((float*)p.out + o + c) = float4_t{v[c], v[c + 1], v[c + 2], v[c + 3]};
                        } else {
                            u32x4 w;
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                if constexpr (DT == GLA_DT_FP16)
                                    w[q] = pack_half2(v[c + 2 * q], v[c + 2 * q + 1]);
                                else
                                    w[q] = pack_bf16x2(v[c + 2 * q], v[c + 2 * q + 1]);
                            }
                            *(u32x4*)((uint16_t*)p.out + o + c) = w;
                        }
                    } else {
#pragma unroll
                        for (int q = 0; q < PER; ++q)
                            if (col + c + q < p.N) store_typed<DT>(p.out, o + c + q, v[c + q]);
                    }
                }
            }
        }
    };
    if (p.out_dt == GLA_DT_FP16) emit(std::integral_constant<int, GLA_DT_FP16>{});
    else if (p.out_dt == GLA_DT_BF16) emit(std::integral_constant<int, GLA_DT_BF16>{});
    else emit(std::integral_constant<int, GLA_DT_FP32>{});
}

// Sum the K splits in order, apply the channel scales and store: one thread per 4 adjacent columns.
__global__ __launch_bounds__(256) void splitk_finish_kernel(GemmWnArgs p) {
    const int n4 = p.N / 4;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * n4) return;
    const int m = (int)(idx / n4), n = (int)(idx % n4) * 4;
    const size_t slab = (size_t)p.M * p.N;
    const float* src = p.partials + (size_t)m * p.N + n;
    float4_t v = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < p.S; ++s) v += *(const float4_t*)(src + s * slab);
    const float sa = (p.csm & 2) ? load_as_float(p.scales_x, p.sx_dt, (int64_t)m * p.sxm) : 1.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float sb = (p.csm & 1) ? load_as_float(p.scales, p.meta_dt, n + j) : 1.0f;
        float r = v[j] * (sa * sb);
        if (p.bias != nullptr) r = round_to_dtype(p.out_dt, r) + load_as_float(p.bias, p.bias_dt, n + j);
        store_from_float(p.out, p.out_dt, (int64_t)m * p.osm + n + j, r);
    }
}

template <int BITS, bool BF16, int WAVES_M, int TI, int TJ>
int launch_wn(const GemmWnArgs& a, hipStream_t stream) {
    constexpr int BM = WAVES_M * TI * 32;
    const size_t smem = (size_t)ring_slots(BM) * slot_bytes(BITS, BM);
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = gemm_wn_kernel<BITS, BF16, WAVES_M, TI, TJ>;
    if (smem > 48 * 1024 && once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "gemm_wn: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n, a.S), dim3(WAVES_M * (8 / TJ) * 64), smem, stream, a);
    int rc = check_hip(hipGetLastError(), "gemm_wn launch");
    if (rc == GLA_OK && a.S > 1) {
        const int64_t items = (int64_t)a.M * (a.N / 4);
        hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, a);
        rc = check_hip(hipGetLastError(), "gemm_wn split-K reduction launch");
    }
    return rc;
}

template <int BITS, bool BF16>
int launch_wn_m(const GemmWnArgs& a, int bm, hipStream_t stream) {
    // four wave columns of 64 at every tile height: a wave unpacks only its own 64 columns
    if (bm == 256) return launch_wn<BITS, BF16, 2, 4, 2>(a, stream);
    if (bm == 128) return launch_wn<BITS, BF16, 1, 4, 2>(a, stream);
    if (bm == 64) return launch_wn<BITS, BF16, 1, 2, 2>(a, stream);
    return launch_wn<BITS, BF16, 1, 1, 2>(a, stream);
}

// tile_config encoding: BM (32, 64, 128 or 256; other = chosen here) + 1000 * K splits (0 = chosen here)
struct WnPlan {
    int bm, tiles_m, tiles_n, S, sps;
};

WnPlan wn_plan(const gla_matmul_args& p) {
    WnPlan g;
    const int cfg = p.tile_config > 0 ? p.tile_config : 0;
    const int bm_asked = cfg % 1000;
    const int total_steps = p.K / kBKw;
    // Tile height and K split from the cost model of dispatch.hpp, fitted to timings of every (tile, split) pair on
    // 4096^2 .. 16384^2 layers at 32..1024 rows.  What it reproduces for 2- and 4-bit codes: the 128-row tile up to
    // 256 rows (half the splits and partials of the 256-row one); above that the 128-row tile while 256-row ones would
    // leave CUs idle, unless K is long enough that a split of the 256-row tile costs less than it saves (16384^2 at 512
    // rows: 256-row tiles with 2 splits 295 us, 128-row tiles unsplit 316; 4096^2 at 2048 rows the other way round,
    // 105 and 85); tiles of up to 128 rows (4 waves) two to a CU on large layers (16384^2 at 64 rows: 8 splits 65 us,
    // 4 splits 69; 4096 x 14336 at 1024 rows: 128-row tiles with 4 splits 142 us, 256-row ones 158) and one to a CU on
    // medium ones (14336 x 4096 at 64 rows: 4 splits 26 us, 8 splits 30); whole rounds of workgroups.
    // 8-bit codes gain nothing from a second workgroup on the CU (4096^2 at 1024 rows, 32-row tiles: 512 workgroups
    // 117 us, 256 of them at 512 rows 60 us), so they count one to a CU: then the 256-row tile with splits wins from
    // 256 rows on 16384^2 (4 splits 166 us, 128-row tiles with 2 splits 185) and short tiles cost more per stage.
    static const int bms[4] = {32, 64, 128, 256};
    static const float cost_4[4] = {0.62f, 0.92f, 1.23f, 2.15f};  // us per 64-K stage, the chip full
    static const float cost_8[4] = {0.86f, 0.98f, 1.27f, 2.19f};
    const bool w8 = p.W_nbits == 8;
    const float* cost = w8 ? cost_8 : cost_4;
    TileModel model;
    model.underfill = w8 ? 0.9 : 0.78;
    model.split_us_per_elem = 1.4e-6;
    model.pair_up_to = w8 ? 0 : 128;  // one wave row: 4 waves, two workgroups fit a CU
    model.pair_cost = 1.7;
    const TilePick pick = pick_tile_and_split(p.M, p.N, kBNw, total_steps, 8, 32, bms, cost, 4,
                                              (bm_asked == 32 || bm_asked == 64 || bm_asked == 128 || bm_asked == 256) ? bm_asked : 0,
                                              cfg / 1000, model);
    g.bm = pick.bm;
    g.tiles_m = ceil_div(p.M, g.bm);
    g.tiles_n = ceil_div(p.N, kBNw);
    int want = pick.S;
    if (want > total_steps) want = total_steps;
    if (want < 1) want = 1;
    g.sps = ceil_div(total_steps, want);
    g.S = ceil_div(total_steps, g.sps);
    return g;
}

}  // namespace

bool gemm_wn_eligible(const gla_matmul_args& p) {
    if (p.w_dtype != GLA_DT_INT32) return false;
    if (!(p.W_nbits == 2 || p.W_nbits == 4 || p.W_nbits == 8)) return false;
    if (p.elements_per_sample * p.W_nbits != 32) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16)) return false;
    // (an int32 accumulator with 16-bit activations is the library's own call for widened int8 activations: the fp32
    // sums of integer products are exact below 2^24)
    if (!(p.acc_dtype == GLA_DT_FP32 || p.acc_dtype == GLA_DT_INT32)) return false;
    if (p.W_group_mode < 0 || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.channel_scale_mode < 0 || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    if (p.N < 4 || p.N % 4 != 0 || p.w_stride_n != 1 || p.w_stride_k % 4 != 0) return false;
    if (p.x_stride_k != 1 || p.x_stride_m % 8 != 0 || p.out_stride_n != 1) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    if (p.K % kBKw != 0) return false;
    // lane offsets inside the activation and weight arrays are 32-bit
    if ((int64_t)p.M * p.x_stride_m >= (1ll << 31) || (int64_t)(p.K / p.elements_per_sample) * p.w_stride_k >= (1ll << 31))
        return false;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if (uses_scales && (p.scales == nullptr || p.meta_stride_n != 1)) return false;
    if (uses_zeros && p.zeros == nullptr) return false;
    if (uses_zeros && !p.zero_is_scalar && p.meta_stride_n != 1) return false;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    if (grouped && (p.group_size % kBKw != 0 || p.K % p.group_size != 0)) return false;
    // scales and tensor zeros are read as four adjacent 16-bit values per lane
    const bool zeros_tensor = uses_zeros && !p.zero_is_scalar;
    if ((uses_scales || zeros_tensor) && !(p.meta_dtype == GLA_DT_FP16 || p.meta_dtype == GLA_DT_BF16)) return false;
    if (zeros_tensor && p.zeros_dtype != p.meta_dtype) return false;
    const bool one_group = !grouped || p.group_size == p.K;  // then the stride between groups is never used
    if (uses_scales && (((uintptr_t)p.scales & 3) || (!one_group && p.meta_stride_g % 2 != 0))) return false;
    if (zeros_tensor && (((uintptr_t)p.zeros & 3) || (!one_group && p.meta_stride_g % 2 != 0))) return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    return true;
}

int64_t gemm_wn_workspace_bytes(const gla_matmul_args& p) {
    const WnPlan g = wn_plan(p);
    return g.S > 1 ? kWsReserved + (int64_t)g.S * p.M * p.N * 4 : 0;
}

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
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    const WnPlan g = wn_plan(p);
    a.tiles_m = g.tiles_m; a.tiles_n = g.tiles_n; a.S = g.S; a.sps = g.sps;
    a.partials = nullptr;
    if (g.S > 1) {
        const int64_t need = gemm_wn_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemm_wn: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.partials = (float*)((char*)p.workspace + kWsReserved);
    }
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.W_nbits) {
        case 2: return bf16 ? launch_wn_m<2, true>(a, g.bm, stream) : launch_wn_m<2, false>(a, g.bm, stream);
        case 4: return bf16 ? launch_wn_m<4, true>(a, g.bm, stream) : launch_wn_m<4, false>(a, g.bm, stream);
        default: return bf16 ? launch_wn_m<8, true>(a, g.bm, stream) : launch_wn_m<8, false>(a, g.bm, stream);
    }
}

}  // namespace gla
