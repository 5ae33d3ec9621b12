// Mid-batch matmul (up to 64 rows per pass) for fp16/bf16 activations x 32-bit packed low-bit weights stored [K/e, N], N fastest:
// out[M,N] = x[M,K] * dequant(W)[K,N].  The batch sizes between the streaming GEMV (up to 16 rows) and the tiled GEMM,
// where the weights are still read once but every weight meets 2-4 MFMA row tiles.
//
// Takes the place of the reference's split-K GEMM at these batch sizes (reference:
// gemlite/triton_kernels/gemm_splitK_kernels.py:300-523; dequantisation gemlite/triton_kernels/utils.py:73-105).
//
//  * A wave owns 64 output columns and never shares weights with anybody: a lane loads 128 bits = the packed words
//    of 4 adjacent columns of one word row straight into registers (a wave load is 4 word rows x 256 contiguous
//    bytes), and the word a lane holds is, once unpacked, its share of the B operand of v_mfma_f32_16x16x32: lane
//    (column group cg, K-quarter kb) feeds 8 K-values of column 4 cg + j to MFMA j.  No weight passes through LDS.
//  * The NW waves of a workgroup sit side by side on 64 NW columns and walk the same K slab, so the activation rows
//    are shared: every stage of 128 (8-bit codes: 64) K-values is copied global -> LDS once per workgroup by the load
//    unit (global_load_lds) into a ring of D stages, as 16-row x 128-byte tiles whose 16-byte slots are XOR-swizzled by
//    row >> 1, and each wave reads its A operands from there (one ds_read_b128 per row tile and K-step).
//  * Weights and group metadata of the next D - 1 stages wait in registers; a wave waits on the vector-memory counter
//    once per stage, then the workgroup meets at one bare barrier, behind which the slot read last is refilled.
//  * 1-bit codes: a lane's word is 32 K-values, its share of all four K-steps of a 128-K stage (one load per stage).
//  * Dequantisation as in the tiled GEMM (wn_dequant.hpp): fp16 in natural K order (one v_perm + one masked OR per code
//    pair, packed fp16 subtract and fma), bf16 with codes paired (j, j + 4) or (j, j + 8) and the activation fragment
//    permuted to match, 2-bit codes on bf16 through a four-entry table per column and group, byte codes on bf16 by
//    direct conversion.
//  * K is split over gridDim.y when the column blocks alone do not fill the chip; the splits leave fp32 partials in
//    the workspace and a small second launch adds them in order (deterministic, no float atomics).
#include <type_traits>

#include "common.hpp"
#include "dispatch.hpp"
#include "wn_dequant.hpp"

namespace gla {

namespace {

struct WnMidArgs {
    const unsigned char* x;
    const unsigned char* w;
    const unsigned char* scales;  // group scales, or any readable address when the mode has none
    const unsigned char* zeros;   // group zeros, likewise
    const void* ch_scales;        // per-channel scales of channel_scale_mode (the same array as the group scales)
    const void* scales_x;
    void* out;
    float* partials;  // [S][M][N] when S > 1
    int M, N;
    int stages;  // stages in all of K
    int sps;     // stages per split
    int S;
    int spg;        // stages per quantisation group when a group spans whole stages (else 1)
    int spg_shift;  // log2(spg) when it is a power of two, else -1
    // groups that follow from the lane (a lane's word spans 16 or 32 K-values, so one MFMA K-step mixes 32-blocks):
    // group of (stage st, metadata slot gi, K-quarter kb) = st gt + gi gmul + (kb >> kbs)
    int lane_g, gt, gmul, kbs;
    int64_t xsm_b, wsk_b, msg_b, zsg_b;  // bytes per activation row, word row, group row of scales / zeros
    int64_t osm, sxm;
    int has_s, has_zt;  // the scales / zeros arrays are read per group
    const void* z_scalar;  // scalar zero point on the device, or NULL
    int z_dt;
    int wgm, csm, meta_dt, out_dt, sx_dt;
    const void* bias;
    int bias_dt;
};

template <int N>
__device__ __forceinline__ void wait_vmcnt_m() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <bool BF16>
__device__ __forceinline__ float4_t mfma16m(const u32x4& a, const u32x4& b, float4_t c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
}

template <int BITS>
struct MidShape {
    static constexpr int E = 32 / BITS;
    static constexpr int KS = BITS == 8 ? 64 : 128;                          // K-values per stage
    static constexpr int KSTEPS = KS / 32;                                   // MFMA K-steps per stage
    static constexpr int WR = KS / E;                                        // word rows per stage
    static constexpr int CW = WR / 4;                                        // 128-bit weight loads per lane and stage
    static constexpr int XT = KS / 64;                                       // 64-K activation tiles per 16 rows and stage
};

// RT: 16-row tiles (M <= 16 RT).  NW: waves = 64-column tiles per workgroup.  D: LDS ring depth.  GPS: groups per stage.
template <int BITS, bool BF16, int RT, int NW, int D, int GPS>
__global__ __launch_bounds__(NW * 64) void wn_mid_kernel(WnMidArgs a) {
    using SH = MidShape<BITS>;
    constexpr int KS = SH::KS, KSTEPS = SH::KSTEPS, WR = SH::WR, CW = SH::CW, XT = SH::XT;
    constexpr int TILE = 2048;                     // 16 rows x 128 bytes
    constexpr int STAGE_BYTES = RT * XT * TILE;
    constexpr int AJOBS = RT * XT * 2;             // copy instructions of a stage (8 rows each)
    constexpr int CA = (AJOBS + NW - 1) / NW;      // ... per wave
    constexpr int CM = 2 * GPS;                    // metadata loads per lane and stage
    constexpr int OPS = CA + CM + CW;              // vector-memory instructions per wave and stage
    constexpr int P = D - 1;                       // stages whose weights wait in registers
    constexpr bool NATURAL = !BF16 || BITS == 8;   // adjacent codes in adjacent K-slots: activations used as they lie
    constexpr int OFF = BITS == 8 ? 0 : 128;       // what the bf16 unpacking leaves on the codes
    static_assert((D - 2) * OPS < 64 && D >= 3, "outstanding loads must fit the vmcnt counter");
    static_assert(GPS == 1 || KSTEPS % GPS == 0, "a group is a whole number of K-steps");

    extern __shared__ __align__(16) unsigned char smem[];  // [D][RT * XT][TILE]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cg = lane & 15, kb = lane >> 4;
    const int n0w = (blockIdx.x * NW + wave) * 64;
    int col = n0w + 4 * cg;
    const bool col_ok = col < a.N;
    if (col > a.N - 4) col = a.N - 4;  // clamped lanes compute something and store nothing
    const int split = blockIdx.y;
    const int m0 = blockIdx.z * (16 * RT);  // batches above 64 rows run as row chunks that each read the weights again
    const int st0 = split * a.sps;
    const int nst = (a.stages - st0) < a.sps ? (a.stages - st0) : a.sps;
    const int st_last = st0 + nst - 1;

    // ---- activation copies: job q = rows 8 (q % 2) .. + 7 of tile q / 2 = (row tile, 64-K half); lane (row l / 8,
    // position l % 8) fetches the 16-byte piece that belongs at that position of the swizzled row
    uint32_t a_off[CA];
    int a_dst[CA];
#pragma unroll
    for (int i = 0; i < CA; ++i) {
        int q = wave + NW * i;
        if (q > AJOBS - 1) q = AJOBS - 1;  // surplus jobs repeat the last one: same data, same place
        const int t = q >> 1, j = q & 1;
        const int rt = t / XT, h = t % XT;
        const int row = 8 * j + (lane >> 3);
        const int piece = ((lane & 7) ^ (row >> 1)) & 7;
        int m = m0 + 16 * rt + row;
        if (m > a.M - 1) m = a.M - 1;
        a_off[i] = (uint32_t)m * (uint32_t)a.xsm_b + (uint32_t)(h * 128 + piece * 16);
        a_dst[i] = t * TILE + j * 1024;
    }
    auto issue_a = [&](int st, int slot) __attribute__((always_inline)) {
        const unsigned char* xk = a.x + (int64_t)st * (KS * 2);
        unsigned char* base = smem + slot * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < CA; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xk + a_off[i]),
                                             (__attribute__((address_space(3))) void*)(base + a_dst[i]), 16, 0, 0);
    };

    // ---- weights and metadata of a stage, into registers
    struct InFlight {
        uint4 w[CW];
        uint2 s[GPS], z[GPS];
    };
    uint32_t w_off[CW];
#pragma unroll
    for (int u = 0; u < CW; ++u) {
        // 2- and 4-bit codes: load u is word rows 4u .. 4u + 3; byte codes: K-step u / 2 is word rows 8 (u / 2) + 2 kb + u % 2
        const int row = BITS == 8 ? 8 * (u / 2) + 2 * kb + (u % 2) : 4 * u + kb;
        w_off[u] = (uint32_t)col * 4u + (uint32_t)row * (uint32_t)a.wsk_b;
    }
    const uint32_t m_off = (uint32_t)col * 2u;
    auto group_of = [&](int st) { return a.spg_shift >= 0 ? st >> a.spg_shift : st / a.spg; };
    auto issue_w = [&](int st, InFlight& f) __attribute__((always_inline)) {
        const unsigned char* wk = a.w + (int64_t)st * WR * a.wsk_b;
#pragma unroll
        for (int u = 0; u < CW; ++u) f.w[u] = load_streaming_u4(wk + w_off[u]);
#pragma unroll
        for (int gi = 0; gi < GPS; ++gi) {
            // (2-bit codes in groups of 32 and 1-bit codes in groups of 32 or 64: the lane's group follows from its
            // K-quarter)
            const int g = a.lane_g ? st * a.gt + gi * a.gmul + (kb >> a.kbs) : (GPS > 1 ? st * GPS + gi : group_of(st));
            f.s[gi] = load_streaming_u2(a.scales + (a.has_s ? (int64_t)g * a.msg_b + m_off : 0));
            f.z[gi] = load_streaming_u2(a.zeros + (a.has_zt ? (int64_t)g * a.zsg_b + m_off : 0));
        }
    };

    // ---- dequant constants: branch-free; absent scales / zeros are masked to 0 and replaced by constants, and the
    // zero-point term of every W_group_mode is z * (c1 + c2 * s)
    const bool meta_bf16 = a.meta_dt == GLA_DT_BF16;
    const uint32_t s_mask = a.has_s ? 0xffffu : 0u, z_mask = a.has_zt ? 0xffffu : 0u;
    const float z_const = a.z_scalar != nullptr ? load_as_float(a.z_scalar, a.z_dt, 0) : 0.0f;
    const float s_add = a.has_s ? 0.0f : 1.0f, z_add = a.has_zt ? 0.0f : z_const;
    const float c1 = a.wgm == GLA_WGM_SHIFT ? -1.0f : (a.wgm == GLA_WGM_FMA ? 1.0f : 0.0f);
    const float c2 = a.wgm == GLA_WGM_SHIFT_SCALE ? -1.0f : 0.0f;
    ColMeta<BF16> meta[4];
    auto convert_meta = [&](const uint2& rs, const uint2& rz) __attribute__((always_inline)) {
        const uint32_t raw_s[2] = {rs.x, rs.y}, raw_z[2] = {rz.x, rz.y};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t sv = (raw_s[j / 2] >> (16 * (j & 1))) & s_mask;
            const uint32_t zv = (raw_z[j / 2] >> (16 * (j & 1))) & z_mask;
            const float s_h = half_bits_to_float((uint16_t)sv), s_b = __builtin_bit_cast(float, sv << 16);
            const float z_h = half_bits_to_float((uint16_t)zv), z_b = __builtin_bit_cast(float, zv << 16);
            const float s = (meta_bf16 ? s_b : s_h) + s_add;
            const float z = (meta_bf16 ? z_b : z_h) + z_add;
            meta[j] = make_meta<BF16, OFF>(s, z * __builtin_fmaf(c2, s, c1));
            if constexpr (BF16 && BITS == 2) {
                // the four values a 2-bit code can take in this column and group, made once (the arithmetic of
                // dequant_pair: (128 + q) s + (z' - 128 s) in fp32, one round-to-nearest-even conversion)
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                const f32x2 w01 = {__builtin_fmaf(128.0f, meta[j].s, meta[j].z), __builtin_fmaf(129.0f, meta[j].s, meta[j].z)};
                const f32x2 w23 = {__builtin_fmaf(130.0f, meta[j].s, meta[j].z), __builtin_fmaf(131.0f, meta[j].s, meta[j].z)};
                meta[j].lut01 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w01, bf16x2_t));
                meta[j].lut23 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w23, bf16x2_t));
            }
        }
    };

    uint32_t pair_mask = ((1u << BITS) - 1u) * 0x00010001u, magic = 0x43004300u;
    asm volatile("" : "+s"(pair_mask), "+v"(magic));  // registers, so that v_and_or_b32 is selected
    uint32_t nat_mask0 = BITS == 4 ? 0x00F0000Fu : 0x000C0003u, nat_magic0 = BITS == 4 ? 0x54006400u : 0x5C006400u;
    uint32_t nat_mask1 = 0x00C00030u, nat_magic1 = 0x4C005400u;
    asm volatile("" : "+s"(nat_mask0), "+v"(nat_magic0), "+s"(nat_mask1), "+v"(nat_magic1));

    // B operand of column set j for K-step ks of the stage: the lane's 8 codes of column 4 cg + j, dequantised
    auto b_operand = [&](const InFlight& f, int ks, int j) __attribute__((always_inline)) {
        auto word = [&](int u) __attribute__((always_inline)) {
            const uint4& v = f.w[u];
            return j == 0 ? v.x : (j == 1 ? v.y : (j == 2 ? v.z : v.w));
        };
        u32x4 bq;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t t;
            if constexpr (BITS == 8 && BF16) {
                // 128 + q is not exact in bf16 above 127: bytes straight to fp32, scaled there, packed once
                const uint32_t w = word(2 * ks + q / 2);
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                const f32x2 v = {__builtin_fmaf((float)((w >> ((q % 2) * 16)) & 0xffu), meta[j].s, meta[j].z),
                                 __builtin_fmaf((float)((w >> ((q % 2) * 16 + 8)) & 0xffu), meta[j].s, meta[j].z)};
                bq[q] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
            } else if constexpr (NATURAL) {
                // register q gets the adjacent codes 2q and 2q + 1 of the lane's eight: one v_perm puts the byte(s)
                // that hold them into both halves, the mask keeps one code per half where it lies, and each half's
                // magic exponent is the one whose last-place unit matches the code's position
                if constexpr (BITS == 8) {
                    const uint32_t w = word(2 * ks + q / 2);
                    t = __builtin_amdgcn_perm(w, w, q % 2 ? 0x0c030c02u : 0x0c010c00u) | 0x64006400u;
                    bq[q] = dequant_pair<BF16>(t, meta[j]);
                } else if constexpr (BITS == 1) {
                    // a word is 32 K-values = the lane's share of all four K-steps: step ks takes byte ks, whose bits 2q and
                    // 2q + 1 land in the mantissas of 2^(10 - 2q) and 2^(9 - 2q)
                    const uint32_t w = word(0);
                    const uint32_t u = __builtin_amdgcn_perm(w, w, 0x0c000c00u | ((uint32_t)ks << 16) | (uint32_t)ks);
                    const uint32_t mk = (1u << (2 * q)) | (1u << (2 * q + 17));
                    const uint32_t mg = ((uint32_t)(25 - 2 * q) << 10) | ((uint32_t)(24 - 2 * q) << 26);
                    t = (u & mk) | mg;
                    bq[q] = dequant_pair<BF16>(t, meta[j], (float)(1024 >> (2 * q)), (float)(512 >> (2 * q)));
                } else if constexpr (BITS == 4) {
                    const uint32_t w = word(ks);
                    t = (__builtin_amdgcn_perm(w, w, 0x0c000c00u | (q << 16) | q) & nat_mask0) | nat_magic0;
                    bq[q] = dequant_pair<BF16>(t, meta[j], 1024.0f, 64.0f);
                } else {
                    // a word is 16 K-values = both K-steps of its load: step ks % 2 takes bytes 2 (ks % 2), + 1
                    const uint32_t w = word(ks / 2);
                    const uint32_t b = 2 * (ks % 2) + q / 2;
                    const uint32_t u = __builtin_amdgcn_perm(w, w, 0x0c000c00u | (b << 16) | b);
                    if (q % 2 == 0) bq[q] = dequant_pair<BF16>((u & nat_mask0) | nat_magic0, meta[j], 1024.0f, 256.0f);
                    else bq[q] = dequant_pair<BF16>((u & nat_mask1) | nat_magic1, meta[j], 64.0f, 16.0f);
                }
            } else if constexpr (BITS == 1) {
                t = ((word(0) >> (4 * ks + q)) & pair_mask) | magic;  // codes (4 ks + q, + 16) of the lane's 32
                bq[q] = dequant_pair<BF16>(t, meta[j]);
            } else if constexpr (BITS == 4) {
                t = ((word(ks) >> (q * 4)) & pair_mask) | magic;  // codes (q, q + 4)
                bq[q] = dequant_pair<BF16>(t, meta[j]);
            } else {
                // 2-bit codes on bf16: codes (4 (ks % 2) + q, + 8) pick their values from the column's table with one
                // byte permute; the selector bytes (2c, 2c + 1) of each code come from one 24-bit multiply-add
                t = (word(ks / 2) >> ((4 * (ks % 2) + q) * 2)) & pair_mask;
                const uint32_t sel = __umul24(t, 0x0202u) + 0x01000100u;
                bq[q] = __builtin_amdgcn_perm(meta[j].lut23, meta[j].lut01, sel);
            }
        }
        return bq;
    };

    float4_t acc[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rt][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int a_row = cg * 128, swz = cg >> 1;
    auto a_piece = [&](const unsigned char* tile, int piece) __attribute__((always_inline)) {
        return *(const u32x4*)(tile + a_row + ((piece ^ swz) & 7) * 16);
    };

    int g_have = -1;  // group whose constants `meta` holds (a group that spans stages is converted once)
    auto compute = [&](int st, int slot, const InFlight& f) __attribute__((always_inline)) {
        const unsigned char* base = smem + slot * STAGE_BYTES;
        u32x4 keep_lo[RT], keep_hi[RT];  // 2-bit codes on bf16: the lane's 16 activations serve two K-steps
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            if constexpr (GPS > 1) {
                if (ks % (KSTEPS / GPS) == 0) convert_meta(f.s[ks / (KSTEPS / GPS)], f.z[ks / (KSTEPS / GPS)]);
            } else {
                if (ks == 0) {
                    const int g = a.lane_g ? st : group_of(st);
                    if (g != g_have) convert_meta(f.s[0], f.z[0]);
                    g_have = g;
                }
            }
            u32x4 av[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const unsigned char* tile = base + (rt * XT + (XT > 1 ? ks / 2 : 0)) * TILE;
                if constexpr (BITS == 1) {
                    // the lane's 32 K-values are half a 64-K tile: tile kb / 2, pieces 4 (kb % 2) .. + 3
                    const unsigned char* t1 = base + (rt * XT + (kb >> 1)) * TILE;
                    if constexpr (BF16) {
                        // codes (4 ks + r, + 16): activations 4 ks .. + 3 and 16 + 4 ks .. + 3 of the lane's 32
                        if (ks % 2 == 0) {
                            keep_lo[rt] = a_piece(t1, 4 * (kb & 1) + ks / 2);
                            keep_hi[rt] = a_piece(t1, 4 * (kb & 1) + ks / 2 + 2);
                        }
                        const int t2 = 2 * (ks % 2);
                        av[rt] = pair_order(keep_lo[rt][t2], keep_lo[rt][t2 + 1], keep_hi[rt][t2], keep_hi[rt][t2 + 1]);
                    } else {
                        av[rt] = a_piece(t1, 4 * (kb & 1) + ks);
                    }
                } else if constexpr (BF16 && BITS == 2) {
                    if (ks % 2 == 0) {
                        keep_lo[rt] = a_piece(tile, 2 * kb);
                        keep_hi[rt] = a_piece(tile, 2 * kb + 1);
                    }
                    const int t2 = 2 * (ks % 2);
                    av[rt] = pair_order(keep_lo[rt][t2], keep_lo[rt][t2 + 1], keep_hi[rt][t2], keep_hi[rt][t2 + 1]);
                } else if constexpr (!BF16 && BITS == 2) {
                    av[rt] = a_piece(tile, 2 * kb + ks % 2);
                } else {
                    const u32x4 v = a_piece(tile, (XT > 1 ? 4 * (ks % 2) : 4 * ks) + kb);
                    if constexpr (NATURAL) av[rt] = v;
                    else av[rt] = pair_order(v.x, v.y, v.z, v.w);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const u32x4 bq = b_operand(f, ks, j);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) acc[rt][j] = mfma16m<BF16>(av[rt], bq, acc[rt][j]);
            }
        }
    };

    // ---- pipeline: iteration `it` waits for what iteration it - (D - 1) asked for, meets the other waves, refills the
    // slot everybody has just left, multiplies, and asks for the weights of stage it + D - 1.  Past the end of the slab
    // the last stage is asked for again, so that every iteration issues the same number of loads.
    auto clamp_st = [&](int i) { return st0 + (i < nst ? i : nst - 1); };
    InFlight fl[P];
#pragma unroll
    for (int b = 0; b < P; ++b) {
        issue_a(clamp_st(b), b);
        issue_w(clamp_st(b), fl[b]);
    }
    int slot = 0, islot = D - 1;
    for (int it0 = 0; it0 < nst; it0 += P) {
#pragma unroll
        for (int u = 0; u < P; ++u) {
            const int it = it0 + u;
            wait_vmcnt_m<(D - 2) * OPS>();
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_a(clamp_st(it + D - 1), islot);
            islot = islot == D - 1 ? 0 : islot + 1;
            __builtin_amdgcn_sched_barrier(0);
            if (it < nst) compute(st0 + it, slot, fl[u]);
            slot = slot == D - 1 ? 0 : slot + 1;
            __builtin_amdgcn_sched_barrier(0);
            issue_w(clamp_st(it + P), fl[u]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    (void)st_last;
    wait_vmcnt_m<0>();  // the surplus copies of the last iterations must have landed before the LDS is given back

    // ---- lane (cg, kb) holds rows m0 + 16 rt + 4 kb + e of columns n0w + 4 cg + j in acc[rt][j][e]
    if (!col_ok) return;
    if (a.S > 1) {
        float* dst = a.partials + (size_t)split * a.M * a.N;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + 16 * rt + 4 * kb + e;
                if (m < a.M) *(float4_t*)(dst + (size_t)m * a.N + col) = float4_t{acc[rt][0][e], acc[rt][1][e], acc[rt][2][e], acc[rt][3][e]};
            }
        return;
    }
    float sb[4], bias[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        sb[j] = (a.csm & 1) ? load_as_float(a.ch_scales, a.meta_dt, col + j) : 1.0f;
        bias[j] = a.bias != nullptr ? load_as_float(a.bias, a.bias_dt, col + j) : 0.0f;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + 16 * rt + 4 * kb + e;
            if (m >= a.M) continue;
            const float sa = (a.csm & 2) ? load_as_float(a.scales_x, a.sx_dt, (int64_t)m * a.sxm) : 1.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v = acc[rt][j][e] * (sa * sb[j]);
                if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + bias[j];
                store_from_float(a.out, a.out_dt, (int64_t)m * a.osm + col + j, v);
            }
        }
}

// Sum the K splits in order, apply the channel scales and store: one thread per 4 adjacent columns.
__global__ __launch_bounds__(256) void wn_mid_finish_kernel(WnMidArgs p) {
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
        const float sb = (p.csm & 1) ? load_as_float(p.ch_scales, p.meta_dt, n + j) : 1.0f;
        float r = v[j] * (sa * sb);
        if (p.bias != nullptr) r = round_to_dtype(p.out_dt, r) + load_as_float(p.bias, p.bias_dt, n + j);
        store_from_float(p.out, p.out_dt, (int64_t)m * p.osm + n + j, r);
    }
}

struct MidPlan {
    int rt, nw, S, sps, stages, gps, gt;
    bool lane_groups;  // 2-bit codes in groups of 32, 1-bit codes in groups of 32 / 64: the lane picks its group (gt per stage)
};

int stage_k(int bits) { return bits == 8 ? 64 : 128; }

MidPlan mid_plan(const gla_matmul_args& p) {
    // tile_config: waves per workgroup (4 or 8) + 1000 * K splits; anything else leaves both to the rule below
    MidPlan g;
    g.rt = p.M > 64 ? 4 : ceil_div(p.M, 16);
    const int cfg = p.tile_config > 0 ? p.tile_config : 0;
    // Four waves (256 columns) per workgroup: half the K splits, and with them half the fp32 partials, of eight waves
    // for the same number of workgroups (8-bit codes, 16384^2 at 16 / 64 rows: 50 / 70 us against 60 / 75)
    g.nw = cfg % 1000 == 8 ? 8 : 4;
    g.stages = p.K / stage_k(p.W_nbits);
    const bool grouped = p.W_group_mode >= GLA_WGM_SCALE || (p.W_group_mode == GLA_WGM_SHIFT && !p.zero_is_scalar);
    const int gs = grouped ? p.group_size : p.K;
    g.gps = gs < stage_k(p.W_nbits) ? stage_k(p.W_nbits) / gs : 1;
    // a lane's word of 2-bit codes is 16 K-values, of 1-bit codes 32: below groups of 64 (128) the group follows
    // from the lane.  So it does in groups of 16, two of which share every K-step (a lane's eight codes of a K-step lie
    // in one group): metadata per K-step (4- and 8-bit codes) or per word (2-bit codes).
    const bool g16 = gs == 16;
    g.lane_groups = g16 || (p.W_nbits == 2 && g.gps == 4) || (p.W_nbits == 1 && g.gps > 1);
    g.gt = g.gps;
    if (g.lane_groups) g.gps = p.W_nbits == 2 ? 2 : (g16 ? (p.W_nbits == 4 ? 4 : 2) : 1);
    // one workgroup per CU; a split is at least 4 stages long
    const int blocks = ceil_div(p.N, 64 * g.nw);
    const int chunks = ceil_div(p.M, 64);
    int want = cfg >= 1000 ? cfg / 1000 : (256 + blocks * chunks - 1) / (blocks * chunks);
    if (want > g.stages / 4) want = g.stages / 4;
    if (want < 1) want = 1;
    g.sps = ceil_div(g.stages, want);
    g.S = ceil_div(g.stages, g.sps);
    return g;
}

template <int BITS, bool BF16, int RT, int GPS, int NW>
int launch_mid(const WnMidArgs& a, const MidPlan& g, hipStream_t stream) {
    constexpr int D = 4;
    using SH = MidShape<BITS>;
    const size_t smem = (size_t)D * RT * SH::XT * 2048;
    static DeviceOnce once;  // per instantiation; the attribute is sticky per function and device
    auto kern = wn_mid_kernel<BITS, BF16, RT, NW, D, GPS>;
    if (smem > 48 * 1024 && once.first()) {
        const int rc = check_hip(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem),
                                 "wn_mid: raising the dynamic LDS limit");
        if (rc != GLA_OK) return rc;
    }
    (void)g;
    hipLaunchKernelGGL(kern, dim3(ceil_div(a.N, 64 * NW), a.S, ceil_div(a.M, 16 * RT)), dim3(NW * 64), smem, stream, a);
    int rc = check_hip(hipGetLastError(), "wn_mid launch");
    if (rc == GLA_OK && a.S > 1) {
        const int64_t items = (int64_t)a.M * (a.N / 4);
        hipLaunchKernelGGL(wn_mid_finish_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream, a);
        rc = check_hip(hipGetLastError(), "wn_mid split-K reduction launch");
    }
    return rc;
}

template <int BITS, bool BF16, int RT>
int launch_mid_gps(const WnMidArgs& a, const MidPlan& g, hipStream_t stream) {
    if constexpr (BITS == 4) {
        if (g.gps == 4) return launch_mid<BITS, BF16, RT, 4, 4>(a, g, stream);  // groups of 32: four waves only
    }
    if (g.nw == 4) {
        if (g.gps == 2) return launch_mid<BITS, BF16, RT, 2, 4>(a, g, stream);
        return launch_mid<BITS, BF16, RT, 1, 4>(a, g, stream);
    }
    if (g.gps == 2) return launch_mid<BITS, BF16, RT, 2, 8>(a, g, stream);
    return launch_mid<BITS, BF16, RT, 1, 8>(a, g, stream);
}

template <int BITS, bool BF16>
int launch_mid_rt(const WnMidArgs& a, const MidPlan& g, hipStream_t stream) {
    switch (g.rt) {
        case 1: return launch_mid_gps<BITS, BF16, 1>(a, g, stream);
        case 2: return launch_mid_gps<BITS, BF16, 2>(a, g, stream);
        case 3: return launch_mid_gps<BITS, BF16, 3>(a, g, stream);
        default: return launch_mid_gps<BITS, BF16, 4>(a, g, stream);
    }
}

}  // namespace

bool wn_mid_eligible(const gla_matmul_args& p) {
    // operand types, layouts and alignments as for the tiled packed-weight GEMM, whose rule on groups (whole 64-K
    // stages) is replaced by this kernel's own below; 1-bit codes, which that one does not take, pass as 2-bit ones
    gla_matmul_args q = p;
    q.group_size = p.K;
    if (p.W_nbits == 1 && p.elements_per_sample == 32) {
        q.W_nbits = 2;
        q.elements_per_sample = 16;
    }
    if (p.K <= 0 || !gemm_wn_eligible(q)) return false;
    if (p.M < 1) return false;
    const int ks = stage_k(p.W_nbits);
    if (p.K % ks != 0) return false;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool zeros_tensor = (p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE) && !p.zero_is_scalar;
    const bool grouped = uses_scales || zeros_tensor;
    const int gs = grouped ? p.group_size : p.K;
    if (gs <= 0 || p.K % gs != 0) return false;
    // a group is whole stages, or a stage is a whole number of groups of at least 16 (1-bit codes: 32, a pair of
    // the codes that share a register on bf16 lies 16 K-values apart)
    if (!(gs % ks == 0 || (ks % gs == 0 && gs >= (p.W_nbits == 1 ? 32 : 16)))) return false;
    if ((int64_t)(p.K / p.elements_per_sample) * p.w_stride_k >= (1ll << 31)) return false;
    // metadata is read as four adjacent 16-bit values per lane
    const bool one_group = gs == p.K;
    if (uses_scales && (((uintptr_t)p.scales & 7) || (!one_group && p.meta_stride_g % 4 != 0))) return false;
    if (zeros_tensor && (((uintptr_t)p.zeros & 7) || (!one_group && p.meta_stride_g % 4 != 0))) return false;
    if ((int64_t)p.M * p.x_stride_m * 2 >= (1ll << 31)) return false;
    return true;
}

int64_t wn_mid_workspace_bytes(const gla_matmul_args& p) {
    const MidPlan g = mid_plan(p);
    return g.S > 1 ? kWsPrivateBytes + (int64_t)g.S * p.M * p.N * 4 : 0;
}

int launch_wn_mid(const gla_matmul_args& p, hipStream_t stream) {
    if (!wn_mid_eligible(p)) {
        set_error("wn_mid: fp16 / bf16 activations on 1-, 2-, 4- or 8-bit packed codes, groups of whole 128-K stages (8-bit: 64) "
                  "or of 16 / 32 / 64 (1-bit: 32 / 64)");
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    const MidPlan g = mid_plan(p);
    WnMidArgs a;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    const int gs = grouped ? p.group_size : p.K;
    a.x = (const unsigned char*)p.x; a.w = (const unsigned char*)p.w;
    a.has_s = uses_scales; a.has_zt = uses_zeros && !p.zero_is_scalar;
    a.scales = a.has_s ? (const unsigned char*)p.scales : (const unsigned char*)p.w;
    a.zeros = a.has_zt ? (const unsigned char*)p.zeros : (const unsigned char*)p.w;
    a.ch_scales = p.scales; a.scales_x = p.scales_x; a.out = p.out;
    a.M = p.M; a.N = p.N;
    a.stages = g.stages; a.sps = g.sps; a.S = g.S;
    const int ks = stage_k(p.W_nbits);
    a.spg = gs >= ks ? gs / ks : 1;
    a.lane_g = g.lane_groups; a.gt = g.gt;
    if (gs == 16) {
        // 2-bit: metadata slot gi is the 64-K load, a group per lane quarter; 4- and 8-bit: slot gi is the K-step, a
        // group per pair of lane quarters
        a.gmul = p.W_nbits == 2 ? 4 : 2;
        a.kbs = p.W_nbits == 2 ? 0 : 1;
    } else {
        a.gmul = p.W_nbits == 2 ? 2 : 0;                   // 2-bit: metadata slot gi is the 64-K load, two groups each
        a.kbs = (p.W_nbits == 1 && g.gt == 4) ? 0 : 1;     // 1-bit gs 32: a group per K-quarter; otherwise per pair of them
    }
    a.spg_shift = -1;
    for (int s = 0; s < 31; ++s)
        if ((1 << s) == a.spg) a.spg_shift = s;
    const bool one_group = gs == p.K;
    a.xsm_b = p.x_stride_m * 2; a.wsk_b = p.w_stride_k * 4;
    a.msg_b = one_group ? 0 : p.meta_stride_g * 2; a.zsg_b = a.msg_b;
    a.osm = p.out_stride_m; a.sxm = p.sx_stride_m;
    a.z_scalar = (uses_zeros && p.zero_is_scalar) ? p.zeros : nullptr; a.z_dt = p.zeros_dtype;
    a.wgm = p.W_group_mode; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.out_dt = p.output_dtype; a.sx_dt = p.sx_dtype;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    a.partials = nullptr;
    if (g.S > 1) {
        const int64_t need = wn_mid_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("wn_mid: workspace of %lld bytes required, %llu given", (long long)need, (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.partials = (float*)((char*)p.workspace + kWsPrivateBytes);
    }
    const bool bf16 = p.input_dtype == GLA_DT_BF16;
    switch (p.W_nbits) {
        case 1: return bf16 ? launch_mid_rt<1, true>(a, g, stream) : launch_mid_rt<1, false>(a, g, stream);
        case 2: return bf16 ? launch_mid_rt<2, true>(a, g, stream) : launch_mid_rt<2, false>(a, g, stream);
        case 4: return bf16 ? launch_mid_rt<4, true>(a, g, stream) : launch_mid_rt<4, false>(a, g, stream);
        default: return bf16 ? launch_mid_rt<8, true>(a, g, stream) : launch_mid_rt<8, false>(a, g, stream);
    }
}

}  // namespace gla
