// Streaming small-batch matmul (M <= 16 per pass) for 32-bit packed weight words stored
// [K/e, N], N fastest: the decode path.
//
// Takes the place of the reference's GEMV / RevSplit-K kernels and of its split-K GEMM at
// small batch (reference: gemlite/triton_kernels/gemv_revsplitK_kernels.py:248-443,
// gemlite/triton_kernels/gemv_kernels.py:245-426,
// gemlite/triton_kernels/gemm_splitK_kernels.py:300-523) with a different decomposition:
//
//  * A workgroup (4 waves) owns 64 output columns and a slab of RW word rows; its waves split
//    the slab.  A lane owns 4 adjacent columns (one 128-bit load) and the four 16-lane quarters
//    own four consecutive "super rows" (8 codes along K, i.e. one word for <= 4-bit codes, two
//    words for 8-bit codes), so a wave load covers 4 rows x 256 contiguous bytes.
//  * The lane's word is exactly one B operand of v_mfma_f32_16x16x32 (8 K-values of one
//    column).  Codes are turned into fp16/bf16 numbers OFF+q by OR-ing their bits into the
//    mantissa of the constant OFF (1024 in fp16, 128 in bf16): two codes per VALU op, in the
//    pair order (j, j + e/2).  The activation rows are staged in LDS in the same pair order
//    and are the A operand (up to 16 rows, so every batch size up to 16 costs the same).
//  * Scales and zero points are applied per quantisation group, not per weight: with
//    C = sum_k x_k (OFF + q_k) and SX = sum_k x_k (one more MFMA against a B of ones) the
//    group adds s*C + zz*SX, where (s, zz) folds scale, zero point and -OFF*s in fp32.  All
//    five dequant modes are a choice of (s, zz), staged per slab in LDS.
//  * The K reduction is deterministic: k-blocks inside the MFMA, waves through LDS, slabs through a
//    pairwise tree in the workspace (no float atomics, no second launch).  Every output element has,
//    per tree node, one 64-bit slot (value, tag); the two children of a node each swap their partial
//    into it with one atomic exchange.  The one that finds the slot empty is done; the one that gets
//    its sibling's partial back adds it (the tree is fixed and a sum of two is the same either way
//    round, so the result never depends on who arrived first), clears the slot for the next launch
//    and goes on to the parent.  Whoever leaves
//    the root holds the total and stores the output.  Every thread decides for its own element: no
//    ticket, no barrier, no polling.  Problems whose slots do not fit the private region of the
//    workspace use fp32 partials and a ticket counter per column tile instead (the last-arriving
//    workgroup sums the slabs in order).
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

constexpr int kTileN = 64;  // output columns per workgroup
constexpr int kBatch = 8;   // 128-bit loads in flight per lane
constexpr int64_t kCounterBytes = kWsCounterBytes;  // ticket-counter region at the start of the workspace
constexpr int kCounterStride = 32;  // words between the counters of two column tiles: a 128-byte line each.  The atomic
                                    // unit takes the adds to one line one after the other; with the counters of 32 tiles in
                                    // one line, the 256 tickets of a launch queued up there for ~2 us
constexpr int64_t kSlotBytes = kWsPrivateBytes - kWsCounterBytes;  // tagged partial slots, private to this family
constexpr uint32_t kSlotValid = 0x7fc5a11du;  // tag of a published slot; a consumed slot is all zeros

struct GemvArgs {
    const uint32_t* w;
    const void* x;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    float* partials;             // [S][Mp][N] fp32 (plain protocol: problems whose slots do not fit the private region)
    unsigned long long* slots;   // [S][Mp][N] (value, tag) (tagged protocol), or NULL
    unsigned* counters;
    int M, N, K;
    int R;      // word rows = K / E
    int RW;     // word rows per workgroup
    int S;      // number of slabs along K
    int tiles;  // column tiles
    int Mp;     // M rounded up to the row tile
    int gr;     // word rows per quantisation group
    int G;      // number of groups along K
    int GW;     // (s, zz) table rows staged per workgroup
    int FL;     // wave iterations per flush
    int waves;  // waves per workgroup (4, 8 or 16)
    int nfb;      // direct variant: flush blocks per batch of loads
    int fl_log2;  // log2(FL)
    int srww;     // direct variant: super rows per wave = RW / LW / waves, divided on the host
    int gr_shift; // log2(gr) when gr is a power of two, else -1 (the kernels then divide)
    int wgm, csm, meta_dt, z_dt, z_scalar, out_dt, sx_dt;
    int64_t wsk, xsm, osm, msg, sxm;
    const void* bias;  // [N] or NULL: added to the result rounded to the output type
    int bias_dt;
};

// word row -> quantisation group: a shift for the usual power-of-two groups
__device__ __forceinline__ int div_group(const GemvArgs& a, int word_row) {
    return a.gr_shift >= 0 ? word_row >> a.gr_shift : word_row / a.gr;
}

template <bool BF16>
struct Magic;
template <>
struct Magic<false> {
    static constexpr uint32_t bits = 0x64006400u;  // fp16 1024.0 twice
    static constexpr uint32_t ones = 0x3c003c00u;  // fp16 1.0 twice
    static constexpr float off = 1024.0f;
};
template <>
struct Magic<true> {
    static constexpr uint32_t bits = 0x43004300u;  // bf16 128.0 twice
    static constexpr uint32_t ones = 0x3f803f80u;  // bf16 1.0 twice
    static constexpr float off = 128.0f;
};

template <bool BF16>
__device__ __forceinline__ float4_t mfma16(const uint4& a, const uint4& b, float4_t c) {
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                       c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c,
                                                      0, 0, 0);
    }
}

__device__ __forceinline__ float meta_to_float(uint16_t v, int dt) {
    return dt == GLA_DT_BF16 ? bf16_bits_to_float(v) : half_bits_to_float(v);
}

__device__ __forceinline__ float2 fold_meta(float s, float z, int wgm, float OFF) {
    float zz;
    switch (wgm) {
        case GLA_WGM_SHIFT: zz = -z - OFF; break;
        case GLA_WGM_SCALE: zz = -OFF * s; break;
        case GLA_WGM_SHIFT_SCALE: zz = -(z + OFF) * s; break;
        case GLA_WGM_FMA: zz = __builtin_fmaf(-OFF, s, z); break;
        default: zz = -OFF; break;
    }
    return make_float2(s, zz);
}

// Geometry shared by kernel and host: per code width, a "super row" is the run of word rows
// that holds the 8..32 K-values one lane feeds to the MFMAs of one wave iteration.
template <int BITS>
struct Shape {
    static constexpr int E = 32 / BITS;             // codes per word
    static constexpr int LW = (E < 8) ? 8 / E : 1;  // word rows per super row (2 for 8-bit codes)
    static constexpr int KPS = E * LW;              // K-values per super row (8, 16 or 32)
    static constexpr int T = KPS / 8;               // MFMA K-steps per super row
};

// (w & mask) | magic.  Callers keep `mask` and `magic` in registers (made opaque to constant
// folding) so that the compiler can select the single-instruction v_and_or_b32, which takes no
// literal operands on this target.  Plain C on purpose: an inline-asm VALU op is invisible to the
// compiler's MFMA hazard tracking.
__device__ __forceinline__ uint32_t and_or(uint32_t w, uint32_t mask, uint32_t magic) {
    return (w & mask) | magic;
}

// Lane l of every row of 16 lanes receives the value of lane l + n of the same row (lanes past the row's end: zero).
// n is a constant after unrolling.
template <int N>
__device__ __forceinline__ uint32_t row_down_c(uint32_t v) {
    if constexpr (N == 0) return v;
    else return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x100 + N, 0xf, 0xf, true);  // row_shl:N
}
__device__ __forceinline__ uint32_t row_down(uint32_t v, int n) {
    switch (n) {
        case 1: return row_down_c<1>(v);
        case 2: return row_down_c<2>(v);
        case 3: return row_down_c<3>(v);
        case 4: return row_down_c<4>(v);
        case 5: return row_down_c<5>(v);
        case 6: return row_down_c<6>(v);
        case 7: return row_down_c<7>(v);
        case 8: return row_down_c<8>(v);
        case 9: return row_down_c<9>(v);
        case 10: return row_down_c<10>(v);
        case 11: return row_down_c<11>(v);
        case 12: return row_down_c<12>(v);
        case 13: return row_down_c<13>(v);
        case 14: return row_down_c<14>(v);
        case 15: return row_down_c<15>(v);
        default: return v;
    }
}
__device__ __forceinline__ uint4 row_down(const uint4& v, int n) {
    return make_uint4(row_down(v.x, n), row_down(v.y, n), row_down(v.z, n), row_down(v.w, n));
}

__device__ __forceinline__ uint32_t pick(const uint4& v, int j) {
    return j == 0 ? v.x : (j == 1 ? v.y : (j == 2 ? v.z : v.w));
}

// Shared end of both kernels: sum the waves of the workgroup through LDS, combine the K slabs
// (last-arriving workgroup of a column tile sums the partials in slab order), apply the channel
// scales and store.  Lane (cg, kb) holds rows 4*kb + i of columns 4*cg + j in acc[j][i].
// kWaves = 0: the number of waves is blockDim.x / 64 (any count from 4 to 16; RT <= 4 only).
template <int RT, int kWaves, int RI>
__device__ __forceinline__ void wg_finish(const GemvArgs& a, float (&acc)[4][RI], float* red, unsigned& ticket,
                                          int tile, int split, int m0, int n0) {
    const int waves = kWaves ? kWaves : (int)(blockDim.x >> 6);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wv = tid >> 6;
    const int cg = lane & 15, kb = lane >> 4;
    // ---- reduce the waves: lane (cg, kb) holds rows 4*kb + i of columns 4*cg + j
    if (RT == 16 || kb == 0) {
#pragma unroll
        for (int i = 0; i < RI; ++i) {
            const int m = 4 * kb + i;
            *(float4*)(red + ((size_t)wv * RT + m) * kTileN + cg * 4) =
                make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
        }
    }
    __syncthreads();

    // output rows per thread; a run-time wave count is at least 4 (row tiles up to 4) or 8 (the 16-row tile)
    constexpr int NT = kWaves ? (RT + kWaves - 1) / kWaves : (RT <= 4 ? 1 : 2);
    const int n_out = n0 + lane;
    const bool col_ok = n_out < a.N;
    // loaded before the reduction, so that its latency is not the kernel's tail
    const float bias = (a.bias != nullptr && col_ok) ? load_as_float(a.bias, a.bias_dt, n_out) : 0.0f;
    float total[NT];
    bool alive[NT];  // this thread still owes the output element of row t
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int m = wv + t * waves;
        alive[t] = true;
        float v = 0.0f;
        if (m < RT) {
            for (int w2 = 0; w2 < waves; ++w2) v += red[((size_t)w2 * RT + m) * kTileN + lane];
        }
        total[t] = v;
    }

    if (a.S > 1 && a.slots != nullptr) {
        // ---- exchange tree.  The slabs of a column tile are the leaves of a binary tree; at every level the
        // two children of a node meet in one 64-bit slot: each swaps (value, tag) into it with one atomic
        // exchange.  The child that finds the slot empty has left its partial there and is done; the one that
        // finds the other's partial adds it to its own (a sum of two floats does not depend on who came first),
        // empties the slot for the next launch and climbs.  The root stores the output.  Every thread decides for
        // its own output element: no ticket, no barrier, no polling, and the last arriver is log2(S) atomic
        // round trips from the end.  The sum order is the tree's, whatever the order of arrival.
        const size_t stride = (size_t)a.Mp * a.N;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int m = wv + t * waves;
            alive[t] = m < RT && col_ok;
            if (!alive[t]) continue;
            unsigned long long* lvl = a.slots + (size_t)(m0 + m) * a.N + n_out;
            float v = total[t];
            int node = split;
            for (int nodes = a.S; nodes > 1; nodes = (nodes + 1) >> 1) {
                const int pair = node >> 1;
                if ((node ^ 1) < nodes) {  // an odd node out climbs without meeting anybody
                    unsigned long long* slot = lvl + (size_t)pair * stride;
                    const unsigned long long mine = ((unsigned long long)kSlotValid << 32) | __builtin_bit_cast(uint32_t, v);
                    const unsigned long long was = __hip_atomic_exchange(slot, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if ((uint32_t)(was >> 32) != kSlotValid) {
                        alive[t] = false;
                        break;
                    }
                    v += __builtin_bit_cast(float, (uint32_t)was);
                    __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                lvl += (size_t)((nodes + 1) >> 1) * stride;
                node = pair;
            }
            total[t] = v;
        }
    } else if (a.S > 1) {
        // ---- plain protocol (partials too large for the slot region): publish this slab's partial, wait
        // for it to land, then take a ticket; the last slab to arrive sums all
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int m = wv + t * waves;
            if (m < RT && col_ok)
                __hip_atomic_store(a.partials + ((size_t)split * a.Mp + (m0 + m)) * a.N + n_out, total[t],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The partials were stored with agent scope (written through to the point every XCD reads
        // from), so waiting for their acknowledgement orders them before the ticket; a full release
        // fence would also write back the whole L2 and is far too expensive here.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0)
            ticket = __hip_atomic_fetch_add(a.counters + (size_t)(blockIdx.y * a.tiles + tile) * kCounterStride, 1u, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket != (unsigned)(a.S - 1)) return;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int m = wv + t * waves;
            float v = 0.0f;
            if (m < RT && col_ok) {
                const float* p = a.partials + (size_t)(m0 + m) * a.N + n_out;
                const size_t stride = (size_t)a.Mp * a.N;
                int sl = 0;
                for (; sl + 8 <= a.S; sl += 8) {  // loads of a batch are independent; the sum keeps slab order
                    float q[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        q[u] = __hip_atomic_load(p + (size_t)(sl + u) * stride, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int u = 0; u < 8; ++u) v += q[u];
                }
                for (; sl < a.S; ++sl)
                    v += __hip_atomic_load(p + (size_t)sl * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            total[t] = v;
        }
        if (tid == 0)
            __hip_atomic_store(a.counters + (size_t)(blockIdx.y * a.tiles + tile) * kCounterStride, 0u, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue: channel scales, cast, store
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int m = wv + t * waves;
        if (m >= RT || !col_ok || (m0 + m) >= a.M || !alive[t]) continue;
        float v = total[t];
        if (a.csm == GLA_CSM_WEIGHT) {
            v *= load_as_float(a.scales, a.meta_dt, n_out);
        } else if (a.csm == GLA_CSM_ACTIVATION) {
            v *= load_as_float(a.scales_x, a.sx_dt, (int64_t)(m0 + m) * a.sxm);
        } else if (a.csm == GLA_CSM_BOTH) {
            v *= load_as_float(a.scales_x, a.sx_dt, (int64_t)(m0 + m) * a.sxm) *
                 load_as_float(a.scales, a.meta_dt, n_out);
        }
        if (a.bias != nullptr) v = round_to_dtype(a.out_dt, v) + bias;  // `out += bias` on the rounded output
        store_from_float(a.out, a.out_dt, (int64_t)(m0 + m) * a.osm + n_out, v);
    }
}

// BITS: code width.  BF16: activation type.  RT: rows of x per pass (1, 2, 4 or 16).
// kWaves: waves per workgroup; 16 lets one workgroup own all of K with every load in flight at once.
template <int BITS, bool BF16, int RT, int kWaves>
__global__ __launch_bounds__(kWaves * 64) void gemv_packed_kernel(GemvArgs a) {
    constexpr int kThreads = kWaves * kWave;
    using SH = Shape<BITS>;
    constexpr int E = SH::E, LW = SH::LW, KPS = SH::KPS, T = SH::T;
    constexpr int RI = RT < 4 ? RT : 4;  // accumulator rows a lane folds
    constexpr uint32_t kPairMask = ((1u << BITS) - 1u) * 0x00010001u;
    constexpr float OFF = Magic<BF16>::off;

    extern __shared__ __align__(16) unsigned char smem[];
    const int SRW = a.RW / LW;                          // super rows per workgroup
    uint4* xs = (uint4*)smem;                           // [SRW][RT][T] A-operand chunks
    float2* mt = (float2*)(xs + (size_t)SRW * RT * T);  // [GW][64] (s, zz)
    float* red = (float*)(mt + (size_t)a.GW * kTileN);  // [kWaves][RT][64]
    __shared__ unsigned ticket;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wv = tid >> 6;
    const int cg = lane & 15, kb = lane >> 4;
    // grid (column tiles, row tiles, K slabs): nothing in front of the first load is divided at run time
    // (the wave's share of the slab and the group size as a shift come from the host)
    const int tile = blockIdx.x;
    const int split = blockIdx.z;
    const int m0 = blockIdx.y * RT;
    const int n0 = tile * kTileN;
    const int r0 = split * a.RW;
    const int SRWW = SRW / kWaves;  // super rows per wave
    const int nit = SRWW / 4;       // wave iterations (multiple of kBatch / LW)

    // ---- phase A: small loads first (activation chunk and metadata of the first staging pass)
    const int x_items = SRW * RT;
    const int sr_a = tid / RT, m_a = tid - sr_a * RT;
    uint4 xraw[T];
    const bool x_first = tid < x_items;
    bool x_valid = false;
    {
        // unconditional, clamped load: validity is applied when the chunk is written to LDS
        int row = r0 + sr_a * LW;
        int mrow = m0 + m_a;
        x_valid = x_first && row < a.R && mrow < a.M;
        if (row > a.R - LW) row = a.R - LW;
        if (mrow > a.M - 1) mrow = a.M - 1;
        const uint4* src = (const uint4*)((const uint16_t*)a.x + (int64_t)mrow * a.xsm + (int64_t)row * E);
#pragma unroll
        for (int t = 0; t < T; ++t) xraw[t] = src[t];
    }
    const int g0 = div_group(a, r0);
    const bool fast_meta = (a.meta_dt == GLA_DT_FP16 || a.meta_dt == GLA_DT_BF16) && !a.z_scalar &&
                           (a.z_dt == a.meta_dt) && a.wgm >= GLA_WGM_SHIFT_SCALE;
    uint2 sraw = make_uint2(0, 0), zraw = make_uint2(0, 0);
    const int gl_a = tid >> 4, c4_a = (tid & 15) * 4;
    const bool meta_first = fast_meta && gl_a < a.GW;
    if (fast_meta) {  // uniform branch; lanes past the table load a clamped row and drop it
        int g = g0 + gl_a;
        if (g > a.G - 1) g = a.G - 1;
        int n = n0 + c4_a;
        if (n > a.N - 4) n = a.N - 4;
        sraw = *(const uint2*)((const uint16_t*)a.scales + (int64_t)g * a.msg + n);
        zraw = *(const uint2*)((const uint16_t*)a.zeros + (int64_t)g * a.msg + n);
    }

    // ---- phase B: first batch of the weight stream
    int col = n0 + cg * 4;
    if (col > a.N - 4) col = a.N - 4;  // clamped lanes are never stored
    const uint32_t* wbase = a.w + col;
    const int lsr0 = wv * SRWW + kb;  // local super row of iteration 0
    uint4 buf[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
        int row = r0 + (lsr0 + 4 * (u / LW)) * LW + (u % LW);
        if (row > a.R - 1) row = a.R - 1;  // activation rows there are staged as zeros
        buf[u] = load_streaming_u4(wbase + (int64_t)row * a.wsk);
    }
    // keep every load above in flight before anything below consumes one of them
    __builtin_amdgcn_sched_barrier(0);

    // ---- phase C: fill LDS
    auto stage_x = [&](int sr, int m, bool valid, const uint4(&raw)[T]) {
        uint4* dst = xs + ((size_t)sr * RT + m) * T;
        if (!valid) {
#pragma unroll
            for (int t = 0; t < T; ++t) dst[t] = make_uint4(0, 0, 0, 0);
            return;
        }
        uint16_t v[KPS];
#pragma unroll
        for (int t = 0; t < T; ++t) ((uint4*)v)[t] = raw[t];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t o[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int lo, hi;
                if constexpr (E >= 8) {
                    lo = 4 * t + r;
                    hi = lo + E / 2;
                } else {  // 8-bit codes: register r pairs (j, j + 2) of word r / 2
                    lo = 4 * (r / 2) + (r % 2);
                    hi = lo + 2;
                }
                o[r] = (uint32_t)v[lo] | ((uint32_t)v[hi] << 16);
            }
            dst[t] = make_uint4(o[0], o[1], o[2], o[3]);
        }
    };
    if (x_first) stage_x(sr_a, m_a, x_valid, xraw);
    for (int idx = tid + kThreads; idx < x_items; idx += kThreads) {
        const int sr = idx / RT, m = idx - sr * RT;
        const int row = r0 + sr * LW;
        const bool valid = row < a.R && (m0 + m) < a.M;
        uint4 raw[T];
        if (valid) {
            const uint4* src = (const uint4*)((const uint16_t*)a.x + (int64_t)(m0 + m) * a.xsm + (int64_t)row * E);
#pragma unroll
            for (int t = 0; t < T; ++t) raw[t] = src[t];
        }
        stage_x(sr, m, valid, raw);
    }

    if (fast_meta) {
        auto stage_meta = [&](int gl, int c4, uint2 sr_, uint2 zr_) {
            const uint16_t sv[4] = {(uint16_t)(sr_.x & 0xffff), (uint16_t)(sr_.x >> 16), (uint16_t)(sr_.y & 0xffff),
                                    (uint16_t)(sr_.y >> 16)};
            const uint16_t zv[4] = {(uint16_t)(zr_.x & 0xffff), (uint16_t)(zr_.x >> 16), (uint16_t)(zr_.y & 0xffff),
                                    (uint16_t)(zr_.y >> 16)};
            float2 o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o[j] = fold_meta(meta_to_float(sv[j], a.meta_dt), meta_to_float(zv[j], a.meta_dt), a.wgm, OFF);
            float4* dst = (float4*)(mt + gl * kTileN + c4);
            dst[0] = make_float4(o[0].x, o[0].y, o[1].x, o[1].y);
            dst[1] = make_float4(o[2].x, o[2].y, o[3].x, o[3].y);
        };
        if (meta_first) stage_meta(gl_a, c4_a, sraw, zraw);
        for (int idx = tid + kThreads; idx < a.GW * 16; idx += kThreads) {
            const int gl = idx >> 4, c4 = (idx & 15) * 4;
            int g = g0 + gl;
            if (g > a.G - 1) g = a.G - 1;
            int n = n0 + c4;
            if (n > a.N - 4) n = a.N - 4;
            const uint2 s2 = *(const uint2*)((const uint16_t*)a.scales + (int64_t)g * a.msg + n);
            const uint2 z2 = *(const uint2*)((const uint16_t*)a.zeros + (int64_t)g * a.msg + n);
            stage_meta(gl, c4, s2, z2);
        }
    } else {
        for (int idx = tid; idx < a.GW * kTileN; idx += kThreads) {
            const int gl = idx / kTileN, c = idx - gl * kTileN;
            int g = g0 + gl;
            if (g > a.G - 1) g = a.G - 1;
            int n = n0 + c;
            if (n > a.N - 1) n = a.N - 1;
            float s = 1.0f, z = 0.0f;
            if (a.wgm >= GLA_WGM_SCALE) s = load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + n);
            if (a.wgm == GLA_WGM_SHIFT || a.wgm >= GLA_WGM_SHIFT_SCALE)
                z = a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0)
                               : load_as_float(a.zeros, a.z_dt, (int64_t)g * a.msg + n);
            mt[idx] = fold_meta(s, z, a.wgm, OFF);
        }
    }
    __syncthreads();

    // ---- main loop
    float acc[4][RI];
    float4_t c[4], csx;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        c[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < RI; ++i) acc[j][i] = 0.0f;
    }
    csx = float4_t{0.f, 0.f, 0.f, 0.f};
    const uint4 ones = make_uint4(Magic<BF16>::ones, Magic<BF16>::ones, Magic<BF16>::ones, Magic<BF16>::ones);
    const int mA = (RT == 16) ? cg : (cg & (RT - 1));  // rows >= RT of the A operand may hold anything
    constexpr int IPB = kBatch / LW;                   // wave iterations per batch of loads
    uint32_t pair_mask = kPairMask, magic = Magic<BF16>::bits;
    asm volatile("" : "+s"(pair_mask), "+v"(magic));  // keep both in registers, not literals
    const int fl_mask = a.FL - 1;                      // FL is a power of two

    for (int ib = 0; ib < nit; ib += IPB) {
        uint4 cur[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) cur[u] = buf[u];
        if (ib + IPB < nit) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                int row = r0 + (lsr0 + 4 * (ib + IPB + u / LW)) * LW + (u % LW);
                if (row > a.R - 1) row = a.R - 1;
                buf[u] = load_streaming_u4(wbase + (int64_t)row * a.wsk);
            }
        }
#pragma unroll
        for (int ii = 0; ii < IPB; ++ii) {
            const int it = ib + ii;
            const int lsr = lsr0 + 4 * it;
            const uint4* xa = xs + ((size_t)lsr * RT + mA) * T;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const uint4 av = xa[t];
                csx = mfma16<BF16>(av, ones, csx);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t b[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if constexpr (E >= 8) {
                            b[r] = and_or(pick(cur[ii], j) >> ((4 * t + r) * BITS), pair_mask, magic);
                        } else {
                            b[r] = and_or(pick(cur[ii * LW + r / 2], j) >> ((r % 2) * 8), pair_mask, magic);
                        }
                    }
                    c[j] = mfma16<BF16>(av, make_uint4(b[0], b[1], b[2], b[3]), c[j]);
                }
            }
            if (((it + 1) & fl_mask) == 0) {
                // group of this iteration: the four quarters' super rows lie in one group
                int gl = div_group(a, r0 + (wv * SRWW + 4 * it) * LW) - g0;
                if (gl > a.GW - 1) gl = a.GW - 1;
                const float4* mrow = (const float4*)(mt + gl * kTileN + cg * 4);
                const float4 m01 = mrow[0], m23 = mrow[1];
                const float sj[4] = {m01.x, m01.z, m23.x, m23.z};
                const float zj[4] = {m01.y, m01.w, m23.y, m23.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int i = 0; i < RI; ++i)
                        acc[j][i] = __builtin_fmaf(sj[j], c[j][i], __builtin_fmaf(zj[j], csx[i], acc[j][i]));
                    c[j] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
                csx = float4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
    }

    wg_finish<RT, kWaves, RI>(a, acc, red, ticket, tile, split, m0, n0);
}

// ---------------------------------------------------------------------------------------------
// Direct variant for 4- and 8-bit codes at M <= 4: no workgroup staging and no barrier before the
// stream.  Every wave loads, right ahead of its own weight words, the activation chunks those
// words meet (from L2) and the scales / zero points of its own groups (into a wave-private LDS
// table), so waves run independently until the final reduction and compute overlaps the stream.
// LOOP = false: exactly one batch of kBatch loads per lane (everything in flight at once).
// ---------------------------------------------------------------------------------------------
// kWaves = 0: the wave count is blockDim.x / 64, any number from 4 to 16 (row tiles up to 4), so that
// the K slabs of a column tile can be cut equal: 56 wave-batches are 4 slabs of 14 waves, not 16/16/16/8.
// FLC: wave iterations per fold when the host knows them to be 4 (the usual group of 128), else 0 (a.FL decides):
// with the folds at fixed places of the unrolled batch, the accumulators of a group start from the MFMA's zero
// operand instead of being cleared, and no branch stands between the iterations.
template <int BITS, bool BF16, int RT, int kWaves, bool LOOP, int FLC = 0>
__global__ __launch_bounds__(kWaves ? kWaves * 64 : 1024) void gemv_direct_kernel(GemvArgs a) {
    using SH = Shape<BITS>;
    constexpr int E = SH::E, LW = SH::LW, T = SH::T;  // T MFMA K-steps per super row (2 for 2-bit codes)
    static_assert(BITS == 2 || BITS == 4 || BITS == 8, "direct variant: 2-, 4- and 8-bit codes");
    constexpr int RI = RT < 4 ? RT : 4;  // accumulator rows a lane folds
    constexpr int IPB = kBatch / LW;  // wave iterations per batch
    // Up to 4 rows the 16 rows of the MFMA's A operand are mostly idle, so one activation load serves several
    // iterations: lane (quarter q, i) loads the chunk of iteration i / RT for row i % RT, and iteration u takes
    // its A operand from the lanes RT * u further up the row of 16 (a DPP move per register instead of a load
    // per iteration: an eighth of the activation requests at one row).
    constexpr bool XS = RT <= 4 && T == 1;
    constexpr int IPL = XS ? ((16 / RT) < IPB ? (16 / RT) : IPB) : 1;  // iterations per activation load
    constexpr int NXL = XS ? IPB / IPL : IPB * T;                       // activation loads per batch
    // 8-bit codes with bf16 activations: 128 + q is exact in bf16 only up to q = 127, so a code is fed as
    // two nibbles, q = lo + 16 hi: one MFMA multiplies x by 128 + lo, a second 16 x by 128 + hi, both into
    // the same accumulator, which then holds sum x q + 128 * 17 * sum x.
    constexpr bool SPLIT8 = BITS == 8 && BF16;
    constexpr uint32_t kPairMask = SPLIT8 ? 0x000F000Fu : ((1u << BITS) - 1u) * 0x00010001u;
    constexpr float OFF = SPLIT8 ? Magic<BF16>::off * 17.0f : Magic<BF16>::off;

    extern __shared__ __align__(16) unsigned char smem[];
    const int nfb = a.nfb;                                        // flush blocks per batch
    const int waves = kWaves ? kWaves : (int)(blockDim.x >> 6);
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // wave-uniform, kept in an SGPR
    float2* mtw = (float2*)smem + (size_t)wv * nfb * kTileN;                  // [nfb][64], this wave's
    float* red = (float*)((float2*)smem + (size_t)waves * nfb * kTileN);      // [waves][RT][64]
    __shared__ unsigned ticket;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int cg = lane & 15, kb = lane >> 4;
    // grid (column tiles, row tiles, K slabs): nothing in front of the first load is divided at run time
    // (the wave's share of the slab and the group size as a shift come from the host)
    const int tile = blockIdx.x;
    const int split = blockIdx.z;
    const int m0 = blockIdx.y * RT;
    const int n0 = tile * kTileN;
    const int r0 = split * a.RW;
    const int SRWW = a.srww;   // super rows per wave
    const int nit = SRWW / 4;  // wave iterations
    const int wrow0 = r0 + wv * SRWW * LW;  // first word row of this wave
    int g0w = div_group(a, wrow0);          // first group this wave touches
    if (g0w > a.G - 1) g0w = a.G - 1;

    int col = n0 + cg * 4;
    if (col > a.N - 4) col = a.N - 4;  // clamped lanes are never stored
    int mrow = m0 + (RT == 16 ? cg : (cg & (RT - 1)));  // rows >= RT of the A operand may hold anything
    if (mrow > a.M - 1) mrow = a.M - 1;
    // Every address of the stream is a wave-uniform 64-bit base (scalar arithmetic) plus a 32-bit lane
    // offset (the host has checked that a wave's span fits): one add and one clamp per load.  With 64-bit
    // products per load, the address arithmetic of the four waves of a SIMD stood in front of the later
    // loads of each for several hundred cycles.
    const uint32_t sb = (uint32_t)a.wsk * 4u;  // bytes between word rows
    const char* ws_base = (const char*)a.w + (int64_t)(wrow0 < a.R - 1 ? wrow0 : a.R - 1) * a.wsk * 4;
    const uint32_t w_lane = (uint32_t)col * 4u + (uint32_t)(kb * LW) * sb;
    const uint32_t w_lim = (uint32_t)col * 4u + (uint32_t)(wrow0 < a.R - 1 ? a.R - 1 - wrow0 : 0) * sb;
    const int x_rel_max = a.R - LW - wrow0;  // rows this wave may still multiply (negative: none)
    const char* xs_base = (const char*)a.x + (int64_t)(x_rel_max > 0 ? wrow0 : a.R - LW) * (E * 2);
    if constexpr (XS) {  // lane (kb, cg): row cg % RT of iteration cg / RT (lanes past the last iteration repeat)
        mrow = m0 + (cg % RT);
        if (mrow > a.M - 1) mrow = a.M - 1;
    }
    const uint32_t x_lane0 = (uint32_t)mrow * (uint32_t)a.xsm * 2u;
    const uint32_t x_lane = x_lane0 + (uint32_t)((XS ? 4 * ((cg / RT) % IPL) + kb : kb) * LW * E * 2);
    const uint32_t x_lim = x_lane0 + (uint32_t)(x_rel_max > 0 ? x_rel_max : 0) * (uint32_t)(E * 2);
    const char* ss_base = (const char*)a.scales + (int64_t)g0w * a.msg * 2;
    const char* zs_base = (const char*)a.zeros + (int64_t)g0w * a.msg * 2;
    const bool fast_meta = (a.meta_dt == GLA_DT_FP16 || a.meta_dt == GLA_DT_BF16) && !a.z_scalar &&
                           (a.z_dt == a.meta_dt) && a.wgm >= GLA_WGM_SHIFT_SCALE;

    struct Batch {
        uint2 sr[2], zr[2];
        uint4 xr[NXL];
        uint4 wr[kBatch];
        unsigned xvalid;  // bit u: activation load u of the batch lies inside K (a ragged last slab runs past it)
    };

    // group (relative to g0w) whose fold closes flush block `fbl` of the batch starting at iteration ib
    auto block_group = [&](int ib, int fbl) {
        const int it_f = (a.FL <= IPB) ? (ib + (fbl + 1) * a.FL - 1) : (ib + IPB - 1);
        int g = div_group(a, wrow0 + 4 * it_f * LW);
        if (g > a.G - 1) g = a.G - 1;
        return g;
    };

    // Order of a batch's requests: the first iteration's activation chunk and weight words, then the
    // scales / zero points, then the other iterations, each activation chunk right ahead of its weight
    // words.  The first weight request of a wave leaves after a handful of instructions (what stands in
    // front of it is added to the kernel's duration), and every iteration's operands are complete when its
    // weight words arrive.
    auto issue = [&](int ib, Batch& b) {
        b.xvalid = 0;
        if constexpr (XS) {
#pragma unroll
            for (int xl = 0; xl < NXL; ++xl) {
                uint32_t xo = x_lane + (uint32_t)(4 * (ib + xl * IPL) * LW * E * 2);
                if (x_rel_max >= 0 && xo <= x_lim) b.xvalid |= 1u << xl;
                else xo = x_lim;  // loads stay in bounds; the chunk is zeroed when it is used
                b.xr[xl] = *(const uint4*)(xs_base + xo);
            }
        }
        auto pair = [&](int u) __attribute__((always_inline)) {
            if constexpr (!XS) {
                uint32_t xo = x_lane + (uint32_t)(4 * (ib + u) * LW * E * 2);
                if (x_rel_max >= 0 && xo <= x_lim) b.xvalid |= 1u << u;
                else xo = x_lim;  // loads stay in bounds; the activations are zeroed when they are used
#pragma unroll
                for (int t = 0; t < T; ++t) b.xr[u * T + t] = *(const uint4*)(xs_base + xo + 16 * t);
            }
#pragma unroll
            for (int v = 0; v < LW; ++v) {
                uint32_t wo = w_lane + (uint32_t)(4 * (ib + u) * LW + v) * sb;
                if (wo > w_lim) wo = w_lim;
                b.wr[u * LW + v] = load_streaming_u4((const uint32_t*)(ws_base + wo));
            }
        };
        if (fast_meta) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int item = lane + 64 * p;
                int fbl = item >> 4;
                if (fbl > nfb - 1) fbl = nfb - 1;  // surplus lanes reload the last block and drop it
                const int g = block_group(ib, fbl);
                int n = n0 + (item & 15) * 4;
                if (n > a.N - 4) n = a.N - 4;
                if (p == 0 || nfb > 4) {
                    const uint32_t mo = (uint32_t)(g - g0w) * ((uint32_t)a.msg * 2u) + (uint32_t)n * 2u;
                    b.sr[p] = load_streaming_u2((const uint16_t*)(ss_base + mo));
                    b.zr[p] = load_streaming_u2((const uint16_t*)(zs_base + mo));
                }
            }
        }
#pragma unroll
        for (int u = 0; u < IPB; ++u) pair(u);
    };

    float acc[4][RI];
    float4_t c[4], csx;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        c[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < RI; ++i) acc[j][i] = 0.0f;
    }
    csx = float4_t{0.f, 0.f, 0.f, 0.f};
    uint4 ones = make_uint4(Magic<BF16>::ones, Magic<BF16>::ones, Magic<BF16>::ones, Magic<BF16>::ones);
    // four registers that stay put: left to itself the compiler builds the operand anew before every use
    asm volatile("" : "+v"(ones.x), "+v"(ones.y), "+v"(ones.z), "+v"(ones.w));
    uint32_t pair_mask = kPairMask, magic = Magic<BF16>::bits;
    asm volatile("" : "+s"(pair_mask), "+v"(magic));  // keep both in registers, not literals
    const int fl_mask = a.FL - 1;                      // FL is a power of two

    auto stage_meta = [&](int ib, const Batch& b) {
        if (fast_meta) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int item = lane + 64 * p;
                if ((p == 0 || nfb > 4) && item < nfb * 16) {
                    const uint32_t sw[2] = {b.sr[p].x, b.sr[p].y}, zw[2] = {b.zr[p].x, b.zr[p].y};
                    float2 o[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint16_t sv = (uint16_t)(sw[j >> 1] >> (16 * (j & 1)));
                        const uint16_t zv = (uint16_t)(zw[j >> 1] >> (16 * (j & 1)));
                        o[j] = fold_meta(meta_to_float(sv, a.meta_dt), meta_to_float(zv, a.meta_dt), a.wgm, OFF);
                    }
                    float4* dst = (float4*)(mtw + (item >> 4) * kTileN + (item & 15) * 4);
                    dst[0] = make_float4(o[0].x, o[0].y, o[1].x, o[1].y);
                    dst[1] = make_float4(o[2].x, o[2].y, o[3].x, o[3].y);
                }
            }
        } else {
            for (int idx = lane; idx < nfb * kTileN; idx += kWave) {
                const int fbl = idx / kTileN, cc = idx - fbl * kTileN;
                const int g = block_group(ib, fbl);
                int n = n0 + cc;
                if (n > a.N - 1) n = a.N - 1;
                float s = 1.0f, z = 0.0f;
                if (a.wgm >= GLA_WGM_SCALE) s = load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + n);
                if (a.wgm == GLA_WGM_SHIFT || a.wgm >= GLA_WGM_SHIFT_SCALE)
                    z = a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0)
                                   : load_as_float(a.zeros, a.z_dt, (int64_t)g * a.msg + n);
                mtw[idx] = fold_meta(s, z, a.wgm, OFF);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // chunk of 8 activations as loaded -> the pair order of the code extraction (one K-step)
    auto pair_order = [&](const uint4& xr) {
        uint4 av;
        if constexpr (E == 8) {  // pairs (j, j + 4)
            av.x = __builtin_amdgcn_perm(xr.z, xr.x, 0x05040100u);
            av.y = __builtin_amdgcn_perm(xr.z, xr.x, 0x07060302u);
            av.z = __builtin_amdgcn_perm(xr.w, xr.y, 0x05040100u);
            av.w = __builtin_amdgcn_perm(xr.w, xr.y, 0x07060302u);
        } else {  // two words of 4 codes: pairs (j, j + 2) inside each word
            av.x = __builtin_amdgcn_perm(xr.y, xr.x, 0x05040100u);
            av.y = __builtin_amdgcn_perm(xr.y, xr.x, 0x07060302u);
            av.z = __builtin_amdgcn_perm(xr.w, xr.z, 0x05040100u);
            av.w = __builtin_amdgcn_perm(xr.w, xr.z, 0x07060302u);
        }
        return av;
    };
    // 16 x: add 4 to the exponent of every non-zero bf16 half (zeros and denormals stay)
    auto times16 = [](uint32_t v) {
        const uint32_t lo_nz = (v & 0x00007f80u) ? 0x00000200u : 0u;
        const uint32_t hi_nz = (v & 0x7f800000u) ? 0x02000000u : 0u;
        return v + (lo_nz | hi_nz);
    };

    auto process = [&](int ib, const Batch& b) {
        stage_meta(ib, b);
        const uint4 zero4 = make_uint4(0, 0, 0, 0);
        // shared activation loads: zero what lies past K, order the pairs once per load
        uint4 xp[XS ? NXL : 1], xp16[XS ? NXL : 1];
        if constexpr (XS) {
#pragma unroll
            for (int xl = 0; xl < NXL; ++xl) {
                xp[xl] = pair_order(((b.xvalid >> xl) & 1u) ? b.xr[xl] : zero4);
                if constexpr (SPLIT8)
                    xp16[xl] = make_uint4(times16(xp[xl].x), times16(xp[xl].y), times16(xp[xl].z), times16(xp[xl].w));
            }
        }
#pragma unroll
        for (int ii = 0; ii < IPB; ++ii) {
            const int it = ib + ii;
            // first iteration after a fold: the accumulators start from zero (FLC: known at compile time)
#pragma unroll
            for (int t = 0; t < T; ++t) {
                uint4 av, av16;
                if constexpr (XS) {
                    av = row_down(xp[ii / IPL], RT * (ii % IPL));
                    if constexpr (SPLIT8) av16 = row_down(xp16[ii / IPL], RT * (ii % IPL));
                } else {
                    const bool xok = (b.xvalid >> ii) & 1u;
                    if constexpr (E == 16) {  // 16 codes per word: K-step t pairs (4t + r, 4t + r + 8)
                        const uint4 lo = xok ? b.xr[ii * T] : zero4, hi = xok ? b.xr[ii * T + 1] : zero4;
                        const uint32_t l0 = t ? lo.z : lo.x, l1 = t ? lo.w : lo.y, h0 = t ? hi.z : hi.x, h1 = t ? hi.w : hi.y;
                        av.x = __builtin_amdgcn_perm(h0, l0, 0x05040100u);
                        av.y = __builtin_amdgcn_perm(h0, l0, 0x07060302u);
                        av.z = __builtin_amdgcn_perm(h1, l1, 0x05040100u);
                        av.w = __builtin_amdgcn_perm(h1, l1, 0x07060302u);
                    } else {
                        av = pair_order(xok ? b.xr[ii] : zero4);
                    }
                    if constexpr (SPLIT8) av16 = make_uint4(times16(av.x), times16(av.y), times16(av.z), times16(av.w));
                }
                csx = mfma16<BF16>(av, ones, csx);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t bq[4], bh[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if constexpr (E >= 8) {
                            bq[r] = and_or(pick(b.wr[ii], j) >> ((4 * t + r) * BITS), pair_mask, magic);
                        } else {
                            bq[r] = and_or(pick(b.wr[ii * LW + r / 2], j) >> ((r % 2) * 8), pair_mask, magic);
                            if constexpr (SPLIT8)
                                bh[r] = and_or(pick(b.wr[ii * LW + r / 2], j) >> ((r % 2) * 8 + 4), pair_mask, magic);
                        }
                    }
                    c[j] = mfma16<BF16>(av, make_uint4(bq[0], bq[1], bq[2], bq[3]), c[j]);
                    if constexpr (SPLIT8) c[j] = mfma16<BF16>(av16, make_uint4(bh[0], bh[1], bh[2], bh[3]), c[j]);
                }
            }
            const bool fold_now = FLC ? ((ii + 1) % (FLC ? FLC : 1) == 0) : (((it + 1) & fl_mask) == 0);
            if (fold_now) {
                const int fbl = FLC ? ((ii + 1) / (FLC ? FLC : 1) - 1) : ((a.FL <= IPB) ? (((ii + 1) >> a.fl_log2) - 1) : 0);
                const float4* mrow = (const float4*)(mtw + fbl * kTileN + cg * 4);
                const float4 m01 = mrow[0], m23 = mrow[1];
                const float sj[4] = {m01.x, m01.z, m23.x, m23.z};
                const float zj[4] = {m01.y, m01.w, m23.y, m23.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int i = 0; i < RI; ++i)
                        acc[j][i] = __builtin_fmaf(sj[j], c[j][i], __builtin_fmaf(zj[j], csx[i], acc[j][i]));
                    c[j] = float4_t{0.f, 0.f, 0.f, 0.f};
                }
                csx = float4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
        __builtin_amdgcn_wave_barrier();  // the table is rewritten by the next batch
    };

    if constexpr (!LOOP) {
        Batch b;
        issue(0, b);
        __builtin_amdgcn_sched_barrier(0);
        process(0, b);
    } else {
        Batch nxt;
        issue(0, nxt);
        for (int ib = 0; ib < nit; ib += IPB) {
            const Batch cur = nxt;
            if (ib + IPB < nit) issue(ib + IPB, nxt);
            __builtin_amdgcn_sched_barrier(0);
            process(ib, cur);
        }
    }
    wg_finish<RT, kWaves, RI>(a, acc, red, ticket, tile, split, m0, n0);
}

// Rows per workgroup: 3 and 4 rows take the 4-row tile (its cross-wave buffer and reduction are a quarter of
// the 16-row tile's: 8192^2 4-bit at M=4 12.0 -> 10.3 us, 14336 -> 4096 10 % faster).
int row_tile(int M) { return M >= 5 ? 16 : (M >= 3 ? 4 : (M == 2 ? 2 : 1)); }

struct Geometry {
    int E, LW, KPS, T, R, RW, S, tiles, RT, mchunks, Mp, gr, G, GW, FL, waves, unit, nb, nfb;
    bool direct;  // 4/8-bit codes at M <= 4: the variant without workgroup staging
    size_t smem;
};

// tile_config encoding: (waves per workgroup) * 1000 + (batches of kBatch loads per wave).
bool geometry(const gla_matmul_args& p, Geometry& g, bool allow_direct = true, int rt_cap = 16) {
    g.E = 32 / p.W_nbits;
    g.LW = g.E < 8 ? 8 / g.E : 1;
    g.KPS = g.E * g.LW;
    g.T = g.KPS / 8;
    g.R = p.K / g.E;
    g.tiles = ceil_div(p.N, kTileN);
    g.RT = row_tile(p.M);
    if (g.RT > rt_cap) g.RT = rt_cap;
    g.mchunks = ceil_div(p.M, g.RT);
    g.Mp = g.mchunks * g.RT;
    const bool grouped = p.W_group_mode >= GLA_WGM_SCALE || (p.W_group_mode == GLA_WGM_SHIFT && !p.zero_is_scalar);
    const int gs = grouped ? p.group_size : p.K;
    // every K-block of one MFMA step must lie in one group
    const int k_per_iter = 4 * g.KPS;
    if (gs % k_per_iter != 0) return false;
    g.gr = gs / g.E;
    g.G = p.K / gs;
    // one wave, one batch: 4 quarters x kBatch loads of word rows
    g.unit = 4 * kBatch;
    const int units = ceil_div(g.R, g.unit);  // wave-batches along K
    // 2-bit codes: direct for the 16-row tile, and up to 4 rows on layers of up to 64 M weights, where a launch is short
    // and the staged kernel's fill of its LDS tables stands in front of the stream (bf16, groups of 64, one row: 8192^2
    // 10.5 -> 8.9 us, 4096^2 7.2 -> 5.8, at 4 rows 12.6 -> 9.7 and 8.5 -> 6.7; 16384^2 27 -> 32, so larger layers stay
    // staged).  Its 2-bit instantiations fit the register file at 4 and 8 waves only.
    const bool w2_short = p.W_nbits == 2 && g.RT <= 4 && (int64_t)p.N * p.K <= ((int64_t)1 << 26);
    const bool can_direct = allow_direct && (p.W_nbits == 4 || p.W_nbits == 8 || (p.W_nbits == 2 && g.RT == 16) || w2_short);
    // the cross-wave buffer is [waves][RT][64] floats; the staged 16-row kernel runs 4 waves
    int max_waves = (g.RT == 16) ? (can_direct ? 16 : 4) : (w2_short && can_direct ? 8 : 16);
    // Large layers: once 8-wave workgroups still give every CU two or more, they stream better than
    // 16-wave ones (measured on 16384^2: 4-bit 27.9 against 32.2 us, 8-bit 44 against 53 us).
    if (max_waves > 8 && (int64_t)g.tiles * ceil_div(p.M, g.RT) * ceil_div(units, 8) >= 512) max_waves = 8;
    // ... and 2-bit codes at the 16-row tile better still with 4 (35.5 against 43.6 us)
    if (p.W_nbits == 2 && g.RT == 16 && max_waves > 4 && (int64_t)g.tiles * ceil_div(p.M, g.RT) * ceil_div(units, 4) >= 512)
        max_waves = 4;
    int waves, nb;
    if (p.tile_config >= 1000) {
        waves = p.tile_config / 1000;
        nb = p.tile_config % 1000;
        const bool any_count = can_direct && !w2_short && nb == 1 && waves >= (g.RT <= 4 ? 4 : 8) && waves <= 16;
        if (!(waves == 4 || waves == 8 || waves == 16 || any_count) || waves > max_waves || nb < 1) return false;
    } else {
        // Slabs along K: enough workgroups to cover the CUs, and few enough wave-batches per
        // workgroup that every load of the kernel is in flight at once (one batch per wave).
        // A chip's worth of workgroups (256 CUs) unless the column tiles alone nearly give that: with
        // 200+ tiles a second slab buys little bandwidth and costs the combining round trip.
        const int cols = g.tiles * g.mchunks;
        int s_min = cols >= 192 ? 1 : ceil_div(g.RT <= 4 ? 256 : 128, cols);  // the 16-row tile: half as many, larger workgroups
        int want_s = ceil_div(units, max_waves);
        if (want_s < s_min) want_s = s_min;
        if (want_s > units) want_s = units;
        int per_wg = ceil_div(units, want_s);  // wave-batches per workgroup
        if (can_direct && per_wg <= max_waves && (g.RT <= 4 || per_wg > 8)) {
            // one batch per wave and exactly as many waves as batches: equal slabs
            waves = per_wg < 4 ? 4 : (w2_short && per_wg > 4 ? 8 : per_wg);
            nb = 1;
        } else {
            waves = per_wg <= 4 ? 4 : (per_wg <= 8 && max_waves >= 8 ? 8 : max_waves);
            nb = ceil_div(per_wg, waves);
        }
    }
    g.direct = can_direct;
    if (g.direct && nb > 1 && waves != 4) {  // the looping direct variant runs 4 waves
        nb *= waves / 4;
        waves = 4;
    }
    const int it_per_group = gs / k_per_iter;
    for (;;) {
        g.waves = waves;
        g.nb = nb;
        g.RW = waves * nb * g.unit;
        g.GW = g.RW / g.gr + 2;
        // iterations per flush: whole groups, at most 1024 K-values between folds
        const int nit = g.RW / g.LW / waves / 4;
        int fl = 1;
        // ... at most 64 when an int32 accumulator was asked for (integer-valued activations, widened from int8):
        // |x| <= 127 times 1024 + q over 64 K-values (128 for 1-bit codes) stays below 2^24, so every fp32 sum is exact
        const int fold_k = p.acc_dtype == GLA_DT_INT32 ? 64 : 1024;
        while (fl * 2 * k_per_iter <= fold_k && it_per_group % (fl * 2) == 0 && nit % (fl * 2) == 0) fl *= 2;
        g.FL = fl;
        const int ipb = kBatch / g.LW;
        g.nfb = fl >= ipb ? 1 : ipb / fl;
        if (g.direct)
            g.smem = (size_t)waves * g.nfb * kTileN * 8 + (size_t)waves * g.RT * kTileN * 4;
        else
            g.smem = (size_t)(g.RW / g.LW) * g.RT * g.T * 16 + (size_t)g.GW * kTileN * 8 +
                     (size_t)waves * g.RT * kTileN * 4;
        if (g.smem <= (g.direct && g.RT == 16 ? 100 : 60) * 1024) break;
        if (nb > 1) {
            --nb;
        } else if (waves > 4) {
            waves = waves > 8 ? 8 : 4;
        } else {
            // the staged 16-row tile of 1-bit codes does not fit the LDS at any wave count (its activation
            // chunk alone is 1 KiB per super row): more rows than 4 then run as chunks of 4
            if (g.RT == 16) return geometry(p, g, allow_direct, 4);
            return false;
        }
    }
    g.S = ceil_div(g.R, g.RW);
    if (g.direct) {
        // the direct variant addresses with a 64-bit base per wave plus 32-bit lane offsets
        const int64_t lim = (int64_t)1 << 31;
        const int64_t w_span = (int64_t)p.w_stride_k * 4 * (g.RW / g.waves) + (int64_t)p.N * 4;
        const int64_t x_span = (int64_t)p.x_stride_m * 2 * 16 + (int64_t)p.K * 2;
        const int64_t m_span = (int64_t)p.meta_stride_g * 2 * g.GW + (int64_t)p.N * 2;
        if (p.w_stride_k < 0 || p.x_stride_m < 0 || p.meta_stride_g < 0 || w_span >= lim || x_span >= lim || m_span >= lim)
            return geometry(p, g, false, rt_cap);
    }
    // 8-bit codes with bf16 activations exist only in the direct variant (nibble-split MFMAs)
    const bool split8 = p.W_nbits == 8 && p.input_dtype == GLA_DT_BF16;
    if (split8 && !g.direct) return false;
    // a ragged last slab is fine in either variant: rows past K multiply zeroed activations
    if (g.S > 1 && (int64_t)g.tiles * g.mchunks * kCounterStride * 4 > kCounterBytes) return false;
    return true;
}

// The single-batch direct kernel at the wave count the geometry chose.
template <int BITS, bool BF16, int RT, int FLC>
void launch_direct(const GemvArgs& a, const Geometry& g, dim3 grid, hipStream_t stream) {
    if (g.waves == 16) {
        if constexpr (RT == 16) {  // its cross-wave buffer alone is 64 KiB
            static DeviceOnce once;
            if (once.first())
                (void)hipFuncSetAttribute((const void*)gemv_direct_kernel<BITS, BF16, RT, 16, false, FLC>,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024);
        }
        hipLaunchKernelGGL((gemv_direct_kernel<BITS, BF16, RT, 16, false, FLC>), grid, dim3(1024), g.smem, stream, a);
    } else if (g.waves == 8) {
        hipLaunchKernelGGL((gemv_direct_kernel<BITS, BF16, RT, 8, false, FLC>), grid, dim3(512), g.smem, stream, a);
    } else if (g.waves == 4) {
        hipLaunchKernelGGL((gemv_direct_kernel<BITS, BF16, RT, 4, false, FLC>), grid, dim3(256), g.smem, stream, a);
    } else {
        if constexpr (RT == 16) {  // a cross-wave buffer of up to 60 KiB
            static DeviceOnce once;
            if (once.first())
                (void)hipFuncSetAttribute((const void*)gemv_direct_kernel<BITS, BF16, RT, 0, false, FLC>,
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024);
        }
        hipLaunchKernelGGL((gemv_direct_kernel<BITS, BF16, RT, 0, false, FLC>), grid, dim3(g.waves * 64), g.smem, stream, a);
    }
}

template <int BITS, bool BF16, int RT>
void launch_one(const GemvArgs& a, const Geometry& g, hipStream_t stream) {
    dim3 grid(g.tiles, g.mchunks, g.S);
    if constexpr (BITS == 2 || BITS == 4 || BITS == 8) {
        if (g.direct) {
            if (g.nb > 1) {
                hipLaunchKernelGGL((gemv_direct_kernel<BITS, BF16, RT, 4, true>), grid, dim3(256), g.smem, stream, a);
                return;
            }
            if constexpr (BITS == 4 || BITS == 8) {
                if (g.FL == 4) {  // groups of 128 (and channel-wise 8-bit codes): folds at fixed places of the batch
                    launch_direct<BITS, BF16, RT, 4>(a, g, grid, stream);
                    return;
                }
            }
            if constexpr (BITS == 2) {
                // 2-bit codes in groups of 64: a fold after every iteration, so that the group sums start from the MFMA's
                // zero operand instead of being cleared (16384^2 at 16 rows 36.0-37.0 -> 32.7-33.5 us, 8192^2 17.5 -> 16.8).
                // (The same in the staged kernel, which serves up to 4 rows: 16384^2 at one row 26.7 -> 35 us; not kept.)
                if (g.FL == 1) {
                    launch_direct<BITS, BF16, RT, 1>(a, g, grid, stream);
                    return;
                }
            }
            launch_direct<BITS, BF16, RT, 0>(a, g, grid, stream);
            return;
        }
    }
    if constexpr (RT == 16) {
        hipLaunchKernelGGL((gemv_packed_kernel<BITS, BF16, RT, 4>), grid, dim3(256), g.smem, stream, a);
    } else {
        if (g.waves == 16)
            hipLaunchKernelGGL((gemv_packed_kernel<BITS, BF16, RT, 16>), grid, dim3(1024), g.smem, stream, a);
        else if (g.waves == 8)
            hipLaunchKernelGGL((gemv_packed_kernel<BITS, BF16, RT, 8>), grid, dim3(512), g.smem, stream, a);
        else
            hipLaunchKernelGGL((gemv_packed_kernel<BITS, BF16, RT, 4>), grid, dim3(256), g.smem, stream, a);
    }
}

template <int BITS, bool BF16>
void launch_rt(const GemvArgs& a, const Geometry& g, hipStream_t stream) {
    switch (g.RT) {
        case 1: launch_one<BITS, BF16, 1>(a, g, stream); break;
        case 2: launch_one<BITS, BF16, 2>(a, g, stream); break;
        case 4: launch_one<BITS, BF16, 4>(a, g, stream); break;
        default: launch_one<BITS, BF16, 16>(a, g, stream); break;
    }
}

template <bool BF16>
void launch_bits(const GemvArgs& a, const Geometry& g, int bits, hipStream_t stream) {
    switch (bits) {
        case 1: launch_rt<1, BF16>(a, g, stream); break;
        case 2: launch_rt<2, BF16>(a, g, stream); break;
        case 4: launch_rt<4, BF16>(a, g, stream); break;
        default: launch_rt<8, BF16>(a, g, stream); break;
    }
}

}  // namespace

bool gemv_packed_eligible(const gla_matmul_args& p) {
    if (p.w_dtype != GLA_DT_INT32) return false;
    if (!(p.W_nbits == 1 || p.W_nbits == 2 || p.W_nbits == 4 || p.W_nbits == 8)) return false;
    if (p.elements_per_sample * p.W_nbits != 32) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16)) return false;
    // (an int32 accumulator with 16-bit activations is the library's own call for widened int8 activations)
    if (!(p.acc_dtype == GLA_DT_FP32 || p.acc_dtype == GLA_DT_INT32)) return false;
    if (p.W_group_mode < 0 || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.channel_scale_mode < 0 || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32))
        return false;
    if (p.N < 4 || p.N % 4 != 0 || p.w_stride_n != 1 || p.w_stride_k % 4 != 0) return false;
    if (p.x_stride_k != 1 || p.x_stride_m % 8 != 0 || p.out_stride_n != 1) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    const int E = 32 / p.W_nbits;
    const int KPS = E < 8 ? 8 : E;
    if (p.K % KPS != 0) return false;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if (uses_scales && (p.scales == nullptr || p.meta_stride_n != 1)) return false;
    if (uses_zeros && p.zeros == nullptr) return false;
    if (uses_zeros && !p.zero_is_scalar && p.meta_stride_n != 1) return false;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    if (grouped && (p.group_size < E || p.K % p.group_size != 0)) return false;
    const bool one_group = !grouped || p.group_size == p.K;  // then the stride between groups is never used
    if (grouped && ((uses_scales && ((uintptr_t)p.scales & 7)) ||
                    (uses_zeros && !p.zero_is_scalar && ((uintptr_t)p.zeros & 7)) ||
                    (!one_group && p.meta_stride_g % 4 != 0)))
        return false;
    if ((p.channel_scale_mode & 1) && p.scales == nullptr) return false;
    if ((p.channel_scale_mode & 2) && p.scales_x == nullptr) return false;
    Geometry g;
    return geometry(p, g);
}

int gemv_packed_default_config(const gla_matmul_args& p) {
    Geometry g;
    gla_matmul_args q = p;
    q.tile_config = -1;
    if (!geometry(q, g)) return -1;
    return g.waves * 1000 + g.nb;
}

// Tagged slots when they fit the region no other kernel writes; else fp32 partials behind it.
static bool slots_fit(const Geometry& g, const gla_matmul_args& p) {
    return (int64_t)g.S * g.Mp * p.N * 8 <= kSlotBytes;
}

int64_t gemv_packed_workspace_bytes(const gla_matmul_args& p) {
    Geometry g;
    if (!geometry(p, g)) return 0;
    if (g.S <= 1) return 0;
    return slots_fit(g, p) ? kWsPrivateBytes : kWsPrivateBytes + (int64_t)g.S * g.Mp * p.N * 4;
}

int launch_gemv_packed(const gla_matmul_args& p, hipStream_t stream) {
    Geometry g;
    if (!geometry(p, g)) {
        set_error("gemv_packed: shape does not fit the kernel's tiling or LDS budget");
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    GemvArgs a;
    a.w = (const uint32_t*)p.w; a.x = p.x; a.scales = p.scales; a.zeros = p.zeros; a.scales_x = p.scales_x;
    a.out = p.out; a.partials = nullptr; a.slots = nullptr; a.counters = nullptr;
    a.bias = p.bias; a.bias_dt = p.bias_dtype;
    if (g.S > 1) {
        const int64_t need = gemv_packed_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemv_packed: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.counters = (unsigned*)p.workspace;
        if (slots_fit(g, p)) a.slots = (unsigned long long*)((char*)p.workspace + kCounterBytes);
        else a.partials = (float*)((char*)p.workspace + kWsPrivateBytes);
    }
    a.M = p.M; a.N = p.N; a.K = p.K; a.R = g.R; a.RW = g.RW; a.S = g.S; a.tiles = g.tiles; a.Mp = g.Mp;
    a.gr = g.gr; a.G = g.G; a.GW = g.GW; a.FL = g.FL; a.waves = g.waves; a.nfb = g.nfb;
    a.srww = g.RW / g.LW / g.waves;
    a.gr_shift = (g.gr & (g.gr - 1)) == 0 ? __builtin_ctz((unsigned)g.gr) : -1;
    a.fl_log2 = 0;
    while ((1 << a.fl_log2) < g.FL) ++a.fl_log2;
    a.wgm = p.W_group_mode; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.z_dt = p.zeros_dtype;
    a.z_scalar = p.zero_is_scalar; a.out_dt = p.output_dtype; a.sx_dt = p.sx_dtype;
    a.wsk = p.w_stride_k; a.xsm = p.x_stride_m; a.osm = p.out_stride_m; a.msg = p.meta_stride_g;
    a.sxm = p.sx_stride_m;
    if (p.input_dtype == GLA_DT_BF16) launch_bits<true>(a, g, p.W_nbits, stream);
    else launch_bits<false>(a, g, p.W_nbits, stream);
    return check_hip(hipGetLastError(), "gemv_packed launch");
}

}  // namespace gla
