// Streaming GEMV for 32-bit packed weight words stored [K/e, N], N fastest.
//
// Takes the place of the reference's GEMV / RevSplit-K kernels for packed data
// (reference: gemlite/triton_kernels/gemv_revsplitK_kernels.py:248-443 and
// gemlite/triton_kernels/gemv_kernels.py:245-426), with a different
// decomposition:
//
//  * A workgroup (4 waves) owns 64 output columns and a slab of RW word rows.
//    In every wave a lane owns 4 adjacent columns (one 128-bit load) and the
//    four 16-lane quarters own four consecutive word rows, so one wave load
//    covers 4 rows x 256 contiguous bytes.
//  * Codes are never dequantised one by one.  Within a quantisation group the
//    lane accumulates dq = sum_k x_k * (OFF + q_k) with v_dot2 on fp16/bf16
//    pairs built by OR-ing the code bits into the mantissa of the constant
//    OFF (1024 in fp16, 128 in bf16), and sx = sum_k x_k.  At the group end
//    acc += s * dq + zz * sx, where (s, zz) folds the scale, the zero point
//    and -OFF*s in fp32.  All five dequant modes reduce to a choice of (s, zz).
//  * The activation slab, its per-row sums and the (s, zz) table of the slab
//    are staged in LDS once per workgroup, so every global load of the kernel
//    is issued up front.
//  * The K reduction is deterministic: quarters by wave shuffles, waves through
//    LDS, slabs by fp32 partials in a workspace that the last-arriving
//    workgroup of a column tile sums in slab order (no float atomics).
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

constexpr int kWaves = 4;        // waves per workgroup
constexpr int kThreads = kWaves * kWave;
constexpr int kTileN = 64;       // output columns per workgroup
constexpr int kBatch = 8;        // 128-bit loads in flight per lane
constexpr int kSlabRows = kWaves * kBatch * 4;  // 128: granularity of RW
constexpr int64_t kCounterBytes = 256 * 1024;   // fixed ticket-counter region at the start of the workspace

struct GemvArgs {
    const uint32_t* w;
    const void* x;
    const void* scales;
    const void* zeros;
    const void* scales_x;
    void* out;
    float* partials;
    unsigned* counters;
    int M, N, K;
    int R;        // word rows = K / E
    int RW;       // word rows per workgroup (multiple of kSlabRows)
    int S;        // number of slabs along K
    int tiles;    // column tiles
    int Mp;       // M rounded up to the row-tile
    int gr;       // word rows per quantisation group (>= 1)
    int G;        // number of groups along K
    int GW;       // (s, zz) table rows staged per workgroup
    int FL;       // loads per flush
    int wgm, csm, meta_dt, z_dt, z_scalar, out_dt, sx_dt;
    int64_t wsk, xsm, osm, msg, sxm;
};

template <bool BF16>
struct Magic;
template <>
struct Magic<false> {
    static constexpr uint32_t bits = 0x64006400u;  // fp16 1024.0 twice
    static constexpr float off = 1024.0f;
};
template <>
struct Magic<true> {
    static constexpr uint32_t bits = 0x43004300u;  // bf16 128.0 twice
    static constexpr float off = 128.0f;
};

template <bool BF16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    if constexpr (BF16) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c,
                                               false);
    } else {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
    }
}

__device__ __forceinline__ float elem16_to_float(uint16_t v, bool bf16) {
    return bf16 ? bf16_bits_to_float(v) : half_bits_to_float(v);
}

// BITS: code width.  BF16: activation type.  MT: rows of x per workgroup.
// F32: convert codes and activations to fp32 and use FMAs (8-bit codes with
// bf16 activations, where OFF + q is not exact in bf16).
template <int BITS, bool BF16, int MT, bool F32>
__global__ __launch_bounds__(kThreads) void gemv_packed_kernel(GemvArgs a) {
    constexpr int E = 32 / BITS;       // codes per word
    constexpr int XW = F32 ? E : E / 2;  // 32-bit LDS words per staged activation row
    constexpr uint32_t kPairMask = ((1u << BITS) - 1u) * 0x00010001u;
    constexpr float OFF = F32 ? 0.0f : Magic<BF16>::off;

    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* xs = (uint32_t*)smem;                        // [MT][RW][XW]
    float* rs = (float*)(xs + (size_t)MT * a.RW * XW);       // [MT][RW]
    float2* mt = (float2*)(rs + (size_t)MT * a.RW);          // [GW][64]
    float* red = (float*)(mt + (size_t)a.GW * kTileN);       // [kWaves][MT][64]
    __shared__ unsigned ticket;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wv = tid >> 6;
    const int cg = lane & 15, rg = lane >> 4;
    const int tile = blockIdx.x % a.tiles;
    const int split = blockIdx.x / a.tiles;
    const int m0 = blockIdx.y * MT;
    const int n0 = tile * kTileN;
    const int r0 = split * a.RW;
    const int RWW = a.RW / kWaves;
    const int nl = RWW / 4;  // loads per lane (multiple of kBatch)

    // ---- weight stream: first batch of loads goes out before anything else
    int col = n0 + cg * 4;
    if (col > a.N - 4) col = a.N - 4;  // clamped lanes are never stored
    const uint32_t* wbase = a.w + col;
    const int lrow0 = wv * RWW + rg;  // local row of load 0
    uint4 buf[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
        int row = r0 + lrow0 + 4 * u;
        if (row > a.R - 1) row = a.R - 1;  // activation rows there are staged as zeros
        buf[u] = *(const uint4*)(wbase + (int64_t)row * a.wsk);
    }

    // ---- stage the activation slab (permuted for the pair extraction) and row sums
    for (int idx = tid; idx < MT * a.RW; idx += kThreads) {
        const int m = idx / a.RW, rl = idx - m * a.RW;
        const int row = r0 + rl;
        uint32_t* dst = xs + (size_t)idx * XW;
        float sum = 0.0f;
        if (row < a.R && (m0 + m) < a.M) {
            const uint16_t* src = (const uint16_t*)a.x + (int64_t)(m0 + m) * a.xsm + (int64_t)row * E;
            uint16_t v[E];
            if constexpr (E == 4) {
                *(uint2*)v = *(const uint2*)src;
            } else {
#pragma unroll
                for (int q = 0; q < E / 8; ++q) ((uint4*)v)[q] = ((const uint4*)src)[q];
            }
#pragma unroll
            for (int j = 0; j < E; ++j) sum += elem16_to_float(v[j], BF16);
            if constexpr (F32) {
#pragma unroll
                for (int j = 0; j < E; ++j) dst[j] = __builtin_bit_cast(uint32_t, elem16_to_float(v[j], BF16));
            } else {
#pragma unroll
                for (int j = 0; j < E / 2; ++j) dst[j] = (uint32_t)v[j] | ((uint32_t)v[j + E / 2] << 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < XW; ++j) dst[j] = 0u;
        }
        rs[idx] = sum;
    }

    // ---- stage the (s, zz) table of this slab
    const int g0 = r0 / a.gr;
    for (int idx = tid; idx < a.GW * kTileN; idx += kThreads) {
        const int gl = idx / kTileN, c = idx - gl * kTileN;
        int g = g0 + gl;
        if (g > a.G - 1) g = a.G - 1;
        int n = n0 + c;
        if (n > a.N - 1) n = a.N - 1;
        float s = 1.0f, z = 0.0f;
        if (a.wgm >= GLA_WGM_SCALE) s = load_as_float(a.scales, a.meta_dt, (int64_t)g * a.msg + n);
        if (a.wgm == GLA_WGM_SHIFT || a.wgm >= GLA_WGM_SHIFT_SCALE)
            z = a.z_scalar ? load_as_float(a.zeros, a.z_dt, 0) : load_as_float(a.zeros, a.z_dt, (int64_t)g * a.msg + n);
        float zz;
        switch (a.wgm) {
            case GLA_WGM_SHIFT: zz = -z - OFF; break;
            case GLA_WGM_SCALE: zz = -OFF * s; break;
            case GLA_WGM_SHIFT_SCALE: zz = -(z + OFF) * s; break;
            case GLA_WGM_FMA: zz = __builtin_fmaf(-OFF, s, z); break;
            default: zz = -OFF; break;
        }
        mt[idx] = make_float2(s, zz);
    }
    __syncthreads();

    // ---- main loop
    float acc[4][MT], dq[4][MT], sx[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        sx[m] = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) { acc[c][m] = 0.0f; dq[c][m] = 0.0f; }
    }

    for (int ib = 0; ib < nl; ib += kBatch) {
        uint4 cur[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) cur[u] = buf[u];
        if (ib + kBatch < nl) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                int row = r0 + lrow0 + 4 * (ib + kBatch + u);
                if (row > a.R - 1) row = a.R - 1;
                buf[u] = *(const uint4*)(wbase + (int64_t)row * a.wsk);
            }
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int i = ib + u;
            const int rl = lrow0 + 4 * i;
            uint32_t xv[MT][XW];
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const uint32_t* src = xs + ((size_t)m * a.RW + rl) * XW;
                if constexpr (XW == 2) {
                    *(uint2*)xv[m] = *(const uint2*)src;
                } else {
#pragma unroll
                    for (int q = 0; q < XW / 4; ++q) ((uint4*)xv[m])[q] = ((const uint4*)src)[q];
                }
                sx[m] += rs[m * a.RW + rl];
            }
            const uint32_t wq[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if constexpr (F32) {
#pragma unroll
                    for (int j = 0; j < E; ++j) {
                        const float q = (float)((wq[c] >> (j * BITS)) & ((1u << BITS) - 1u));
#pragma unroll
                        for (int m = 0; m < MT; ++m)
                            dq[c][m] = __builtin_fmaf(q, __builtin_bit_cast(float, xv[m][j]), dq[c][m]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < E / 2; ++j) {
                        const uint32_t t = ((wq[c] >> (j * BITS)) & kPairMask) | Magic<BF16>::bits;
#pragma unroll
                        for (int m = 0; m < MT; ++m) dq[c][m] = dot2<BF16>(t, xv[m][j], dq[c][m]);
                    }
                }
            }
            if ((i + 1) % a.FL == 0) {
                int gl = (r0 + rl) / a.gr - g0;
                if (gl > a.GW - 1) gl = a.GW - 1;
                const float2* mrow = mt + gl * kTileN + cg * 4;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float2 sz = mrow[c];
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        acc[c][m] = __builtin_fmaf(sz.x, dq[c][m], __builtin_fmaf(sz.y, sx[m], acc[c][m]));
                        dq[c][m] = 0.0f;
                    }
                }
#pragma unroll
                for (int m = 0; m < MT; ++m) sx[m] = 0.0f;
            }
        }
    }

    // ---- reduce the four row quarters of each wave, then the waves
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = acc[c][m];
            v += wave_xor(v, 16);
            v += wave_xor(v, 32);
            acc[c][m] = v;
        }
    if (rg == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            *(float4*)(red + ((size_t)wv * MT + m) * kTileN + cg * 4) =
                make_float4(acc[0][m], acc[1][m], acc[2][m], acc[3][m]);
    }
    __syncthreads();

    const int n_out = n0 + (tid & 63);
    float total[(MT + kWaves - 1) / kWaves];
#pragma unroll
    for (int t = 0; t < (MT + kWaves - 1) / kWaves; ++t) {
        const int m = wv + t * kWaves;
        float v = 0.0f;
        if (m < MT) {
#pragma unroll
            for (int w2 = 0; w2 < kWaves; ++w2) v += red[((size_t)w2 * MT + m) * kTileN + (tid & 63)];
        }
        total[t] = v;
    }

    const bool col_ok = n_out < a.N;
    if (a.S > 1) {
        // publish this slab's partial, then take a ticket; the last slab to arrive sums all
#pragma unroll
        for (int t = 0; t < (MT + kWaves - 1) / kWaves; ++t) {
            const int m = wv + t * kWaves;
            if (m < MT && col_ok)
                __hip_atomic_store(a.partials + ((size_t)split * a.Mp + (m0 + m)) * a.N + n_out, total[t],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // The partials were stored with agent scope (written through to the point every XCD reads
        // from), so waiting for their acknowledgement orders them before the ticket; a full release
        // fence would also write back the whole L2 and is far too expensive here.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0)
            ticket = __hip_atomic_fetch_add(a.counters + blockIdx.y * a.tiles + tile, 1u, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket != (unsigned)(a.S - 1)) return;
#pragma unroll
        for (int t = 0; t < (MT + kWaves - 1) / kWaves; ++t) {
            const int m = wv + t * kWaves;
            float v = 0.0f;
            if (m < MT && col_ok) {
                for (int s = 0; s < a.S; ++s)
                    v += __hip_atomic_load(a.partials + ((size_t)s * a.Mp + (m0 + m)) * a.N + n_out, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
            }
            total[t] = v;
        }
        if (tid == 0)
            __hip_atomic_store(a.counters + blockIdx.y * a.tiles + tile, 0u, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue: channel scales, cast, store
#pragma unroll
    for (int t = 0; t < (MT + kWaves - 1) / kWaves; ++t) {
        const int m = wv + t * kWaves;
        if (m >= MT || !col_ok || (m0 + m) >= a.M) continue;
        float v = total[t];
        if (a.csm == GLA_CSM_WEIGHT) {
            v *= load_as_float(a.scales, a.meta_dt, n_out);
        } else if (a.csm == GLA_CSM_ACTIVATION) {
            v *= load_as_float(a.scales_x, a.sx_dt, (int64_t)(m0 + m) * a.sxm);
        } else if (a.csm == GLA_CSM_BOTH) {
            v *= load_as_float(a.scales_x, a.sx_dt, (int64_t)(m0 + m) * a.sxm) *
                 load_as_float(a.scales, a.meta_dt, n_out);
        }
        store_from_float(a.out, a.out_dt, (int64_t)(m0 + m) * a.osm + n_out, v);
    }
}

int row_tile(int M) { return M >= 8 ? 8 : (M >= 3 ? 4 : (M == 2 ? 2 : 1)); }

struct Geometry {
    int E, R, RW, S, tiles, MT, mchunks, Mp, gr, G, GW, FL;
    size_t smem;
};

bool geometry(const gla_matmul_args& p, Geometry& g) {
    g.E = 32 / p.W_nbits;
    g.R = p.K / g.E;
    g.tiles = ceil_div(p.N, kTileN);
    g.MT = row_tile(p.M);
    g.mchunks = ceil_div(p.M, g.MT);
    g.Mp = g.mchunks * g.MT;
    const bool grouped = p.W_group_mode >= GLA_WGM_SCALE || (p.W_group_mode == GLA_WGM_SHIFT && !p.zero_is_scalar);
    const int gs = grouped ? p.group_size : p.K;
    g.gr = gs / g.E;
    if (g.gr < 1) return false;
    g.G = p.K / gs;

    int slabs = ceil_div(g.R, kSlabRows);
    int per_wg;
    if (p.tile_config > 0) {
        per_wg = p.tile_config;
    } else {
        // enough workgroups to fill 256 CUs about four times over, then as few slabs as possible
        int want = ceil_div(1024, g.tiles * g.mchunks);
        if (want < 1) want = 1;
        if (want > slabs) want = slabs;
        per_wg = ceil_div(slabs, want);
    }
    if (per_wg > slabs) per_wg = slabs;
    // LDS budget: activation slab + row sums + (s, zz) table + wave partials
    for (;; --per_wg) {
        g.RW = per_wg * kSlabRows;
        g.GW = g.RW / g.gr + 2;
        const size_t xw = (p.W_nbits == 8 && p.input_dtype == GLA_DT_BF16) ? g.E : g.E / 2;
        g.smem = (size_t)g.MT * g.RW * xw * 4 + (size_t)g.MT * g.RW * 4 + (size_t)g.GW * kTileN * 8 +
                 (size_t)kWaves * g.MT * kTileN * 4;
        if (g.smem <= 60 * 1024) break;
        if (per_wg == 1) return false;
    }
    g.S = ceil_div(g.R, g.RW);
    if (g.S > 1 && (int64_t)g.tiles * g.mchunks * 4 > kCounterBytes) return false;
    const int nl = g.RW / kWaves / 4;
    int fl = 1;
    if (g.gr >= 4 && g.gr % 4 == 0) {
        const int flmax = g.gr / 4;
        while (fl < 16 && flmax % (fl * 2) == 0 && nl % (fl * 2) == 0) fl *= 2;
    }
    g.FL = fl;
    return true;
}

template <int BITS, bool BF16, int MT>
void launch_one(const GemvArgs& a, const Geometry& g, hipStream_t stream) {
    dim3 grid(g.tiles * g.S, g.mchunks);
    constexpr bool F32 = (BITS == 8) && BF16;
    hipLaunchKernelGGL((gemv_packed_kernel<BITS, BF16, MT, F32>), grid, dim3(kThreads), g.smem, stream, a);
}

template <int BITS, bool BF16>
void launch_mt(const GemvArgs& a, const Geometry& g, hipStream_t stream) {
    switch (g.MT) {
        case 1: launch_one<BITS, BF16, 1>(a, g, stream); break;
        case 2: launch_one<BITS, BF16, 2>(a, g, stream); break;
        case 4: launch_one<BITS, BF16, 4>(a, g, stream); break;
        default: launch_one<BITS, BF16, 8>(a, g, stream); break;
    }
}

template <bool BF16>
void launch_bits(const GemvArgs& a, const Geometry& g, int bits, hipStream_t stream) {
    switch (bits) {
        case 1: launch_mt<1, BF16>(a, g, stream); break;
        case 2: launch_mt<2, BF16>(a, g, stream); break;
        case 4: launch_mt<4, BF16>(a, g, stream); break;
        default: launch_mt<8, BF16>(a, g, stream); break;
    }
}

}  // namespace

bool gemv_packed_eligible(const gla_matmul_args& p) {
    if (p.w_dtype != GLA_DT_INT32) return false;
    if (!(p.W_nbits == 1 || p.W_nbits == 2 || p.W_nbits == 4 || p.W_nbits == 8)) return false;
    if (p.elements_per_sample * p.W_nbits != 32) return false;
    if (!(p.input_dtype == GLA_DT_FP16 || p.input_dtype == GLA_DT_BF16)) return false;
    if (p.acc_dtype != GLA_DT_FP32) return false;
    if (p.W_group_mode < 0 || p.W_group_mode > GLA_WGM_FMA) return false;
    if (p.channel_scale_mode < 0 || p.channel_scale_mode > GLA_CSM_BOTH) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32))
        return false;
    if (p.N < 4 || p.N % 4 != 0 || p.w_stride_n != 1 || p.w_stride_k % 4 != 0) return false;
    if (p.x_stride_k != 1 || p.x_stride_m % 8 != 0 || p.out_stride_n != 1) return false;
    if (((uintptr_t)p.w & 15) || ((uintptr_t)p.x & 15)) return false;
    const int E = 32 / p.W_nbits;
    if (p.K % E != 0) return false;
    const bool uses_scales = p.W_group_mode >= GLA_WGM_SCALE;
    const bool uses_zeros = p.W_group_mode == GLA_WGM_SHIFT || p.W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if (uses_scales && (p.scales == nullptr || p.meta_stride_n != 1)) return false;
    if (uses_zeros && p.zeros == nullptr) return false;
    if (uses_zeros && !p.zero_is_scalar && p.meta_stride_n != 1) return false;
    const bool grouped = uses_scales || (uses_zeros && !p.zero_is_scalar);
    if (grouped && (p.group_size < E || p.group_size % E != 0 || p.K % p.group_size != 0)) return false;
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
    return g.RW / kSlabRows;
}

int64_t gemv_packed_workspace_bytes(const gla_matmul_args& p) {
    Geometry g;
    if (!geometry(p, g)) return 0;
    if (g.S <= 1) return 0;
    return kCounterBytes + (int64_t)g.S * g.Mp * p.N * 4;
}

int launch_gemv_packed(const gla_matmul_args& p, hipStream_t stream) {
    Geometry g;
    if (!geometry(p, g)) {
        set_error("gemv_packed: shape does not fit the kernel's LDS budget");
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    GemvArgs a;
    a.w = (const uint32_t*)p.w; a.x = p.x; a.scales = p.scales; a.zeros = p.zeros; a.scales_x = p.scales_x;
    a.out = p.out; a.partials = nullptr; a.counters = nullptr;
    if (g.S > 1) {
        const int64_t need = gemv_packed_workspace_bytes(p);
        if (p.workspace == nullptr || (int64_t)p.workspace_bytes < need) {
            set_error("gemv_packed: workspace of %lld bytes required, %llu given", (long long)need,
                      (unsigned long long)p.workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        a.counters = (unsigned*)p.workspace;
        a.partials = (float*)((char*)p.workspace + kCounterBytes);
    }
    a.M = p.M; a.N = p.N; a.K = p.K; a.R = g.R; a.RW = g.RW; a.S = g.S; a.tiles = g.tiles; a.Mp = g.Mp;
    a.gr = g.gr; a.G = g.G; a.GW = g.GW; a.FL = g.FL;
    a.wgm = p.W_group_mode; a.csm = p.channel_scale_mode; a.meta_dt = p.meta_dtype; a.z_dt = p.zeros_dtype;
    a.z_scalar = p.zero_is_scalar; a.out_dt = p.output_dtype; a.sx_dt = p.sx_dtype;
    a.wsk = p.w_stride_k; a.xsm = p.x_stride_m; a.osm = p.out_stride_m; a.msg = p.meta_stride_g;
    a.sxm = p.sx_stride_m;
    if (p.input_dtype == GLA_DT_BF16) launch_bits<true>(a, g, p.W_nbits, stream);
    else launch_bits<false>(a, g, p.W_nbits, stream);
    return check_hip(hipGetLastError(), "gemv_packed launch");
}

}  // namespace gla
