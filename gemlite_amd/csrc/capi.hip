// C ABI of the library: argument validation, kernel-family choice, error strings.
// Entry points are declared and documented in include/gemlite_amd.h.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return GLA_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return GLA_ERR_LAUNCH_FAILED;
}

namespace {

bool is_mx(int dt) { return dt >= 14 && dt <= 18; }

int closest_m(int M) {
    // {2^i} plus 0.75*2^i and 1.5*2^i for 2^i >= 32, capped at 4096; next value >= M
    if (M > 4096) return 4096;
    int best = 4096;
    for (int i = 0; i <= 12; ++i) {
        const int p = 1 << i;
        const int cands[3] = {p, (p >= 32 && 2 * p <= 4096) ? (3 * p) / 4 : p, (p >= 32 && 2 * p <= 4096) ? (3 * p) / 2 : p};
        for (int c : cands)
            if (c >= M && c < best) best = c;
    }
    return best;
}

int matmul_type_for(int M, int W_nbits, int mx) {
    if (M >= 64) return GLA_MATMUL_GEMM;
    const int gemv_limit = (W_nbits < 8 && !mx) ? 4 : 2;
    if (M > gemv_limit) return GLA_MATMUL_GEMM_SPLITK;
    if (mx) return GLA_MATMUL_GEMM_SPLITK;
    return W_nbits < 8 ? GLA_MATMUL_GEMV_REVSPLITK : GLA_MATMUL_GEMV_SPLITK;
}

constexpr int kMxStreamRows = 2;  // MXFP4 x MXFP4: rows up to which the streaming kernel is chosen

enum Family { F_GENERIC = 0, F_GEMV_PACKED, F_GEMV_KMAJOR, F_GEMM_WN, F_GEMM_8BIT, F_GEMM_MXFP4, F_GEMM_KBYTES, F_GEMM_MXFP8, F_MX_STREAM, F_BLOCKQ_STREAM, F_GEMM_BLOCKQ, F_GEMM_KBYTES_MX, F_MX_SKINNY, F_K_SKINNY, F_WN_MID, F_GEMM_16BIT };

int validate_operands(const gla_matmul_args* p) {
    if (p == nullptr) {
        set_error("matmul: args is NULL");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (p->struct_size != sizeof(gla_matmul_args)) {
        set_error("matmul: struct_size %u does not match the library's %zu", p->struct_size, sizeof(gla_matmul_args));
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (p->M < 0 || p->N <= 0 || p->K <= 0) {
        set_error("matmul: bad shape M=%d N=%d K=%d", p->M, p->N, p->K);
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (p->x == nullptr || p->w == nullptr || p->out == nullptr) {
        if (p->M == 0) return GLA_OK;
        set_error("matmul: x, w and out must not be NULL");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (p->bias != nullptr) {
        const int odt = p->output_dtype;
        const bool float_out = odt == GLA_DT_FP32 || odt == GLA_DT_FP16 || odt == GLA_DT_BF16 || odt == GLA_DT_MXFP16 || odt == GLA_DT_MXBF16;
        const bool float_bias = p->bias_dtype == GLA_DT_FP32 || p->bias_dtype == GLA_DT_FP16 || p->bias_dtype == GLA_DT_BF16;
        if (!float_out || !float_bias) {
            set_error("matmul: a bias needs a floating-point output (type %d) and an fp16, bf16 or fp32 bias (type %d)", odt, p->bias_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
        }
    }
    if (p->matmul_type < GLA_MATMUL_AUTO || p->matmul_type > GLA_MATMUL_GEMM) {
        set_error("matmul: matmul_type %d out of range", p->matmul_type);
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    if (p->elements_per_sample < 1 || p->K % p->elements_per_sample != 0) {
        set_error("matmul: K=%d not divisible by elements_per_sample=%d", p->K, p->elements_per_sample);
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    if (is_mx(p->input_dtype)) {  // every micro-scaled kernel stores fp32, fp16 or bf16
        int odt = p->output_dtype;
        if (odt == GLA_DT_MXFP16) odt = GLA_DT_FP16;  // the reference's weight-only MX processors say it this way
        if (odt == GLA_DT_MXBF16) odt = GLA_DT_BF16;
        if (odt != GLA_DT_FP32 && odt != GLA_DT_FP16 && odt != GLA_DT_BF16) {
            set_error("matmul: micro-scaled inputs need an fp32, fp16 or bf16 output (type %d)", p->output_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
        }
    }
    if (p->input_dtype == GLA_DT_MXFP4) {
        if (p->K % 32 != 0) {
            set_error("matmul: MXFP4 needs K %% 32 == 0 (K=%d)", p->K);
            return GLA_ERR_MISALIGNED_SHAPE;
        }
        return GLA_OK;
    }
    if (p->input_dtype == GLA_DT_MXFP16 || p->input_dtype == GLA_DT_MXBF16) {
        if (!mx_stream_eligible(*p)) {
            set_error("matmul: weight-only MX layers need K-contiguous fp8 bytes or e2m1 nibble pairs with one e8m0 scale "
                      "per 32 values, K %% 32 == 0, 16-byte aligned rows and channel_scale_mode 0 (K=%d, mode %d)",
                      p->K, p->channel_scale_mode);
            return GLA_ERR_UNSUPPORTED_MODE;
        }
        return GLA_OK;
    }
    if (p->input_dtype == GLA_DT_MXFP8) {
        if (!gemm_mxfp8_eligible(*p) && !mx_stream_eligible(*p)) {
            set_error("matmul: MXFP8 needs fp8 weight bytes with K-contiguous e8m0 scales per 32 values, K %% 128 == 0, "
                      "16-byte aligned rows and channel_scale_mode 2 or 4 (K=%d, mode %d)", p->K, p->channel_scale_mode);
            return GLA_ERR_UNSUPPORTED_MODE;
        }
        return GLA_OK;
    }
    if (is_mx(p->input_dtype)) {
        set_error("matmul: micro-scaled input type %d is not supported (MXFP16, MXBF16, MXFP8 and MXFP4 only)", p->input_dtype);
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    switch (p->input_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_FP8: case GLA_DT_INT8: break;
        default:
            set_error("matmul: input type %d not supported", p->input_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    switch (p->output_dtype) {
        case GLA_DT_FP32: case GLA_DT_FP16: case GLA_DT_BF16: case GLA_DT_INT32: break;
        default:
            set_error("matmul: output type %d not supported", p->output_dtype);
            return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    if (p->acc_dtype != GLA_DT_FP32 && p->acc_dtype != GLA_DT_INT32) {
        set_error("matmul: accumulator type %d not supported (fp32 or int32)", p->acc_dtype);
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    if (p->acc_dtype == GLA_DT_INT32 && p->input_dtype != GLA_DT_INT8) {
        set_error("matmul: int32 accumulation needs int8 activations");
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    if (p->W_group_mode < GLA_WGM_NONE || p->W_group_mode > GLA_WGM_FMA) {
        set_error("matmul: W_group_mode %d out of range", p->W_group_mode);
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    if (p->channel_scale_mode == GLA_CSM_BLOCK) {
        if (!blockq_stream_eligible(*p)) {
            set_error("matmul: channel_scale_mode 5 needs int8 or fp8 operands of one type, both K-contiguous with 16-byte "
                      "aligned rows, K %% 128 == 0, W_group_mode 0 and fp32 block scales on both sides (K=%d)", p->K);
            return GLA_ERR_UNSUPPORTED_MODE;
        }
        return GLA_OK;
    }
    if (p->channel_scale_mode < GLA_CSM_NONE || p->channel_scale_mode > GLA_CSM_BOTH) {
        set_error("matmul: channel_scale_mode %d not supported for this input type", p->channel_scale_mode);
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    const bool need_s = p->W_group_mode >= GLA_WGM_SCALE || (p->channel_scale_mode & 1);
    const bool need_z = p->W_group_mode == GLA_WGM_SHIFT || p->W_group_mode >= GLA_WGM_SHIFT_SCALE;
    if ((need_s && p->scales == nullptr) || (need_z && p->zeros == nullptr) ||
        ((p->channel_scale_mode & 2) && p->scales_x == nullptr && !p->x_quant_from)) {
        set_error("matmul: mode (W_group_mode=%d, channel_scale_mode=%d) needs a tensor that is NULL",
                  p->W_group_mode, p->channel_scale_mode);
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (p->W_group_mode != GLA_WGM_NONE && !(p->W_group_mode == GLA_WGM_SHIFT && p->zero_is_scalar)) {
        if (p->group_size < 1 || p->K % p->group_size != 0) {
            set_error("matmul: K=%d not divisible by group_size=%d", p->K, p->group_size);
            return GLA_ERR_MISALIGNED_SHAPE;
        }
    }
    return GLA_OK;
}

Family choose(const gla_matmul_args& p, int type);
int resolve_type(const gla_matmul_args& p);

// Operand checks, then: a call that asks for its activations to be quantised inside the matmul must land on a kernel
// that does it (the others would read the 16-bit rows as codes).
int validate(const gla_matmul_args* p) {
    const int rc = validate_operands(p);
    if (rc != GLA_OK || p->x_quant_from == 0 || p->M == 0) return rc;
    if (!(p->x_quant_from == GLA_DT_FP16 || p->x_quant_from == GLA_DT_BF16)) {
        set_error("matmul: x_quant_from %d: activations are quantised on the fly from fp16 or bf16 rows only", p->x_quant_from);
        return GLA_ERR_UNSUPPORTED_DTYPE;
    }
    const Family f = choose(*p, resolve_type(*p));
    const bool per_token = f == F_GEMV_KMAJOR && (p->input_dtype == GLA_DT_FP8 || p->input_dtype == GLA_DT_INT8);
    const bool mxfp4 = f == F_MX_STREAM && p->input_dtype == GLA_DT_MXFP4 && mx_stream_quantises(*p);
    // ... and only where the same call on ready-made codes would take that kernel too: a batch the matrix-core GEMM
    // serves better is not kept on the streaming kernel for the sake of the quantiser
    gla_matmul_args q = *p;
    q.x_quant_from = 0;
    q.x = (const void*)(uintptr_t)256;         // stand-ins for aligned code and scale arrays
    q.scales_x = (const void*)(uintptr_t)256;
    const bool mx = p->input_dtype == GLA_DT_MXFP4;
    q.x_stride_m = mx ? (p->K / 2 + 15) / 16 * 16 : (p->K + 15) / 16 * 16;
    q.sx_dtype = mx ? GLA_DT_UINT8 : GLA_DT_FP32;
    q.sx_stride_m = mx ? p->K / 32 : 1;
    q.sx_stride_g = 1;
    const bool same = choose(q, resolve_type(q)) == f;
    if (!((per_token || mxfp4) && same)) {
        set_error("matmul: no kernel quantises the activations inside the matmul for this call (M=%d N=%d K=%d, input type %d, "
                  "channel_scale_mode %d): the streaming kernels do, for the first rows of per-token fp8 / int8 and MXFP4 layers; "
                  "run the quantiser launch first", p->M, p->N, p->K, p->input_dtype, p->channel_scale_mode);
        return GLA_ERR_UNSUPPORTED_MODE;
    }
    return GLA_OK;
}

Family choose(const gla_matmul_args& p, int type) {
    // what the caller (or the tuner's cache) prefers where a streaming kernel and a matrix-core GEMM both take the call
    const bool want_stream = p.tile_config == GLA_TILE_PREFER_STREAMING, want_matrix = p.tile_config == GLA_TILE_PREFER_MATRIX;
    if (p.input_dtype == GLA_DT_MXFP4) {
        // Three kernels.  The streaming kernel (dot products on the vector unit; also the one that quantises 16-bit rows
        // itself) for 1-2 rows.  From 3 to 32 rows the weights go as they are into the scaled MFMA, copied to LDS by
        // whole 128-byte lines: no K split, no finishing or scale-regrouping launch (8 / 32 rows: 4096^2 4.7 / 6.5 us
        // against 14.1 / 15.3 of the tiled GEMM, 16384^2 34.3 / 41.2 against 41.0 / 44.4; 3 rows on 4096^2: 4.7 against
        // 9.9 of the streaming kernel).  Above 32 rows the tiled GEMM.
        const int64_t wbytes = (int64_t)p.N * p.K / 2;
        const bool stream_ok = p.tile_config < 1000 && mx_stream_eligible(p), matrix_ok = gemm_mxfp4_eligible(p);
        if (want_stream && stream_ok) return F_MX_STREAM;
        if (want_matrix && matrix_ok) return F_GEMM_MXFP4;
        if (p.M >= 3 && p.M <= 32 && p.tile_config < 1000 && kring_eligible(p)) return F_K_SKINNY;
        // K not a multiple of 256 (or operands the skinny kernel does not take): the streaming kernel up to 2 rows
        // everywhere, up to 4 on layers of 40 MB or less (4096^2 at 4 rows: 10.7 against 14.4 us of the tiled GEMM;
        // 16384^2: 54 against 40)
        const int rows = wbytes <= 40000000 ? 4 : kMxStreamRows;
        if (p.M <= rows && stream_ok) return F_MX_STREAM;
        return matrix_ok ? F_GEMM_MXFP4 : (mx_stream_eligible(p) ? F_MX_STREAM : F_GENERIC);
    }
    if (p.input_dtype == GLA_DT_MXFP8) {  // validated: eligible for one of the two at least
        // fp8 activations on MXFP8 or MXFP4 weights: up to 4 rows the streaming kernel is the faster one at every size
        // (MXFP8 weights, one row: 4096^2 7.9 against 25 us, 16384^2 59 against 84; 4 rows: 13.4 against 25, 79 against
        // 83.  MXFP4 weights, 4 rows: 4096^2 10.4 against 19.8, 16384^2 52 against 54; 6 rows: 85 against 54)
        const bool stream_ok = p.tile_config < 1000 && mx_stream_eligible(p), matrix_ok = gemm_mxfp8_eligible(p);
        if (want_stream && stream_ok) return F_MX_STREAM;
        if (want_matrix && matrix_ok) return F_GEMM_MXFP8;
        // from 3 rows both operands go into the scaled MFMA as they are, copied to LDS by lines, in one launch
        // (two activation tiles, 17..32 rows: only where N is short, as for fp8 x fp8)
        if (p.M >= 3 && p.M <= 32 && (p.M <= 16 || p.N < 7040) && p.tile_config < 1000 && kring_eligible(p)) return F_K_SKINNY;
        if (p.M <= 4 && stream_ok) return F_MX_STREAM;
        return matrix_ok ? F_GEMM_MXFP8 : F_MX_STREAM;
    }
    if (p.input_dtype == GLA_DT_MXFP16 || p.input_dtype == GLA_DT_MXBF16)  // validated as eligible for the streaming kernel
    {
        // 1-2 rows: the streaming kernel; up to 16 rows the weights still go straight into registers, to the
        // matrix cores (16384^2 MXFP4, 8 rows: 48 against 62 us of the tiled GEMM); above that the tiled GEMM
        if (want_stream) return F_MX_STREAM;
        if (want_matrix && gemm_kbytes_mx_eligible(p)) return F_GEMM_KBYTES_MX;
        // ... unless the activations go as sums of e4m3 terms (two per bf16 value, three per fp16 value) into the skinny
        // kernel of the narrow formats, which converts no weight: a small launch in front, so it pays on large layers
        // while the terms of the batch fit one 16-row tile (bf16: 8 rows, fp16: 5), and with two tiles on long-K layers.
        // Measured against the kernel below, 8 rows of bf16: MXFP4 16384^2 48.9 -> 40.8 us, 8192 x 28672 48.7 -> 39.4,
        // 4096 x 14336 17.7 -> 13.2, 14336 x 4096 16.2 -> 14.1, 8192^2 16.5 -> 15.5, 4096^2 6.8 -> 8.6 (stays); MXFP8 8192 x
        // 28672 85.5 -> 73.5, 4096 x 14336 27.1 -> 23.2, 8192^2 27.2 -> 25.3, 16384^2 78.3 -> 78.7 and 14336 x 4096 22.1 -> 23.0
        // (stay); 16 rows of bf16: 4096 x 14336 20.7 -> 17.6, 8192 x 28672 54.7 -> 49.2, 16384^2 51.6 -> 57.9 (stays).
        // GLA_TILE_PREFER_MID asks for it wherever it is eligible.
        if (p.M > 2 && p.M <= 16 && p.tile_config < 1000 && kring_eligible(p)) {
            const int terms = p.input_dtype == GLA_DT_MXBF16 ? 2 : 3;
            const bool one_tile = terms * p.M <= 16, w4 = p.elements_per_sample == 2;
            const bool long_k = p.K >= 14336 && p.N <= 8192;
            const bool pays = one_tile ? (w4 ? (int64_t)p.N * p.K >= 50000000 : (p.K >= 8192 && p.N <= 8192))
                                       : (terms == 2 && long_k);
            if (p.tile_config == GLA_TILE_PREFER_MID || pays) return F_K_SKINNY;
        }
        if (p.M > 2 && p.M <= 16 && p.tile_config < 1000 && mx_skinny_eligible(p)) return F_MX_SKINNY;
        return gemm_kbytes_mx_eligible(p) ? F_GEMM_KBYTES_MX : F_MX_STREAM;
    }
    if (p.channel_scale_mode == GLA_CSM_BLOCK)  // validated as eligible for the streaming kernel at least
        return (gemm_blockq_eligible(p) && !want_stream) ? F_GEMM_BLOCKQ : F_BLOCKQ_STREAM;
    // Up to 16 rows the streaming kernels win whatever type was asked for; above that the MFMA GEMMs.
    // fp8 x fp8 and int8 x int8 at 3..32 rows: operands as they are into the MFMA, one launch (between the vector
    // streaming kernel and the tiled GEMM with its split K and finishing launch)
    // (4096^2 fp8 at 8 / 32 rows: 7.1 / 9.3 against 13.8 / 14.8 us; 8192^2 at 8 rows 17.3 against 21.2; 16384^2 58.6 against
    // 74.6; 3 rows on 4096^2: 7.0 against 13.3 of the streaming kernel.  With two activation tiles, 17..32 rows, the
    // tiled GEMM is ahead from N = 7040: 8192^2 22.2 against 23.8, 14336 x 4096 20.4 against 24.0)
    if (p.M >= 3 && p.M <= 32 && (p.M <= 16 || p.N < 7040) && !want_matrix && p.tile_config < 1000 &&
        !(want_stream && gemv_kmajor_eligible(p)) && kring_eligible(p))
        return F_K_SKINNY;
    // a tile_config that names the mid-batch kernel: -4, or waves per workgroup (4 or 8) + 1000 * K splits
    const bool mid_asked = p.tile_config == GLA_TILE_PREFER_MID || (p.tile_config > 0 && (p.tile_config % 1000 == 4 || p.tile_config % 1000 == 8));
    if (mid_asked && wn_mid_eligible(p)) return F_WN_MID;
    const bool small = !want_matrix && (type <= GLA_MATMUL_GEMV_SPLITK || p.M <= 16 || want_stream);
    if (small) {
        // 8-bit codes on large layers: the mid-batch kernel reads the weights once for all rows and shares the
        // activations through LDS, where the GEMV has every wave fetch its own and, under bf16, feeds a byte as two
        // nibbles.  From 5 rows on layers of 128 M weights (16384 x 8192 at 5 / 16 rows: 29.8 / 30.9 against 37.5 / 39.3 us;
        // 8192 x 16384: 33.5 against 38-40; below 5 rows and on 8192^2 the GEMV is level or ahead), at any row count
        // from 256 M weights (16384^2 at 1 / 4 / 16 rows: 49.7 / 51.0 / 48.8 against 54.1 / 56.1 / 72.9)
        const int64_t weights = (int64_t)p.N * p.K;
        // (a caller that names a GEMV type gets the GEMV)
        const bool big8 = p.W_nbits == 8 && !want_stream && p.tile_config <= 0 &&
                          (type > GLA_MATMUL_GEMV_SPLITK || p.matmul_type == GLA_MATMUL_AUTO) &&
                          (weights >= ((int64_t)1 << 28) || (p.M >= 5 && weights >= ((int64_t)1 << 27)));
        if (big8 && wn_mid_eligible(p)) return F_WN_MID;
        if (gemv_packed_eligible(p)) return F_GEMV_PACKED;
        if (gemv_kmajor_eligible(p)) return F_GEMV_KMAJOR;
    }
    // Above 16 rows the streaming GEMV still runs, as row chunks of 16 that each stream the weights again (the later
    // chunks mostly from L2).  It is the only fast kernel for packed layers the tiled GEMM does not take (1-bit codes,
    // groups of 32, K not a multiple of 64), and up to 64 rows it beats the tiled GEMM on small and medium layers,
    // where that one cannot fill the chip without a deep K split (4096^2 4-bit at 32 rows: 9 against 17 us; 8192^2:
    // 22 against 26 us; 16384^2: 69 against 56 us, so large layers stay with the GEMM).
    // 17..64 rows of 8-bit codes on large layers: weights from registers into the MFMA, activations shared through LDS
    // (16384^2 at 32 / 64 rows: 56 / 70 us against 66 / 78 of the tiled GEMM; 8192^2: 26 / 31 against 27 / 32, left there)
    if (p.M > 16 && p.M <= 64 && p.W_nbits == 8 && (int64_t)p.N * p.K >= ((int64_t)1 << 27) && !want_matrix && !want_stream &&
        p.tile_config <= 0 && wn_mid_eligible(p))
        return F_WN_MID;
    if (p.M > 16 && gemv_packed_eligible(p)) {
        // groups of 32, which the tiled GEMM does not take: the mid-batch kernel (row chunks of 64) once the GEMV's
        // chunks of 16 have re-read the weights often enough (4-bit gs 32, 8192^2 at 64 / 256 rows: 36 / 85 against
        // 42 / 164 us; 4096^2: 23 / 36 against 15 / 43)
        if (!gemm_wn_eligible(p) && !want_stream && p.tile_config <= 0 && (p.M > 64 || (int64_t)p.N * p.K >= ((int64_t)1 << 26)) &&
            wn_mid_eligible(p))
            return F_WN_MID;
        if (!gemm_wn_eligible(p)) return F_GEMV_PACKED;
        const int64_t chunks = (p.M + 15) / 16;
        const int64_t restreamed = chunks * (int64_t)p.N * p.K * (p.W_nbits < 4 ? 4 : p.W_nbits) / 8;  // 2-bit codes cost what 4-bit ones do
        if (!want_matrix && p.tile_config <= 0 && chunks <= 4 && restreamed <= (chunks == 4 ? 48 : 96) * (int64_t)1000000) return F_GEMV_PACKED;
    }
    if (gemm_wn_eligible(p)) return F_GEMM_WN;
    if (gemm_8bit_eligible(p)) return F_GEMM_8BIT;  // also streams K-major 8-bit operands at small M (split-K)
    if (gemm_kbytes_eligible(p)) return F_GEMM_KBYTES;
    // unquantised layers: the generic family's vector kernels serve decode; from 9 rows (5 on layers above 32 M weights),
    // or when asked, the MFMA GEMM (4096^2 bf16 at 8 / 16 / 64 / 4096 rows: 17.1 / 16.7 / 19.9 / 130 us against 16.2 / 25.3 /
    // 70 / 3505; 14336 x 4096 at 4 / 8 rows: 33.7 / 28.8 against 30.4 / 47.2)
    if ((p.M > 8 || (p.M > 4 && (int64_t)p.N * p.K > ((int64_t)1 << 25)) || want_matrix) && !want_stream && gemm_16bit_eligible(p))
        return F_GEMM_16BIT;
    // 2-bit codes in groups of 32 and 1-bit codes in groups of 32 / 64 have no streaming kernel and no tiled GEMM: the
    // mid-batch kernel at every row count (2-bit gs 32, 8192^2 at 1 / 64 / 256 rows: 19.5 / 30 / 63 us against 37 / 408 /
    // 1592 of the generic kernels; 1-bit gs 64, 16384^2 at 64 rows: 72 us against 2.0 ms), except a single row of 1-bit
    // codes on small and medium layers, where the generic K-split kernel is ahead (14336 x 4096: 15.2 against 19.3)
    const bool one_row_1bit = p.W_nbits == 1 && p.M == 1 && (int64_t)p.N * p.K < ((int64_t)1 << 26);
    if (p.tile_config <= 0 && !want_stream && !one_row_1bit && wn_mid_eligible(p)) return F_WN_MID;
    if (want_matrix) {  // no matrix-core kernel takes the call: the streaming ones after all
        if (gemv_packed_eligible(p)) return F_GEMV_PACKED;
        if (gemv_kmajor_eligible(p)) return F_GEMV_KMAJOR;
    }
    return F_GENERIC;
}

int resolve_type(const gla_matmul_args& p) {
    return p.matmul_type == GLA_MATMUL_AUTO ? matmul_type_for(p.M, p.W_nbits, is_mx(p.input_dtype)) : p.matmul_type;
}

int64_t family_workspace(Family f, const gla_matmul_args& a) {
    switch (f) {
        case F_GEMV_PACKED: return gemv_packed_workspace_bytes(a);
        case F_GEMM_WN: return gemm_wn_workspace_bytes(a);
        case F_WN_MID: return wn_mid_workspace_bytes(a);
        case F_GEMM_16BIT: return gemm_16bit_workspace_bytes(a);
        case F_GEMM_8BIT: case F_GEMM_MXFP4: return gemm_8bit_workspace_bytes(a);
        case F_GEMM_KBYTES: return gemm_kbytes_workspace_bytes(a);
        case F_GEMM_MXFP8: return gemm_mxfp8_workspace_bytes(a);
        case F_GEMM_BLOCKQ: return gemm_blockq_workspace_bytes(a);
        case F_GEMM_KBYTES_MX: return gemm_kbytes_mx_workspace_bytes(a);
        case F_K_SKINNY: return kring_workspace_bytes(a);
        default: return 0;
    }
}

// fp8 / int8 activations on 32-bit packed codes (the reference's A8Wn_HQQ_INT_dynamic and A8W158_INT_dynamic
// processors): no kernel of their own.  Both types convert to fp16 exactly, so the activations are widened into
// the workspace by a small launch and the 16-bit kernels run on them, per-token scales in their epilogue.  An int32
// accumulator asked for stays exact: the tiled GEMM's fp32 sums of integer products are exact below 2^24, and the
// streaming kernel folds its offset sums every 64 K-values for such a call (gemv_packed.hip::geometry).
struct Widened {
    gla_matmul_args q;   // the call the 16-bit kernel sees (x and workspace filled in at launch)
    Family f;
    int64_t x_off;       // where the fp16 activations go in the workspace
    int64_t x_stride;    // their row stride in elements
    int64_t total;       // workspace bytes of the whole call
};

bool widen(const gla_matmul_args& p, Widened& w) {
    if (!(p.input_dtype == GLA_DT_FP8 || p.input_dtype == GLA_DT_INT8) || p.w_dtype != GLA_DT_INT32) return false;
    if (p.x_stride_k != 1 || !(p.acc_dtype == GLA_DT_FP32 || p.acc_dtype == GLA_DT_INT32)) return false;
    if (!(p.output_dtype == GLA_DT_FP16 || p.output_dtype == GLA_DT_BF16 || p.output_dtype == GLA_DT_FP32)) return false;
    w.q = p;
    w.q.input_dtype = GLA_DT_FP16;
    w.x_stride = (p.K + 7) / 8 * 8;
    w.q.x_stride_m = w.x_stride;
    w.q.x = (const void*)(uintptr_t)256;  // stands for an aligned pointer while the kernels' rules are asked
    w.q.workspace = nullptr;
    w.q.workspace_bytes = 0;
    w.f = choose(w.q, resolve_type(w.q));
    if (!(w.f == F_GEMV_PACKED || w.f == F_GEMM_WN || w.f == F_WN_MID)) return false;
    // An int32 accumulator was asked for: the 16-bit kernels sum in fp32, which is the same number as long as every
    // partial sum of |x| (<= 128) times |q - z| (below 2^W_nbits for a zero point inside the code range) over K stays
    // below 2^24.  Longer sums go to the generic kernel, which adds integers.
    if (p.acc_dtype == GLA_DT_INT32 && (int64_t)p.K * 128 * ((1 << p.W_nbits) - 1) >= ((int64_t)1 << 24)) return false;
    const int64_t inner = family_workspace(w.f, w.q);
    if (inner < 0) return false;
    // the first kWsPrivateBytes hold the streaming kernels' ticket counters and slots, whoever runs
    w.x_off = ((inner > kWsPrivateBytes ? inner : kWsPrivateBytes) + 255) / 256 * 256;
    w.total = w.x_off + (int64_t)p.M * w.x_stride * 2;
    return true;
}

// Packed layers at prefill size: from 2048 rows of bf16 (4096 of fp16) the weights are first written out as 16-bit
// values into the workspace (wn_unpack16.hip: once per call, at memory speed, 11.6 us for 4096^2) and the 16-bit GEMM
// runs on them, at the rate of an unquantised layer, instead of the fused kernel that unpacks every weight once per
// 128 or 256 rows beside its MFMAs.  Per-channel and per-token scales stay in the GEMM's epilogue.
struct Unpacked {
    gla_matmul_args q;   // the call the 16-bit GEMM sees (w and workspace filled in at launch)
    int64_t w_off;       // where the 16-bit weights go in the workspace
    int64_t total;       // workspace bytes of the whole call
};

bool unpack_first(const gla_matmul_args& p, Family f, Unpacked& u) {
    // (unpacked weight bytes under 16-bit activations likewise: the bytes are converted once, the per-channel scale stays
    // in the epilogue; int8 bytes x bf16, M = 4096, N = K = 8192: see below)
    const bool bytes = p.w_dtype == GLA_DT_INT8 || p.w_dtype == GLA_DT_UINT8 || p.w_dtype == GLA_DT_FP8;
    if (bytes) {
        const bool asked_b = p.tile_config == GLA_TILE_PREFER_UNPACKED && p.M > 16 && gemm_kbytes_eligible(p);
        const bool by_rule_b = f == F_GEMM_KBYTES && p.M >= 2048 && p.tile_config <= 0 && p.tile_config != GLA_TILE_PREFER_MATRIX;
        if (!asked_b && !by_rule_b) return false;
        if (p.K % 16 != 0 || (p.W_group_mode == GLA_WGM_SCALE && (p.channel_scale_mode & 1))) return false;
        if ((p.W_group_mode == GLA_WGM_SCALE || (p.channel_scale_mode & 1)) && p.meta_stride_n != 1) return false;
        if ((int64_t)p.N * p.K >= ((int64_t)1 << 30)) return false;
        u.q = p;
        u.q.W_nbits = 16;
        u.q.unpack_mask = 0xffff;
        u.q.w_dtype = p.input_dtype;
        if (p.W_group_mode == GLA_WGM_SCALE) u.q.channel_scale_mode = p.channel_scale_mode | 1;  // one scale per channel, after the K sum as before
        u.q.W_group_mode = GLA_WGM_NONE;
        u.q.group_size = p.K;
        u.q.zeros = nullptr;
        u.q.zero_is_scalar = 0;
        u.q.w = (const void*)(uintptr_t)256;
        u.q.w_stride_k = 1;
        u.q.w_stride_n = p.K;
        u.q.tile_config = -1;
        u.q.workspace = nullptr;
        u.q.workspace_bytes = 0;
        if (!gemm_16bit_eligible(u.q)) return false;
        const int64_t inner_b = gemm_16bit_workspace_bytes(u.q);
        if (inner_b < 0) return false;
        u.w_off = ((inner_b > kWsPrivateBytes ? inner_b : kWsPrivateBytes) + 255) / 256 * 256;
        u.total = u.w_off + (int64_t)p.N * p.K * 2;
        return true;
    }
    // Layers without a tiled GEMM (groups of 16 / 32, 1-bit codes) run the mid-batch kernel as chunks of 64 rows, each
    // of which streams and unpacks the weights again: they unpack first from 512 rows (1- and 2-bit codes: 1024).
    const bool tiled = gemm_wn_eligible(p);
    const bool asked = p.tile_config == GLA_TILE_PREFER_UNPACKED && p.M > 16 && (tiled || wn_mid_eligible(p));
    // same launches side by side, fused -> unpacked (us): 4-bit gs 128 bf16 4096^2 at 1024 / 2048 / 4096 / 8192 rows 72 ->
    // 74, 107 -> 92, 161 -> 135, 297 -> 246; 8192^2 189 -> 179, 292 -> 261, 573 -> 474, 1179 -> 914; fp16, whose fused
    // unpacking is cheaper: 66 -> 73, 94 -> 96, 146 -> 143, 280 -> 267; 8192^2 158 -> 186, 271 -> 278, 527 -> 505, 1052 -> 968
    const int from_rows = p.input_dtype == GLA_DT_BF16 ? 2048 : 4096;
    // (bf16, mid-batch chunks -> unpacked, us: 8192^2 4-bit gs 32 at 512 / 1024 / 4096 rows 157 -> 133, 254 -> 190, 892 -> 483;
    // 2-bit gs 32 125 -> 131, 197 -> 189, 698 -> 481; 1-bit gs 64 138 -> 124, 216 -> 181, 745 -> 470; 4096^2 4-bit gs 32 51 -> 48,
    // 85 -> 66, 256 -> 132; 2-bit 42 -> 47, 68 -> 66, 209 -> 132)
    const int kMidUnpackRows = p.W_nbits >= 4 ? 512 : 1024;
    const bool free_choice = p.tile_config <= 0 && p.tile_config != GLA_TILE_PREFER_MATRIX && p.tile_config != GLA_TILE_PREFER_MID;
    const bool by_rule = free_choice && ((f == F_GEMM_WN && p.M >= from_rows) || (f == F_WN_MID && !tiled && p.M >= kMidUnpackRows));
    if (!asked && !by_rule) return false;
    if (p.acc_dtype != GLA_DT_FP32 || (p.W_group_mode >= GLA_WGM_SCALE && (p.channel_scale_mode & 1))) return false;
    if ((int64_t)p.N * p.K >= ((int64_t)1 << 30)) return false;
    u.q = p;
    u.q.W_nbits = 16;
    u.q.elements_per_sample = 1;
    u.q.unpack_mask = 0xffff;
    u.q.w_dtype = p.input_dtype;
    u.q.W_group_mode = GLA_WGM_NONE;
    u.q.group_size = p.K;
    u.q.zeros = nullptr;
    u.q.zero_is_scalar = 0;
    if (!(p.channel_scale_mode & 1)) u.q.scales = nullptr;
    u.q.w = (const void*)(uintptr_t)256;  // stands for an aligned pointer while the kernel's rules are asked
    u.q.w_stride_k = 1;
    u.q.w_stride_n = p.K;
    u.q.tile_config = -1;
    u.q.workspace = nullptr;
    u.q.workspace_bytes = 0;
    if (!gemm_16bit_eligible(u.q)) return false;
    const int64_t inner = gemm_16bit_workspace_bytes(u.q);
    if (inner < 0) return false;
    u.w_off = ((inner > kWsPrivateBytes ? inner : kWsPrivateBytes) + 255) / 256 * 256;
    u.total = u.w_off + (int64_t)p.N * p.K * 2;
    return true;
}

}  // namespace
}  // namespace gla

using namespace gla;

extern "C" {

int gla_abi_version(void) { return GLA_ABI_VERSION; }

const char* gla_last_error(void) { return g_error; }

int gla_get_matmul_type(int M, int W_nbits, int is_mx_) { return matmul_type_for(M, W_nbits, is_mx_); }

int gla_get_closest_m(int M) { return closest_m(M); }

int gla_select_config(const gla_matmul_args* args) {
    const int rc = validate(args);
    if (rc != GLA_OK) return rc;
    const Family f = choose(*args, resolve_type(*args));
    if (f == F_GEMV_PACKED) return gemv_packed_default_config(*args);
    Widened w;
    if (f == F_GENERIC && widen(*args, w) && w.f == F_GEMV_PACKED) return gemv_packed_default_config(w.q);
    return 0;
}

int gla_probe_mfma(int dtype, int random_operands, int iters, void* sink, double* flops, void* stream) {
    return gla::launch_probe_mfma(dtype, random_operands, iters, sink, flops, (hipStream_t)stream);
}

int gla_probe_read(const void* buf, int64_t bytes, void* sink, void* stream) {
    return gla::launch_probe_read(buf, bytes, sink, (hipStream_t)stream);
}

int gla_probe_read_cfg(const void* buf, int64_t bytes, void* sink, int workgroups, int threads, int loads, void* stream) {
    return gla::launch_probe_read_cfg(buf, bytes, sink, workgroups, threads, loads, (hipStream_t)stream);
}

int gla_prefetch(const void* buf, int64_t bytes, int workgroups, void* stream) {
    return gla::launch_prefetch(buf, bytes, workgroups, (hipStream_t)stream);
}

int gla_matmul_family(const gla_matmul_args* args) {
    const int rc = validate(args);
    if (rc != GLA_OK) return rc;
    const Family f = choose(*args, resolve_type(*args));
    Widened w;
    if (f == F_GENERIC && widen(*args, w)) return (int)w.f;  // the kernel that runs on the widened activations
    Unpacked u;
    if (unpack_first(*args, f, u)) return (int)F_GEMM_16BIT;   // ... on the unpacked weights
    return (int)f;
}

int64_t gla_matmul_workspace_bytes(const gla_matmul_args* args) {
    const int rc = validate(args);
    if (rc != GLA_OK) return rc;
    if (args->M == 0) return 0;
    const Family f = choose(*args, resolve_type(*args));
    Widened w;
    if (f == F_GENERIC && widen(*args, w)) return w.total;
    Unpacked u;
    if (unpack_first(*args, f, u)) return u.total;
    return family_workspace(f, *args);
}

int gla_matmul(const gla_matmul_args* args, void* stream) {
    const int rc = validate(args);
    if (rc != GLA_OK) return rc;
    if (args->M == 0) return GLA_OK;
    hipStream_t s = (hipStream_t)stream;
    Family f = choose(*args, resolve_type(*args));
    Widened w;
    if (f == F_GENERIC && widen(*args, w)) {
        if (args->workspace == nullptr || (int64_t)args->workspace_bytes < w.total) {
            set_error("matmul: workspace of %lld bytes required (8-bit activations are widened into it), %llu given",
                      (long long)w.total, (unsigned long long)args->workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        void* x16 = (char*)args->workspace + w.x_off;
        const int rcw = launch_widen_x8(args->x, args->x_stride_m, args->M, args->K, args->input_dtype, x16, w.x_stride, s);
        if (rcw != GLA_OK) return rcw;
        w.q.x = x16;
        w.q.workspace = args->workspace;
        w.q.workspace_bytes = (uint64_t)w.x_off;
        return w.f == F_GEMV_PACKED ? launch_gemv_packed(w.q, s) : (w.f == F_WN_MID ? launch_wn_mid(w.q, s) : launch_gemm_wn(w.q, s));
    }
    Unpacked u;
    if (unpack_first(*args, f, u)) {
        if (args->workspace == nullptr || (int64_t)args->workspace_bytes < u.total) {
            set_error("matmul: workspace of %lld bytes required (the weights are unpacked into it), %llu given", (long long)u.total,
                      (unsigned long long)args->workspace_bytes);
            return GLA_ERR_WORKSPACE_TOO_SMALL;
        }
        void* w16 = (char*)args->workspace + u.w_off;
        const bool bytes = args->w_dtype == GLA_DT_INT8 || args->w_dtype == GLA_DT_UINT8 || args->w_dtype == GLA_DT_FP8;
        const int rcu = bytes ? launch_kbytes_unpack16(*args, w16, args->K, s) : launch_wn_unpack16(*args, w16, args->K, s);
        if (rcu != GLA_OK) return rcu;
        u.q.w = w16;
        u.q.workspace = args->workspace;
        u.q.workspace_bytes = (uint64_t)u.w_off;
        return launch_gemm_16bit(u.q, s);
    }
    int rc2;
    switch (f) {
        // Every family adds the bias in its epilogue or split-K finishing kernel (the `return`s) except the generic
        // kernel, which is followed by the elementwise launch below.
        case F_GEMV_PACKED: return launch_gemv_packed(*args, s);
        case F_GEMV_KMAJOR: return launch_gemv_kmajor(*args, s);
        case F_GEMM_WN: return launch_gemm_wn(*args, s);
        case F_GEMM_8BIT: return launch_gemm_8bit(*args, s);
        case F_GEMM_MXFP4: return launch_gemm_mxfp4(*args, s);
        case F_GEMM_KBYTES: return args->bias != nullptr ? launch_gemm_kbytes_bias(*args, s) : launch_gemm_kbytes(*args, s);
        case F_GEMM_MXFP8: return launch_gemm_mxfp8(*args, s);
        case F_MX_STREAM: return launch_mx_stream(*args, s);
        case F_BLOCKQ_STREAM: return launch_blockq_stream(*args, s);
        case F_GEMM_BLOCKQ: return launch_gemm_blockq(*args, s);
        case F_GEMM_KBYTES_MX: return args->bias != nullptr ? launch_gemm_kbytes_mx_bias(*args, s) : launch_gemm_kbytes_mx(*args, s);
        case F_MX_SKINNY: return launch_mx_skinny(*args, s);
        case F_K_SKINNY: return launch_kring(*args, s);
        case F_WN_MID: return launch_wn_mid(*args, s);
        case F_GEMM_16BIT: return launch_gemm_16bit(*args, s);
        default: rc2 = launch_generic(*args, s); break;
    }
    if (rc2 == GLA_OK && args->bias != nullptr) rc2 = launch_bias_add(*args, s);
    return rc2;
}

// ---- gla_matmul without a caller's workspace --------------------------------------------------
// The scratch that gla_matmul takes as `workspace` (split-K partials, ticket counters, regrouped
// block scales) lives here in a device array that the code object brings along: nothing is
// allocated, at set-up or per call.  Each GPU has its own copy at its own address; the array's
// name is only a host-side handle for hipGetSymbolAddress, and everything below uses the address
// that call returned for the current device.
}  // extern "C"

namespace {

static __device__ __align__(256) unsigned char scratch[GLA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of this device's copy of `scratch`, looked up on the first call on a device.  Nothing is cleared: a
// device array without an initialiser is zero-filled when the code object is loaded, and every kernel that keeps
// counters or slots there leaves them at zero again, so the first call may as well be recorded into a graph.
int static_scratch(void** out) {
    int dev = 0;
    int rc = check_hip(hipGetDevice(&dev), "hipGetDevice");
    if (rc != GLA_OK) return rc;
    if (dev < 0 || dev >= kMaxDevices) {
        set_error("gla_matmul_static: device index %d is outside the %d devices this entry point keeps scratch for", dev,
                  kMaxDevices);
        return GLA_ERR_NO_DEVICE;
    }
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        static std::mutex mu;
        std::lock_guard<std::mutex> lock(mu);
        ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
        if (ptr == nullptr) {
            rc = check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
            if (rc != GLA_OK) return rc;
            if (ptr == nullptr) {
                set_error("gla_matmul_static: the device array has no address on device %d", dev);
                return GLA_ERR_LAUNCH_FAILED;
            }
            g_scratch_ptr[dev].store(ptr, std::memory_order_release);
        }
    }
    *out = ptr;
    return GLA_OK;
}

}  // namespace

extern "C" {

int64_t gla_static_scratch_bytes(void) { return (int64_t)GLA_STATIC_SCRATCH_BYTES; }

int gla_matmul_static(const gla_matmul_args* args, void* stream) {
    int64_t need = gla_matmul_workspace_bytes(args);
    if (need < 0) return (int)need;
    gla_matmul_args a = *args;
    if (need > (int64_t)GLA_STATIC_SCRATCH_BYTES && args->tile_config <= 0 && args->tile_config != GLA_TILE_PREFER_MATRIX) {
        // a packed layer at prefill size whose unpacked weights do not fit the array stays on the fused kernel
        a.tile_config = GLA_TILE_PREFER_MATRIX;
        const int64_t fused = gla_matmul_workspace_bytes(&a);
        if (fused >= 0 && fused <= (int64_t)GLA_STATIC_SCRATCH_BYTES)
            need = fused;
        else
            a.tile_config = args->tile_config;
    }
    if (need > (int64_t)GLA_STATIC_SCRATCH_BYTES) {
        set_error("gla_matmul_static: this problem (M=%d N=%d K=%d) needs %lld bytes of scratch; the built-in array holds "
                  "%lld. Use gla_matmul with a workspace of that size", args->M, args->N, args->K, (long long)need,
                  (long long)GLA_STATIC_SCRATCH_BYTES);
        return GLA_ERR_WORKSPACE_TOO_SMALL;
    }
    a.workspace = nullptr;
    a.workspace_bytes = 0;
    if (need > 0) {
        void* ptr = nullptr;
        const int rc = static_scratch(&ptr);
        if (rc != GLA_OK) return rc;
        a.workspace = ptr;
        a.workspace_bytes = (uint64_t)GLA_STATIC_SCRATCH_BYTES;
    }
    return gla_matmul(&a, stream);
}

int gla_scale_activations_per_token(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y,
                                    int y_dtype, float* scales, void* stream) {
    return launch_act_per_token(x, x_dtype, x_stride_m, M, K, y, y_dtype, scales, (hipStream_t)stream);
}

int gla_scale_activations_per_block(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y,
                                    int y_dtype, float* scales, void* stream) {
    return launch_act_per_block(x, x_dtype, x_stride_m, M, K, y, y_dtype, scales, (hipStream_t)stream);
}

int gla_scale_activations_mxfp4(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y,
                                uint8_t* scales, void* stream) {
    return launch_act_mxfp4(x, x_dtype, x_stride_m, M, K, y, scales, (hipStream_t)stream);
}

int gla_scale_activations_mxfp8(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y,
                                uint8_t* scales, void* stream) {
    return launch_act_mxfp8(x, x_dtype, x_stride_m, M, K, y, scales, (hipStream_t)stream);
}

int gla_pack_over_cols(const uint8_t* codes, void* out, int64_t rows, int64_t cols, int W_nbits,
                       int packing_bitwidth, void* stream) {
    return launch_pack_over_cols(codes, out, rows, cols, W_nbits, packing_bitwidth, (hipStream_t)stream);
}

int gla_unpack_over_cols(const void* packed, uint8_t* out, int64_t rows, int64_t packed_cols, int W_nbits,
                         int packing_bitwidth, void* stream) {
    return launch_unpack_over_cols(packed, out, rows, packed_cols, W_nbits, packing_bitwidth, (hipStream_t)stream);
}

}  // extern "C"
