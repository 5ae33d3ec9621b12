// Host-side declarations shared by the C ABI and the kernel-family launchers.
#pragma once

#include "common.hpp"

namespace gla {

// ---- layout-agnostic path (generic.hip) -----------------------------------
int launch_generic(const gla_matmul_args& p, hipStream_t stream);
// out += bias on the finished output, for the families that do not add the bias in their epilogue
int launch_bias_add(const gla_matmul_args& p, hipStream_t stream);
// Tile height and K split of a tiled MFMA GEMM from a small cost model (host only).  A workgroup's time is its
// pipeline stages times a per-stage cost that grows with the tile height (taller tiles do more per stage and are
// the more efficient ones, but only when there are enough of them); workgroups run in rounds of one per CU; a split
// K pays a finishing launch and the fp32 partials' round trip through memory.  The constants come from timing every
// (tile, split) pair on 4096^2, 14336 x 4096 and 4096 x 14336 layers at 64..2048 rows; before, the tallest tile was
// taken above 128 rows whatever the layer, which left small layers with a quarter of the chip busy or with deep
// splits (fp8 4096^2 at 1024 rows: 63 us, 31 with 64-row tiles and no split).
struct TilePick {
    int bm, S;
};
struct TileModel {
    double underfill = 0.8;       // per-stage cost of a workgroup on an almost empty chip, relative to the full one
    double split_fixed_us = 2.0;  // finishing launch
    double split_us_per_elem = 2.0e-6;  // 8 bytes per partial, written and read
    int pair_up_to = 0;           // tiles this tall or shorter run two workgroups per CU ...
    double pair_cost = 1.65;      // ... each at this multiple of its stage cost
};
inline TilePick pick_tile_and_split(int M, int N, int bn, int steps, int min_steps_per_split, int max_splits, const int* bms,
                                    const float* stage_cost_us, int n_bms, int bm_fixed, int s_fixed,
                                    const TileModel& model = TileModel()) {
    TilePick best{bms[0], 1};
    double best_t = 1e30;
    const int tiles_n = (N + bn - 1) / bn;
    for (int i = 0; i < n_bms; ++i) {
        const int bm = bms[i];
        if (bm_fixed > 0 ? bm != bm_fixed : (i > 0 && bm >= 2 * M)) continue;  // no tile more than twice as tall as the batch
        const int tiles = ((M + bm - 1) / bm) * tiles_n;
        const int top = s_fixed > max_splits ? s_fixed : max_splits;  // a split asked for is taken as asked
        for (int want = 1; want <= top; ++want) {
            if (s_fixed > 0 ? want != s_fixed : (want > 1 && steps / want < min_steps_per_split)) continue;
            const int sps = (steps + want - 1) / want, S = (steps + sps - 1) / sps;
            if (s_fixed <= 0 && S != want) continue;  // the same split under another name
            if (s_fixed > 0 && bm_fixed > 0) return TilePick{bm, S};
            const double wgs = (double)tiles * S;
            const bool paired = bm <= model.pair_up_to && wgs > 256.0;
            const double per_round = paired ? 512.0 : 256.0;
            const double rounds = (double)((int64_t)((wgs + per_round - 1) / per_round));
            const double fill = wgs < 256.0 ? wgs / 256.0 : 1.0;
            double t = rounds * sps * stage_cost_us[i] * (model.underfill + (1.0 - model.underfill) * fill) * (paired ? model.pair_cost : 1.0);
            if (S > 1) t += model.split_fixed_us + model.split_us_per_elem * (double)M * N * S;
            if (t < best_t) {
                best_t = t;
                best = TilePick{bm, S};
            }
        }
    }
    return best;
}

// fp8-e4m3 / int8 activations [M, K] (row stride in bytes) -> fp16 rows of out_stride_m elements; both convert exactly
int launch_widen_x8(const void* x, int64_t x_stride_m, int M, int K, int input_dtype, void* out_f16, int64_t out_stride_m, hipStream_t stream);

// ---- streaming GEMV on 32-bit packed words, N fastest (gemv_packed.hip) ----
// tile_config (when >= 1000) = waves per workgroup * 1000 + load batches per wave.
bool gemv_packed_eligible(const gla_matmul_args& p);
int64_t gemv_packed_workspace_bytes(const gla_matmul_args& p);
int gemv_packed_default_config(const gla_matmul_args& p);
int launch_gemv_packed(const gla_matmul_args& p, hipStream_t stream);

// ---- GEMV on K-contiguous 8/16-bit weights (gemv_kmajor.hip) ---------------
bool gemv_kmajor_eligible(const gla_matmul_args& p);
int launch_gemv_kmajor(const gla_matmul_args& p, hipStream_t stream);

// ---- MFMA GEMM with in-register dequant of packed words (gemm_wn.hip) ------
bool gemm_wn_eligible(const gla_matmul_args& p);
int64_t gemm_wn_workspace_bytes(const gla_matmul_args& p);
int launch_gemm_wn(const gla_matmul_args& p, hipStream_t stream);
// the weights of such a call as fp16 / bf16 values, [N, ldo] with K contiguous (wn_unpack16.hip)
int launch_wn_unpack16(const gla_matmul_args& p, void* out, int64_t ldo, hipStream_t stream);
// ... and the same for unpacked int8 / uint8 / fp8 weight bytes (a call of gemm_kbytes)
int launch_kbytes_unpack16(const gla_matmul_args& p, void* out, int64_t ldo, hipStream_t stream);

// ---- MFMA GEMM on 8-bit operands, both K-contiguous (gemm_8bit.hip) --------
bool gemm_8bit_eligible(const gla_matmul_args& p);
int launch_gemm_8bit(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_8bit_workspace_bytes(const gla_matmul_args& p);  // also for the MXFP4 entry

// ---- block-scaled MXFP4 MFMA GEMM (gemm_8bit.hip) -------------------------
bool gemm_mxfp4_eligible(const gla_matmul_args& p);
int launch_gemm_mxfp4(const gla_matmul_args& p, hipStream_t stream);

// ---- MXFP8 weights x fp8 activations (per-token or block-scaled), MFMA GEMM (gemm_8bit.hip)
bool gemm_mxfp8_eligible(const gla_matmul_args& p);
int launch_gemm_mxfp8(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_mxfp8_workspace_bytes(const gla_matmul_args& p);

// ---- streaming kernel for K-contiguous micro-scaled operands (mx_stream.hip): weight-only MX
// layers (fp16/bf16 x MXFP8/MXFP4 weights), MXFP8 activations x MXFP4 weights
bool mx_stream_eligible(const gla_matmul_args& p);
bool mx_stream_quantises(const gla_matmul_args& p);  // the call asks for MXFP4 activations made inside the kernel, and it makes them
int launch_mx_stream(const gla_matmul_args& p, hipStream_t stream);

// ---- 128 x 128 block-quantised int8 / fp8 above 4 rows: MFMA GEMM (gemm_8bit.hip)
bool gemm_blockq_eligible(const gla_matmul_args& p);
int launch_gemm_blockq(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_blockq_workspace_bytes(const gla_matmul_args& p);

// ---- streaming kernel for 128 x 128 block-quantised int8 / fp8 (blockq_stream.hip)
bool blockq_stream_eligible(const gla_matmul_args& p);
int launch_blockq_stream(const gla_matmul_args& p, hipStream_t stream);

// ---- activation quantisation (actquant.hip) and bit packing (bitpack.hip) --
int launch_act_per_token(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y, int y_dtype,
                         float* scales, hipStream_t stream);
int launch_act_per_block(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, void* y, int y_dtype,
                         float* scales, hipStream_t stream);
int launch_act_mxfp4(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                     hipStream_t stream);
int launch_act_mxfp8(const void* x, int x_dtype, int64_t x_stride_m, int M, int K, uint8_t* y, uint8_t* scales,
                     hipStream_t stream);
int launch_pack_over_cols(const uint8_t* codes, void* out, int64_t rows, int64_t cols, int nbits, int width,
                          hipStream_t stream);
int launch_unpack_over_cols(const void* packed, uint8_t* out, int64_t rows, int64_t pcols, int nbits, int width,
                            hipStream_t stream);

// ---- MFMA GEMM for 16-bit activations x K-contiguous weight bytes (gemm_kbytes.hip)
bool gemm_kbytes_eligible(const gla_matmul_args& p);
int launch_gemm_kbytes(const gla_matmul_args& p, hipStream_t stream);
int launch_gemm_kbytes_bias(const gla_matmul_args& p, hipStream_t stream);      // the same with p.bias added in the epilogue
int launch_gemm_kbytes_mx_bias(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_kbytes_workspace_bytes(const gla_matmul_args& p);

// ---- weight-only MX layers above 2 rows: the same MFMA GEMM with micro-scaled weights (gemm_kbytes.hip)
// ---- weight-only MX layers at 3..16 rows: weights straight into registers, matrix cores (mx_skinny.hip)
bool mx_skinny_eligible(const gla_matmul_args& p);
int launch_mx_skinny(const gla_matmul_args& p, hipStream_t stream);
// ---- unquantised layers above 16 rows: fp16 x fp16 / bf16 x bf16 MFMA GEMM, weights [N, K] K-contiguous (gemm_16bit.hip)
bool gemm_16bit_eligible(const gla_matmul_args& p);
int64_t gemm_16bit_workspace_bytes(const gla_matmul_args& p);
int launch_gemm_16bit(const gla_matmul_args& p, hipStream_t stream);

// ---- fp16 / bf16 x packed codes at 17..64 rows: weights from registers into the MFMA, activations shared through LDS (wn_mid.hip)
bool wn_mid_eligible(const gla_matmul_args& p);
int64_t wn_mid_workspace_bytes(const gla_matmul_args& p);
int launch_wn_mid(const gla_matmul_args& p, hipStream_t stream);

// ---- MXFP4 x MXFP4, fp8 x fp8, int8 x int8 at 3..32 rows: operands copied to per-wave LDS rings by lines, MFMA (kring.hip)
bool kring_eligible(const gla_matmul_args& p);
int64_t kring_workspace_bytes(const gla_matmul_args& p);  // 16-bit activations on MX weights: their e4m3 terms
int launch_kring(const gla_matmul_args& p, hipStream_t stream);
bool gemm_kbytes_mx_eligible(const gla_matmul_args& p);
int launch_gemm_kbytes_mx(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_kbytes_mx_workspace_bytes(const gla_matmul_args& p);

// ---- diagnostic: sustained matrix rate (probe.hip) ---------------------------
int launch_probe_mfma(int dtype, int random_operands, int iters, void* sink, double* flops, hipStream_t stream);
// ---- diagnostic: streaming-read ceiling (probe.hip) --------------------------
int launch_probe_read(const void* buf, int64_t bytes, void* sink, hipStream_t stream);
int launch_probe_read_cfg(const void* buf, int64_t bytes, void* sink, int workgroups, int threads, int loads, hipStream_t stream);
int launch_prefetch(const void* buf, int64_t bytes, int workgroups, hipStream_t stream);

}  // namespace gla
