// Host-side declarations shared by the C ABI and the kernel-family launchers.
#pragma once

#include "common.hpp"

namespace gla {

// ---- layout-agnostic path (generic.hip) -----------------------------------
int launch_generic(const gla_matmul_args& p, hipStream_t stream);
// out += bias on the finished output, for the families that do not add the bias in their epilogue
int launch_bias_add(const gla_matmul_args& p, hipStream_t stream);
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
int64_t gemm_kbytes_workspace_bytes(const gla_matmul_args& p);

// ---- weight-only MX layers above 2 rows: the same MFMA GEMM with micro-scaled weights (gemm_kbytes.hip)
// ---- weight-only MX layers at 3..16 rows: weights straight into registers, matrix cores (mx_skinny.hip)
bool mx_skinny_eligible(const gla_matmul_args& p);
int launch_mx_skinny(const gla_matmul_args& p, hipStream_t stream);
bool gemm_kbytes_mx_eligible(const gla_matmul_args& p);
int launch_gemm_kbytes_mx(const gla_matmul_args& p, hipStream_t stream);
int64_t gemm_kbytes_mx_workspace_bytes(const gla_matmul_args& p);

// ---- diagnostic: sustained matrix rate (probe.hip) ---------------------------
int launch_probe_mfma(int dtype, int random_operands, int iters, void* sink, double* flops, hipStream_t stream);
// ---- diagnostic: streaming-read ceiling (probe.hip) --------------------------
int launch_probe_read(const void* buf, int64_t bytes, void* sink, hipStream_t stream);

}  // namespace gla
