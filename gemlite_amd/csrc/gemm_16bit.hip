// The MFMA GEMM of gemm_8bit.hip for 16-bit float operands (unquantised layers: fp16 x fp16, bf16 x bf16, weights
// [N, K] with K contiguous): the same source compiled a second time with only these two modes instantiated, as a
// translation unit of its own so that the two sets of kernels build in parallel.  Entry points: gemm_16bit_eligible,
// gemm_16bit_workspace_bytes, launch_gemm_16bit.
#define GLA_G8_16BIT 1
#include "gemm_8bit.hip"
