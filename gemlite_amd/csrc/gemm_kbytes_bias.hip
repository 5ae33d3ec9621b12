// The byte-weight and weight-only-MX MFMA GEMMs of gemm_kbytes.hip with the bias added in the epilogue (or in the
// split-K finishing kernel): the same source compiled a second time, as a translation unit of its own so that the two
// sets of kernels build in parallel.  Entry points: launch_gemm_kbytes_bias, launch_gemm_kbytes_mx_bias.
// (reference: `out += bias`, gemlite/core.py:271-272.)
#define GLA_KB_BIAS 1
#include "gemm_kbytes.hip"
