/*
 * gemlite_amd.h - C ABI of the MI355X (gfx950) quantized-matmul library.
 *
 * Every entry point takes plain pointers, sizes and integer ids only.  Device
 * pointers are owned by the caller; the library never allocates, frees or
 * retains them, never synchronises the host with the device, and launches on
 * the stream it is given (a hipStream_t passed as void*; NULL = default
 * stream).  All functions return GLA_OK (0) or a negative GLA_ERR_* code and
 * never throw; gla_last_error() returns a thread-local description of the
 * last failure.
 *
 * Element-type ids are the integers of the reference's DType enumeration
 * (reference: gemlite/dtypes.py:8-29).
 */
#ifndef GEMLITE_AMD_H
#define GEMLITE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GLA_ABI_VERSION 1

/* status codes */
#define GLA_OK 0
#define GLA_ERR_INVALID_ARGUMENT (-1) /* NULL pointer, bad size, inconsistent strides */
#define GLA_ERR_UNSUPPORTED_DTYPE (-2)
#define GLA_ERR_UNSUPPORTED_MODE (-3) /* W_group_mode / channel_scale_mode / matmul_type */
#define GLA_ERR_MISALIGNED_SHAPE (-4) /* K not a multiple of group size / word size */
#define GLA_ERR_WORKSPACE_TOO_SMALL (-5)
#define GLA_ERR_LAUNCH_FAILED (-6)    /* HIP runtime reported an error */
#define GLA_ERR_NO_DEVICE (-7)

/* element-type ids (subset used on the hot path) */
#define GLA_DT_FP32 0
#define GLA_DT_FP16 1
#define GLA_DT_BF16 2
#define GLA_DT_FP8 3 /* OCP e4m3fn */
#define GLA_DT_INT8 4
#define GLA_DT_UINT8 5
#define GLA_DT_INT32 6
#define GLA_DT_INT16 9
#define GLA_DT_INT64 11
#define GLA_DT_MXFP16 14 /* fp16 activations x micro-scaled weights (weight-only) */
#define GLA_DT_MXBF16 15 /* bf16 activations x micro-scaled weights (weight-only) */
#define GLA_DT_MXFP8 16
#define GLA_DT_MXFP4 17
#define GLA_DT_E8M0 19

/* matmul kernel families; the ids index the reference's kernel list
 * (reference: gemlite/core.py:57-67). */
#define GLA_MATMUL_AUTO (-1)
#define GLA_MATMUL_GEMV 0
#define GLA_MATMUL_GEMV_REVSPLITK 1
#define GLA_MATMUL_GEMV_SPLITK 2
#define GLA_MATMUL_GEMM_SPLITK 3
#define GLA_MATMUL_GEMM 4

/* weight dequantisation modes (reference: gemlite/triton_kernels/utils.py:73-105) */
#define GLA_WGM_NONE 0          /* w = q                */
#define GLA_WGM_SHIFT 1         /* w = q - zero         */
#define GLA_WGM_SCALE 2         /* w = q * scale        */
#define GLA_WGM_SHIFT_SCALE 3   /* w = (q - zero)*scale */
#define GLA_WGM_FMA 4           /* w = q*scale + zero   */

/* post-accumulation scaling (reference: gemlite/core.py:647-703,
 * gemlite/triton_kernels/gemm_kernels.py:471-485) */
#define GLA_CSM_NONE 0
#define GLA_CSM_WEIGHT 1     /* out *= scales[n]                       */
#define GLA_CSM_ACTIVATION 2 /* out *= scales_x[m]                     */
#define GLA_CSM_BOTH 3       /* out *= scales_x[m] * scales[n]         */
#define GLA_CSM_MX 4         /* per-32 e8m0 micro-scales on both sides */
#define GLA_CSM_BLOCK 5      /* fp32 scales per 128 x 128 weight block and per (row, 128) of x;
                                scales: [K/128, ceil(N/128)], scales_x: [M, K/128] */

/* tile_config values that leave the tile to the library and say which kind of kernel to take where both a streaming
 * (decode) kernel and a matrix-core GEMM could run the call.  The library's own hand-off between the two is a set of
 * thresholds on rows and layer size measured on one machine; the offline tuner times both sides of it for a layer
 * and batch size and stores the winner under the reference's config-cache key (reference: gemlite/core.py:838-906). */
#define GLA_TILE_PREFER_STREAMING (-2)
#define GLA_TILE_PREFER_MATRIX (-3)
/* fp16 / bf16 activations on 2-, 4- or 8-bit packed codes, up to 64 rows: the mid-batch kernel (weights from registers
 * into the MFMA, activations shared through LDS), which the library itself takes for 8-bit codes on large layers only.
 * fp16 / bf16 activations on MXFP8 / MXFP4 weights at 3..16 (fp16: 10) rows: the activations as sums of e4m3 terms
 * through the skinny kernel of the narrow formats (family K_SKINNY; the call then needs a workspace), which the library
 * itself takes on large layers only */
#define GLA_TILE_PREFER_MID (-4)
/* fp16 / bf16 activations on 2-, 4- or 8-bit packed codes, or on unpacked int8 / uint8 / fp8 weight bytes, above 16
 * rows: the weights are first written out as 16-bit values into the workspace (N * K * 2 bytes of it), then the 16-bit
 * matrix-core GEMM runs (family GEMM_16BIT); the library itself does so from 2048 rows (packed codes under fp16: 4096) */
#define GLA_TILE_PREFER_UNPACKED (-5)

/*
 * Arguments of one quantized matmul  out[M,N] = x[M,K] * dequant(w)[K,N].
 *
 * Replaces the argument list of the reference's per-family launchers
 *   gemv_forward            gemlite/triton_kernels/gemv_kernels.py:608-701
 *   gemv_revsplitK_forward  gemlite/triton_kernels/gemv_revsplitK_kernels.py:446-531
 *   gemv_splitK_forward     gemlite/triton_kernels/gemv_splitK_kernels.py:480-542
 *   gemm_splitK_forward     gemlite/triton_kernels/gemm_splitK_kernels.py:772-837
 *   gemm_forward            gemlite/triton_kernels/gemm_kernels.py:741-799
 * All strides are in elements of the tensor they belong to.  `w` is the
 * [K/e, N] view the reference hands to its kernels (e = elements_per_sample):
 * packed integer words are row-major with N fastest (w_stride_k = N,
 * w_stride_n = 1); unpacked 8/16-bit weights are the transposed view of the
 * row-major [N, K] tensor (w_stride_k = 1, w_stride_n = K).
 */
typedef struct gla_matmul_args {
    uint32_t struct_size; /* sizeof(gla_matmul_args), for ABI checking */
    int32_t matmul_type;  /* GLA_MATMUL_*; AUTO applies gla_get_matmul_type */

    const void* x;        /* [M, K] activations (MXFP4: [M, K/2] bytes) */
    const void* w;        /* weights, see above */
    const void* scales;   /* weight scales or NULL */
    const void* zeros;    /* weight zero points or NULL */
    const void* scales_x; /* activation scales or NULL */
    void* out;            /* [M, N] */
    void* workspace;      /* scratch of >= gla_matmul_workspace_bytes() bytes, or NULL if 0 */
    uint64_t workspace_bytes;

    int32_t M, N, K;

    int64_t x_stride_m, x_stride_k;
    int64_t w_stride_k, w_stride_n;
    int64_t out_stride_m, out_stride_n;
    int64_t meta_stride_g, meta_stride_n; /* scales / zeros: [K/group_size, N] */
    int64_t sx_stride_m, sx_stride_g;     /* scales_x: [M, 1] or [M_pad, K/32] */

    /* the reference's meta_args (reference: gemlite/core.py:804-817) */
    int32_t W_nbits;
    int32_t group_size;
    int32_t unpack_mask;
    int32_t elements_per_sample;
    int32_t input_dtype;  /* element type of x as the kernel sees it */
    int32_t output_dtype;
    int32_t acc_dtype;    /* GLA_DT_FP32 or GLA_DT_INT32 */
    int32_t meta_dtype;   /* element type of scales */
    int32_t channel_scale_mode;
    int32_t W_group_mode;
    int32_t data_contiguous;

    int32_t w_dtype;        /* storage type of w (word type for packed data) */
    int32_t zeros_dtype;    /* element type of zeros */
    int32_t zero_is_scalar; /* zeros holds a single element */
    int32_t sx_dtype;       /* element type of scales_x (FP32 or UINT8/E8M0) */
    int32_t tile_config;    /* -1 = library heuristic; an id from gla_select_config or the offline tuner; or one of
                             * GLA_TILE_PREFER_* below */

    /* Optional bias [N] (fp16, bf16 or fp32), or NULL: out = cast(cast(acc ...) + bias[n]), i.e. added to the
     * result already rounded to the output type, as the reference's `out += bias` does
     * (reference: gemlite/core.py:271-272).  Float output types only.  The streaming (decode) kernels
     * and the packed-code GEMM add it in their epilogue; the other kernels are followed by one small launch
     * on the same stream. */
    const void* bias;
    int32_t bias_dtype;

    /* Activation quantisation inside the matmul, for decode sizes (replaces the quantiser launch in front of it;
     * reference: gemlite/core.py:220-250).  0: x holds input_dtype.  GLA_DT_FP16 / GLA_DT_BF16: x holds rows of that
     * 16-bit type ([M, K], x_stride_* in its elements) and the kernel quantises them itself to input_dtype, exactly as
     * gla_scale_activations_per_token (input_dtype FP8 or INT8, channel_scale_mode 2 or 3) or
     * gla_scale_activations_mxfp4 (input_dtype MXFP4, channel_scale_mode 4) would: same codes, same scales, same
     * result as the two launches.  scales_x is not read.  Only the streaming kernels do this (up to 4 rows, fewer on
     * large layers); gla_matmul_family returns GLA_ERR_UNSUPPORTED_MODE for a call they do not take. */
    int32_t x_quant_from;
} gla_matmul_args;

/* Library identification.  No reference counterpart. */
int gla_abi_version(void);
const char* gla_last_error(void);

/* Kernel-family choice from the batch size (reference: gemlite/core.py:163-179). */
int gla_get_matmul_type(int M, int W_nbits, int is_mx);

/* Batch-size bucketing used in config-cache keys
 * (reference: gemlite/triton_kernels/utils.py:185-220). */
int gla_get_closest_m(int M);

/* Shape-based tile choice for a problem; the returned id is meaningful only to
 * gla_matmul (replaces the Triton autotuner's config pruning,
 * reference: gemlite/triton_kernels/gemm_kernels.py:31-145). */
int gla_select_config(const gla_matmul_args* args);

/* Which kernel family gla_matmul would run for a problem: one of GLA_FAMILY_*, or a negative
 * status.  No counterpart in the reference (its registry maps a matmul type to one Triton class,
 * gemlite/core.py:57-67); here several families serve one type, and tests and tuners ask which. */
#define GLA_FAMILY_GENERIC 0      /* layout-agnostic kernels, any mode and stride (packed codes in short groups: K split over waves) */
#define GLA_FAMILY_GEMV_PACKED 1  /* streaming kernels for 32-bit packed codes: up to 16 rows, up to 64 on small layers */
#define GLA_FAMILY_GEMV_KMAJOR 2  /* streaming kernels for K-major weight bytes: 16-bit activations up to 16 rows, fp8 / int8 ones up to 4 */
#define GLA_FAMILY_GEMM_WN 3      /* fused-dequant MFMA GEMM for packed 2/4/8-bit codes */
#define GLA_FAMILY_GEMM_8BIT 4    /* fp8 / int8 MFMA GEMM on K-major operands */
#define GLA_FAMILY_GEMM_MXFP4 5   /* block-scaled FP4 MFMA GEMM */
#define GLA_FAMILY_GEMM_KBYTES 6  /* MFMA GEMM for 16-bit activations x unpacked 8-bit weight bytes */
#define GLA_FAMILY_GEMM_MXFP8 7   /* MXFP8 weights x fp8 activations, MFMA GEMM */
#define GLA_FAMILY_MX_STREAM 8    /* streaming kernel: weight-only MX layers, MXFP8 x MXFP4 */
#define GLA_FAMILY_BLOCKQ_STREAM 9 /* streaming kernel: 128 x 128 block-quantised int8 / fp8 */
#define GLA_FAMILY_GEMM_BLOCKQ 10  /* the same above 2-3 rows: MFMA GEMM with a second, scaled accumulator */
#define GLA_FAMILY_GEMM_KBYTES_MX 11 /* weight-only MX layers above 16 rows: MFMA GEMM, block scale applied on conversion */
#define GLA_FAMILY_MX_SKINNY 12     /* weight-only MX layers at 3..16 rows: weights read once into registers, MFMA */
#define GLA_FAMILY_K_SKINNY 13      /* MXFP4 x MXFP4, fp8 x fp8, int8 x int8 at 3..32 rows: operands as they are into the MFMA, one launch */
#define GLA_FAMILY_WN_MID 14        /* fp16 / bf16 x packed codes at 17..64 rows: weights from registers into the MFMA, activations shared through LDS */
#define GLA_FAMILY_GEMM_16BIT 15    /* unquantised layers above 16 rows: fp16 x fp16 / bf16 x bf16 MFMA GEMM */
int gla_matmul_family(const gla_matmul_args* args);

/* Diagnostic, no counterpart in the reference: launches a register-only loop of
 * 8 * iters independent MFMAs per wave, two waves on every SIMD, no memory
 * traffic, and stores the flops of the launch in *flops (may be NULL).  The
 * caller times it (events on `stream`).  dtype: GLA_DT_FP16, GLA_DT_BF16,
 * GLA_DT_FP8, GLA_DT_INT8 or GLA_DT_MXFP4.  With random_operands = 0 the loop
 * reaches the datasheet rate; with 1 the operands are random bits and the
 * board's power limit sets the clock, which is the rate a GEMM on real data can
 * at most sustain.  sink: 4 bytes of device memory (never written in practice). */
int gla_probe_mfma(int dtype, int random_operands, int iters, void* sink, double* flops, void* stream);

/* Diagnostic, no counterpart in the reference: one kernel that reads `bytes` bytes of `buf` once
 * (contiguous chunk per workgroup, 128-bit non-temporal loads, eight in flight per lane) and stores
 * nothing.  Timed by the caller over rotated buffers, it gives the rate at which a kernel can
 * stream a footprint of that size on the device at hand, launch ramp and tail included: the
 * ceiling of the weight-streaming kernels.  buf: 16-byte aligned device memory, bytes a multiple
 * of 16; sink: 4 bytes of device memory (never written in practice). */
int gla_probe_read(const void* buf, int64_t bytes, void* sink, void* stream);

/* Diagnostic, no counterpart in the reference: gla_probe_read with the launch shape chosen by the
 * caller: `workgroups` workgroups of `threads` threads (a multiple of 64, at most 1024), `loads`
 * (4, 8 or 16) 128-bit loads in flight per lane.  A caller that sweeps a few shapes and keeps the
 * best gets the read ceiling of the device for a footprint rather than that of one launch shape. */
int gla_probe_read_cfg(const void* buf, int64_t bytes, void* sink, int workgroups, int threads, int loads, void* stream);

/* No counterpart in the reference (its kernels rely on the hardware caches as they are).  Reads
 * [buf, buf + bytes) once with cacheable loads and stores nothing, so that the bytes sit in the
 * device's memory-side cache (256 MB on MI355X) when the next kernel asks for them.  Meant for a
 * decode loop that knows which layer runs next: launched on a second stream (or a forked branch of a
 * captured graph) while layer L runs, it streams the weights of layer L+1 during L's launch gap,
 * ramp and tail, when the memory system is otherwise idle.  workgroups: grid size, 0 for the default
 * (256); never allocates, never synchronises. */
int gla_prefetch(const void* buf, int64_t bytes, int workgroups, void* stream);

/* Scratch bytes gla_matmul needs for these arguments (0 if none).  The scratch
 * must be zero-filled once when it is allocated; the library leaves it zeroed
 * where it needs zeros.  (Plays the role of the reference's pre-zeroed output
 * ring, gemlite/triton_kernels/config.py:31-34.) */
int64_t gla_matmul_workspace_bytes(const gla_matmul_args* args);

/* Launch one quantized matmul (reference: the five launchers listed above). */
int gla_matmul(const gla_matmul_args* args, void* stream);

/* gla_matmul for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, same kernels and bit-identical results, except that `workspace` / `workspace_bytes` of
 * the struct are ignored: the scratch is a device array of GLA_STATIC_SCRATCH_BYTES bytes that the
 * library's code object carries (each GPU the library runs on holds its own copy until the process
 * ends).  The call allocates and frees nothing.  A problem whose gla_matmul_workspace_bytes()
 * exceeds GLA_STATIC_SCRATCH_BYTES is refused with GLA_ERR_WORKSPACE_TOO_SMALL, with one exception: a
 * packed layer at prefill size whose unpacked 16-bit weights (N * K * 2 bytes) would not fit runs on
 * the fused kernel instead, as gla_matmul does with GLA_TILE_PREFER_MATRIX.  The first call on
 * a device that needs scratch looks the array's address up; nothing is cleared (the array is zero
 * when the code object is loaded, and every kernel leaves the counters and slots it used at zero
 * again), so that first call may itself be recorded into a graph.  All calls on one GPU share the array: calls that may overlap in time
 * on one GPU (two streams, two graphs replayed concurrently) race and must use gla_matmul with
 * workspaces of their own. */
#define GLA_STATIC_SCRATCH_BYTES (72u << 20)
int64_t gla_static_scratch_bytes(void);
int gla_matmul_static(const gla_matmul_args* args, void* stream);

/* Per-token dynamic activation quantisation to fp8-e4m3fn or int8:
 *   s[m] = max(amax(|x[m,:]|) / qmax, 1e-6);  y = clamp(x / s, qmin, qmax);
 *   int8 rounds with floor(y + 0.5).
 * x: [M, K] fp16/bf16/fp32 with row stride x_stride_m; y: [M, K] contiguous;
 * scales: [M] fp32.
 * (reference: gemlite/quant_utils.py:467-539, rounding :289-296) */
int gla_scale_activations_per_token(const void* x, int x_dtype, int64_t x_stride_m, int M, int K,
                                    void* y, int y_dtype, float* scales, void* stream);

/* MXFP4 dynamic activation quantisation: per 32 consecutive k one e8m0 scale
 * 2^ceil(log2(amax/6)) (exponent clamped to [97, 254]) and 32 e2m1 codes, two
 * per byte, even k in the low nibble.  y: [M, K/2] bytes; scales: [M_pad, K/32]
 * bytes with M_pad = M rounded up to 32; rows M..M_pad-1 are set to 127.
 * (reference: gemlite/quant_utils.py:2005-2135, exponent trick :697-705) */
int gla_scale_activations_mxfp4(const void* x, int x_dtype, int64_t x_stride_m, int M, int K,
                                uint8_t* y, uint8_t* scales, void* stream);

/* MXFP8 dynamic activation quantisation: per 32 consecutive k one e8m0 scale
 * 2^ceil(log2(amax/448)) (exponent clamped to [97, 254]) and 32 fp8-e4m3fn codes
 * of clamp(x / scale, -448, 448), rounded to nearest even.  y: [M, K] bytes;
 * scales: [M_pad, K/32] bytes with M_pad = M rounded up to 32; rows M..M_pad-1
 * are set to 127.  (reference: gemlite/quant_utils.py:1025-1127, exponent trick :697-705) */
int gla_scale_activations_mxfp8(const void* x, int x_dtype, int64_t x_stride_m, int M, int K,
                                uint8_t* y, uint8_t* scales, void* stream);

/* Per-block dynamic activation quantisation for channel_scale_mode 5: one fp32
 * scale max(amax / qmax, 1e-6) per (row, 128 consecutive k), y = clamp(x * (1 / scale))
 * as int8 (rounded floor(v + 0.5)) or fp8-e4m3fn (nearest even).  y: [M, K] bytes
 * contiguous; scales: [M, K/128] fp32 contiguous.  K must be a multiple of 128.
 * (reference: gemlite/quant_utils.py:2614-2676) */
int gla_scale_activations_per_block(const void* x, int x_dtype, int64_t x_stride_m, int M, int K,
                                    void* y, int y_dtype, float* scales, void* stream);

/* Pack rows x cols 8-bit codes into words of packing_bitwidth bits along the
 * column axis; out is [rows, cols/e] contiguous
 * (reference: gemlite/bitpack.py:77-144). */
int gla_pack_over_cols(const uint8_t* codes, void* out, int64_t rows, int64_t cols, int W_nbits,
                       int packing_bitwidth, void* stream);

/* Inverse of gla_pack_over_cols; out is [rows, packed_cols*e] bytes
 * (reference: gemlite/bitpack.py:164-205). */
int gla_unpack_over_cols(const void* packed, uint8_t* out, int64_t rows, int64_t packed_cols,
                         int W_nbits, int packing_bitwidth, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GEMLITE_AMD_H */
