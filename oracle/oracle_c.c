/*
 * C restatement of the reference's CPU path for the quantized linear layer.
 * TEST INFRASTRUCTURE ONLY: used by tests/ (cross-check of the numpy oracle) and
 * by the cpu_baseline leg of bench.py; nothing in gemlite_amd/ links it.
 *
 * The path is "HQQ dequantize, then an fp32 matmul":
 *     W[n,k] = (W_q[n,k] - zeros[g]) * scales[g],  g = (n*K + k) / group_size
 *     y[m,n] = sum_k x[m,k] * W[n,k]
 * (reference: README.md:84, tests/test_int.py:54).  As in the reference's CPU
 * path the dequantised matrix is materialised first and the matmul runs on it.
 */
#include <stddef.h>
#include <stdint.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* W[N*K] = (W_q - zeros[group]) * scales[group], groups of `gs` consecutive elements */
void orc_hqq_dequantize(const uint8_t* W_q, const float* scales, const float* zeros, int64_t N, int64_t K,
                        int64_t gs, float* W, int threads) {
    const int64_t groups = N * K / gs;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads) schedule(static)
#endif
    for (int64_t g = 0; g < groups; ++g) {
        const float s = scales[g], z = zeros[g];
        const uint8_t* q = W_q + g * gs;
        float* w = W + g * gs;
        for (int64_t i = 0; i < gs; ++i) w[i] = ((float)q[i] - z) * s;
    }
}

/* y[M,N] = x[M,K] @ W[N,K]^T in fp32 */
void orc_matmul_nt_f32(const float* x, const float* W, int64_t M, int64_t N, int64_t K, float* y, int threads) {
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads) schedule(static)
#endif
    for (int64_t n = 0; n < N; ++n) {
        const float* w = W + n * K;
        for (int64_t m = 0; m < M; ++m) {
            const float* a = x + m * K;
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            int64_t k = 0;
            for (; k + 8 <= K; k += 8)
                for (int j = 0; j < 8; ++j) acc[j] += a[k + j] * w[k + j];
            float t = 0.f;
            for (; k < K; ++k) t += a[k] * w[k];
            y[m * N + n] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7])) + t;
        }
    }
}

/* word[r, c] = OR_i codes[r, c*e+i] << (nbits*i)  (reference: gemlite/bitpack.py:36-60), 32-bit words */
void orc_pack_over_cols_32(const uint8_t* codes, int64_t rows, int64_t cols, int nbits, int32_t* out) {
    const int e = 32 / nbits;
    const int64_t pcols = cols / e;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < pcols; ++c) {
            uint32_t w = 0;
            for (int i = 0; i < e; ++i) w |= (uint32_t)codes[r * cols + c * e + i] << (nbits * i);
            out[r * pcols + c] = (int32_t)w;
        }
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
