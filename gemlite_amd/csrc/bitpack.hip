// Bit packing / unpacking of weight codes along the column (K) axis.
//
// word[r, c] = OR_i codes[r, c*e + i] << (nbits * i),  e = width / nbits
// (reference: gemlite/bitpack.py:77-144 pack, :164-205 unpack).  One thread
// builds one word; a one-time layout step, not on the per-token path.
#include "common.hpp"
#include "dispatch.hpp"

namespace gla {

namespace {

template <typename WordT>
__global__ __launch_bounds__(256) void pack_cols_kernel(const uint8_t* __restrict__ codes, WordT* __restrict__ out,
                                                        int64_t rows, int64_t pcols, int nbits, int e) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * pcols) return;
    const uint8_t* src = codes + idx * e;  // codes are [rows, pcols * e] contiguous
    uint64_t word = 0;
    const uint64_t mask = (1ull << nbits) - 1ull;
    for (int i = 0; i < e; ++i) word |= ((uint64_t)src[i] & mask) << (nbits * i);
    out[idx] = (WordT)word;
}

template <typename WordT>
__global__ __launch_bounds__(256) void unpack_cols_kernel(const WordT* __restrict__ packed, uint8_t* __restrict__ out,
                                                          int64_t rows, int64_t pcols, int nbits, int e) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * pcols) return;
    const uint64_t word = (uint64_t)packed[idx];
    const uint64_t mask = (1ull << nbits) - 1ull;
    uint8_t* dst = out + idx * e;
    for (int i = 0; i < e; ++i) dst[i] = (uint8_t)((word >> (nbits * i)) & mask);
}

bool check_pack_args(int nbits, int width) {
    if (!(width == 8 || width == 16 || width == 32 || width == 64)) {
        set_error("bitpack: packing width %d not supported (8/16/32/64)", width);
        return false;
    }
    if (!(nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8)) {
        set_error("bitpack: W_nbits %d not supported (1/2/4/8)", nbits);
        return false;
    }
    return true;
}

}  // namespace

int launch_pack_over_cols(const uint8_t* codes, void* out, int64_t rows, int64_t cols, int nbits, int width,
                          hipStream_t stream) {
    if (codes == nullptr || out == nullptr || rows < 0 || cols < 0) {
        set_error("pack_over_cols: null pointer or negative size");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (!check_pack_args(nbits, width)) return GLA_ERR_UNSUPPORTED_MODE;
    const int e = width / nbits;
    if (cols % e != 0) {
        set_error("pack_over_cols: %lld columns not divisible by %d codes per word", (long long)cols, e);
        return GLA_ERR_MISALIGNED_SHAPE;
    }
    const int64_t pcols = cols / e, total = rows * pcols;
    if (total == 0) return GLA_OK;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    switch (width) {
        case 8: hipLaunchKernelGGL(pack_cols_kernel<uint8_t>, grid, block, 0, stream, codes, (uint8_t*)out, rows, pcols, nbits, e); break;
        case 16: hipLaunchKernelGGL(pack_cols_kernel<uint16_t>, grid, block, 0, stream, codes, (uint16_t*)out, rows, pcols, nbits, e); break;
        case 32: hipLaunchKernelGGL(pack_cols_kernel<uint32_t>, grid, block, 0, stream, codes, (uint32_t*)out, rows, pcols, nbits, e); break;
        default: hipLaunchKernelGGL(pack_cols_kernel<uint64_t>, grid, block, 0, stream, codes, (uint64_t*)out, rows, pcols, nbits, e); break;
    }
    return check_hip(hipGetLastError(), "pack_over_cols launch");
}

int launch_unpack_over_cols(const void* packed, uint8_t* out, int64_t rows, int64_t pcols, int nbits, int width,
                            hipStream_t stream) {
    if (packed == nullptr || out == nullptr || rows < 0 || pcols < 0) {
        set_error("unpack_over_cols: null pointer or negative size");
        return GLA_ERR_INVALID_ARGUMENT;
    }
    if (!check_pack_args(nbits, width)) return GLA_ERR_UNSUPPORTED_MODE;
    const int e = width / nbits;
    const int64_t total = rows * pcols;
    if (total == 0) return GLA_OK;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    switch (width) {
        case 8: hipLaunchKernelGGL(unpack_cols_kernel<uint8_t>, grid, block, 0, stream, (const uint8_t*)packed, out, rows, pcols, nbits, e); break;
        case 16: hipLaunchKernelGGL(unpack_cols_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t*)packed, out, rows, pcols, nbits, e); break;
        case 32: hipLaunchKernelGGL(unpack_cols_kernel<uint32_t>, grid, block, 0, stream, (const uint32_t*)packed, out, rows, pcols, nbits, e); break;
        default: hipLaunchKernelGGL(unpack_cols_kernel<uint64_t>, grid, block, 0, stream, (const uint64_t*)packed, out, rows, pcols, nbits, e); break;
    }
    return check_hip(hipGetLastError(), "unpack_over_cols launch");
}

}  // namespace gla
