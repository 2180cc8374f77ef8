// Activation preparation for the tiled kernel: rows whose width is not a multiple of the
// quantisation group are copied into a zero-padded buffer (the module's F.pad,
// quantize/quant_linear_layers.py:96-98).  The streaming kernel pads while loading and does
// not need this.
#include "common.hpp"

namespace uniql {

// dst[m][k] = src[m][0..k_in) followed by zeros; 16-byte pieces, k_in % 8 == 0
__global__ __launch_bounds__(256) void pad_rows_kernel(const u32x4* __restrict__ src, int64_t ld_pieces,
                                                      int in_pieces, u32x4* __restrict__ dst, int out_pieces,
                                                      int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t row = idx / out_pieces;
    const int piece = (int)(idx % out_pieces);
    u32x4 v = u32x4{0u, 0u, 0u, 0u};
    if (piece < in_pieces) v = src[row * ld_pieces + piece];
    dst[idx] = v;
}

int pad_rows_launch(const void* A, int64_t lda, int k_in, void* dst, int k, int m, hipStream_t stream) {
    const int64_t total = (int64_t)m * (k / 8);
    if (total == 0) return UNIQL_OK;
    hipLaunchKernelGGL(pad_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4*>(A), lda / 8, k_in / 8, reinterpret_cast<u32x4*>(dst), k / 8,
                       total);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
