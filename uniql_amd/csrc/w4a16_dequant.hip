// Device-side inverse of the packed weight layout: raw codes and dequantised
// fp16 weights in natural [K, N] order.  A verification and tooling kernel
// (bit-exact contract of the layout), not a fast path.
#include "common.hpp"

namespace uniql {

// One thread per 16-byte piece.  Piece p of packed row r, chunk c (p = 4*c8 + kq)
// holds, in 32-bit word j, nibble pairs
//   low  form of q      : K-rows 2kq, 2kq+1   of column 16j + c8
//   high form of q      : K-rows 2kq+8, 2kq+9 of column 16j + c8
//   low / high of q >> 8: the same rows of column 16j + 8 + c8
__global__ __launch_bounds__(256) void w4a16_dequant_kernel(const u32x4* __restrict__ B,
                                                           const half_t* __restrict__ S,
                                                           half_t* __restrict__ W, uint8_t* __restrict__ codes,
                                                           int N, int K, int per_column) {
    const int64_t pieces_per_row = N >> 1;
    const int64_t total = (int64_t)(K >> 4) * pieces_per_row;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int r = (int)(idx / pieces_per_row);
    const int rem = (int)(idx % pieces_per_row);
    const int chunk = rem >> 5, piece = rem & 31;
    const int c8 = piece >> 2, kq = piece & 3;
    const u32x4 q4 = B[idx];
    const int g = (16 * r) >> 7;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const uint32_t q = blk ? (q4[j] >> 8) : q4[j];
            const int n = 64 * chunk + 16 * j + 8 * blk + c8;
            half_t s;
            if (per_column)
                s = S[single_scale_pos(n)];
            else
                s = S[(size_t)g * N + 64 * chunk + 8 * c8 + 2 * j + blk];
            const h2 sv = h2{s, s};
            const h2 lo = code_pair_low(q) * sv;
            const h2 hi = code_pair_high(q) * sv;
            const int k0 = 16 * r + 2 * kq;
            if (W) {
                W[(size_t)(k0)*N + n] = lo.x;
                W[(size_t)(k0 + 1) * N + n] = lo.y;
                W[(size_t)(k0 + 8) * N + n] = hi.x;
                W[(size_t)(k0 + 9) * N + n] = hi.y;
            }
            if (codes) {
                codes[(size_t)(k0)*N + n] = (uint8_t)(q & 15u);
                codes[(size_t)(k0 + 1) * N + n] = (uint8_t)((q >> 16) & 15u);
                codes[(size_t)(k0 + 8) * N + n] = (uint8_t)((q >> 4) & 15u);
                codes[(size_t)(k0 + 9) * N + n] = (uint8_t)((q >> 20) & 15u);
            }
        }
    }
}

int dequant_launch(const void* B, const void* S, void* W, uint8_t* codes, int n, int k, int groups,
                   hipStream_t stream) {
    const int64_t total = (int64_t)(k / 16) * (n / 2);
    const int grid = (int)((total + 255) / 256);
    hipLaunchKernelGGL(w4a16_dequant_kernel, dim3(grid), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4*>(B), reinterpret_cast<const half_t*>(S),
                       reinterpret_cast<half_t*>(W), codes, n, k, groups == 1 ? 1 : 0);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
