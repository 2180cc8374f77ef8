// Producer side of the packed layout on the device: group-128 quantisation of an fp16 weight
// matrix into int4 codes + fp16 scales, and the packing of codes into the kernel's word order.
// Offline operations (run once per layer): written for clarity and bit-exactness with the
// host arithmetic of the reference (fp16 tensors on the CPU: every operation rounds its fp32
// result to fp16), not for the last GB/s.
#include "common.hpp"

namespace uniql {

// fp16 result of an fp16 x fp32-constant product, an fp16 / fp16 quotient and an fp16 + 8 sum,
// each computed in fp32 and rounded once to fp16, as torch does for half tensors on the CPU
__device__ __forceinline__ half_t half_div(half_t a, half_t b) { return (half_t)((float)a / (float)b); }

// Position of column n's scale inside a permuted scale row (group-128 case): inside every 64
// columns, position 8 i + j holds column i + 8 j.
__device__ __forceinline__ int64_t group_scale_pos(int n) { return (n & ~63) + 8 * (n & 7) + ((n & 63) >> 3); }

// One wavefront per (group g, output row n): scale = fp16(max |w| * (2/15)) over the 128 K values
// of the group (zero beyond in_features and for n >= out_features), written at the permuted
// position.  With `given` the scales are copied from a natural-order [groups][out_features] array.
__global__ __launch_bounds__(256) void w4a16_group_scales_kernel(const half_t* __restrict__ W, int64_t ldw,
                                                                const half_t* __restrict__ given,
                                                                half_t* __restrict__ S, int out_features,
                                                                int in_features, int n_pad, int groups) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= (int64_t)groups * n_pad) return;
    const int g = (int)(wave / n_pad), n = (int)(wave % n_pad);
    half_t scale = (half_t)0.0f;
    if (n < out_features) {
        if (given) {
            scale = given[(size_t)g * out_features + n];
        } else {
            float amax = 0.f;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int k = 128 * g + 2 * lane + i;
                if (k < in_features) amax = fmaxf(amax, fabsf((float)W[(size_t)n * ldw + k]));
            }
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d, kWave));
            scale = scaled_to_half(amax, (float)(2.0 / 15.0));   // fp32 product, then one rounding to fp16
        }
    }
    if (lane == 0) S[(size_t)g * n_pad + group_scale_pos(n)] = scale;
}

// code of one weight; `gptq`: the scales were handed over and the reference computes
// round(w / s + 8) (quantize_helpers.py:216-217) instead of round(w / s) + 8 (:114).
// A quotient that is not finite (0/0 in an all-zero group, x/0 when the scale underflowed)
// becomes INT_MIN in the reference's float -> int conversion and so code 0 after the clamp.
__device__ __forceinline__ uint32_t quantize_code(half_t w, half_t s, bool gptq) {
    const half_t q = half_div(w, s);
    float r;
    if (gptq) {
        const half_t shifted = (half_t)((float)q + 8.0f);
        if (!__builtin_isfinite((float)shifted)) return 0u;
        r = __builtin_rintf((float)shifted);
    } else {
        if (!__builtin_isfinite((float)q)) return 0u;
        r = __builtin_rintf((float)q) + 8.0f;
    }
    return (uint32_t)fminf(fmaxf(r, 0.0f), 15.0f);
}

// One thread per packed 32-bit word.  Word j of piece (c8, kq) of chunk c of packed row r holds,
// in nibble 4 lo + 2 blk + hi, K row 16 r + 2 kq + 8 hi + lo of column 64 c + 16 j + 8 blk + c8.
// SRC 0: quantise fp16 weights W[n][k] (row stride ldw) with the scales already in S (permuted);
// SRC 1: take ready codes[k][n].
template <int SRC>
__global__ __launch_bounds__(256) void w4a16_pack_kernel(const half_t* __restrict__ W, int64_t ldw,
                                                        const uint8_t* __restrict__ codes,
                                                        const half_t* __restrict__ S, uint32_t* __restrict__ B,
                                                        int out_features, int in_features, int n_pad, int k_pad,
                                                        int gptq) {
    const int64_t words_per_row = 2 * (int64_t)n_pad;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)(k_pad >> 4) * words_per_row) return;
    const int r = (int)(idx / words_per_row);
    const int c = (int)(idx % words_per_row);
    const int chunk = c >> 7, piece = (c >> 2) & 31, j = c & 3;
    const int c8 = piece >> 2, kq = piece & 3;
    const int g = r >> 3;
    uint32_t word = 0u;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const int n = 64 * chunk + 16 * j + 8 * blk + c8;
        half_t s = (half_t)0.0f;
        if (SRC == 0) s = S[(size_t)g * n_pad + group_scale_pos(n)];
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
#pragma unroll
            for (int lo = 0; lo < 2; ++lo) {
                const int k = 16 * r + 2 * kq + 8 * hi + lo;
                uint32_t code = 0u;  // columns past out_features: code 0 (and scale 0)
                if (n < out_features) {
                    if (SRC == 0) {
                        const half_t w = k < in_features ? W[(size_t)n * ldw + k] : (half_t)0.0f;
                        code = quantize_code(w, s, gptq != 0);
                    } else {
                        code = k < in_features ? (uint32_t)(codes[(size_t)k * out_features + n] & 15u) : 8u;
                    }
                }
                word |= code << (4 * (4 * lo + 2 * blk + hi));
            }
        }
    }
    B[idx] = word;
}

// natural-order scales [groups][n] -> permuted rows of width n_pad (zeros in the padding)
__global__ __launch_bounds__(256) void w4a16_permute_scales_kernel(const half_t* __restrict__ src,
                                                                  half_t* __restrict__ S, int n, int n_pad,
                                                                  int groups) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)groups * n_pad) return;
    const int g = (int)(idx / n_pad), col = (int)(idx % n_pad);
    S[(size_t)g * n_pad + group_scale_pos(col)] = col < n ? src[(size_t)g * n + col] : (half_t)0.0f;
}

int quantize_launch(const void* W, int64_t ldw, const void* given_scales, void* B, void* S, int out_features,
                    int in_features, int n_pad, int k_pad, hipStream_t stream) {
    const int groups = k_pad / 128;
    const int64_t waves = (int64_t)groups * n_pad;
    hipLaunchKernelGGL(w4a16_group_scales_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream,
                       reinterpret_cast<const half_t*>(W), ldw, reinterpret_cast<const half_t*>(given_scales),
                       reinterpret_cast<half_t*>(S), out_features, in_features, n_pad, groups);
    const int64_t words = (int64_t)(k_pad / 16) * 2 * n_pad;
    hipLaunchKernelGGL(w4a16_pack_kernel<0>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const half_t*>(W), ldw, (const uint8_t*)nullptr,
                       reinterpret_cast<const half_t*>(S), reinterpret_cast<uint32_t*>(B), out_features,
                       in_features, n_pad, k_pad, given_scales ? 1 : 0);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

int pack_launch(const uint8_t* codes, const void* scales, void* B, void* S, int n, int k, int n_pad, int k_pad,
                hipStream_t stream) {
    const int groups = k_pad / 128;
    const int64_t sc = (int64_t)groups * n_pad;
    hipLaunchKernelGGL(w4a16_permute_scales_kernel, dim3((unsigned)((sc + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const half_t*>(scales), reinterpret_cast<half_t*>(S), n, n_pad, groups);
    const int64_t words = (int64_t)(k_pad / 16) * 2 * n_pad;
    hipLaunchKernelGGL(w4a16_pack_kernel<1>, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream,
                       (const half_t*)nullptr, (int64_t)0, codes, (const half_t*)nullptr,
                       reinterpret_cast<uint32_t*>(B), n, k, n_pad, k_pad, 0);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
