// Measurement aids and small utilities that are not part of the product path (declared in
// include/uniql_amd_diag.h, except uniql_clear).
#include "common.hpp"

namespace uniql {

// What the matrix pipe alone sustains: every wave of 256 workgroups x 4 waves issues `iters`
// times eight independent v_mfma_f32_32x32x16_f16 on operands it loaded once (no loads, no LDS
// reads, no expansion in the loop).  The operands decide the switching activity and with it the
// clock the chip settles at, so the caller chooses them (zeros, or values like the workload's).
__global__ __launch_bounds__(256) void mfma_loop_kernel(const h8* __restrict__ operands, float* __restrict__ out,
                                                       int iters) {
    const h8 a = operands[threadIdx.x], b = operands[256 + threadIdx.x];
    f16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = f16{};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][7] + acc[i][15];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void clear_kernel(u32x4* p, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) p[i] = u32x4{0u, 0u, 0u, 0u};
}

}  // namespace uniql

using namespace uniql;

extern "C" {

int uniql_diag_mfma_loop(const void* operands, void* out, int iters, void* stream) {
    if (iters < 0) return UNIQL_E_SHAPE;
    if (!operands || !out) return UNIQL_E_NULL;
    if ((reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return UNIQL_E_ALIGN;
    hipLaunchKernelGGL(mfma_loop_kernel, dim3(256), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       reinterpret_cast<const h8*>(operands), reinterpret_cast<float*>(out), iters);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

int uniql_clear(void* p, size_t bytes, void* stream) {
    if (bytes == 0) return UNIQL_OK;
    if (!p) return UNIQL_E_NULL;
    if ((reinterpret_cast<uintptr_t>(p) & 15u) != 0 || bytes % 16 != 0) return UNIQL_E_ALIGN;
    const size_t count = bytes / sizeof(u32x4);
    if ((count + 255) / 256 > 0x7fffffffull) return UNIQL_E_SHAPE;
    hipLaunchKernelGGL(clear_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), reinterpret_cast<u32x4*>(p), count);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // extern "C"
