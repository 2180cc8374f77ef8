// Walsh-Hadamard transform of fp16 rows: y = fp16((x . H_block) * scale), H the
// Sylvester (natural-order) matrix, applied to consecutive `block`-wide pieces.
// Butterflies run in fp32, lowest index bit first, one rounding to fp16 at the end.
#include "common.hpp"
#include "fwht_device.hpp"
#include "hadamard_base.hpp"

namespace uniql {

// ---- block == 128: one 16-lane group per piece, all in registers ------------------
__global__ __launch_bounds__(256) void fwht128_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ y,
                                                     int64_t pieces, float scale) {
    const int64_t piece = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int seg = threadIdx.x & 15;
    // every lane of a 16-lane group shares `piece`, so the exchange below never
    // crosses into a group that has left
    if (piece >= pieces) return;
    const u32x4 v = x[piece * 16 + seg];
    float f[8];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const h2 hv = bits_to_h2(v[p]);
        f[2 * p] = (float)hv.x;
        f[2 * p + 1] = (float)hv.y;
    }
    wht128_row16(f, seg);
    u32x4 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        h2 hv;
        hv.x = scaled_to_half(f[2 * p], scale);
        hv.y = scaled_to_half(f[2 * p + 1], scale);
        o[p] = h2_to_bits(hv);
    }
    y[piece * 16 + seg] = o;
}

// ---- general power of two: one workgroup per piece, fp32 image in LDS --------------
// A pass handles CNT consecutive index bits starting at bit `lo`: each task gathers
// 2^CNT values whose indices differ only in those bits, runs CNT butterfly stages in
// registers and scatters them back.
template <int CNT>
__device__ __forceinline__ void fwht_pass(float* buf, int L, int lo, int tid, int nthreads) {
    constexpr int E = 1 << CNT;
    const int tasks = L >> CNT;
    const int lowmask = (1 << lo) - 1;
    for (int t = tid; t < tasks; t += nthreads) {
        const int base = ((t >> lo) << (lo + CNT)) | (t & lowmask);
        float v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) v[i] = buf[base + (i << lo)];
#pragma unroll
        for (int h = 1; h < E; h <<= 1) {
#pragma unroll
            for (int i = 0; i < E; ++i) {
                if ((i & h) == 0) {
                    const float p = v[i], q = v[i + h];
                    v[i] = p + q;
                    v[i + h] = p - q;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < E; ++i) buf[base + (i << lo)] = v[i];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void fwht_lds_kernel(const T* __restrict__ x, T* __restrict__ y, int L,
                                                      int log2L, float scale) {
    extern __shared__ __attribute__((aligned(16))) float fbuf[];
    const int tid = threadIdx.x;
    const T* xp = x + (size_t)blockIdx.x * L;
    T* yp = y + (size_t)blockIdx.x * L;
    for (int i = tid; i < L; i += 256) fbuf[i] = (float)xp[i];
    __syncthreads();
    int lo = 0;
    while (lo < log2L) {
        const int left = log2L - lo;
        if (left >= 3) {
            fwht_pass<3>(fbuf, L, lo, tid, 256);
            lo += 3;
        } else if (left == 2) {
            fwht_pass<2>(fbuf, L, lo, tid, 256);
            lo += 2;
        } else {
            fwht_pass<1>(fbuf, L, lo, tid, 256);
            lo += 1;
        }
        __syncthreads();
    }
    for (int i = tid; i < L; i += 256) {
        float p = fbuf[i] * scale;
        asm volatile("" : "+v"(p));  // see scaled_to_half: keep multiply and rounding separate
        yp[i] = (T)p;
    }
}

// ---- fp16, power of two >= 256: vector loads, index bits 0..2 in registers, LDS passes of
// up to four bits (fwht_row_to_lds), vector stores ----------------------------------------------
__global__ __launch_bounds__(1024) void fwht_f16_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ y, int L,
                                                       int log2L, float scale) {
    extern __shared__ __attribute__((aligned(16))) float fbuf[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int chunks = L >> 3;
    const u32x4* xp = x + (size_t)blockIdx.x * chunks;
    u32x4* yp = y + (size_t)blockIdx.x * chunks;
    fwht_row_to_lds(xp, fbuf, L, log2L, tid, nthreads);
    for (int c = tid; c < chunks; c += nthreads) {
        const float* src = fbuf + fwht_pad(8 * c);
        const f4 a = *reinterpret_cast<const f4*>(src), b = *reinterpret_cast<const f4*>(src + 4);
        h2 r0, r1, r2, r3;
        r0.x = scaled_to_half(a[0], scale);
        r0.y = scaled_to_half(a[1], scale);
        r1.x = scaled_to_half(a[2], scale);
        r1.y = scaled_to_half(a[3], scale);
        r2.x = scaled_to_half(b[0], scale);
        r2.y = scaled_to_half(b[1], scale);
        r3.x = scaled_to_half(b[2], scale);
        r3.y = scaled_to_half(b[3], scale);
        yp[c] = u32x4{h2_to_bits(r0), h2_to_bits(r1), h2_to_bits(r2), h2_to_bits(r3)};
    }
}

// Long rows (L >= 4096), fp16: two LDS exchanges instead of one per four index bits.
//   load    every thread takes L/8/T sixteen-byte chunks (consecutive lanes on consecutive chunks),
//           transforms index bits 0..2 in registers and writes fp32 to LDS;
//   middle  index bits 3 .. n-6 in passes of up to five bits (32 values per task in registers);
//   final   the top five bits: a thread reads two neighbouring values at 32 strides of L/32,
//           transforms, scales, rounds and stores 4 bytes per stride: consecutive lanes store
//           consecutive words, no trip back through LDS.
// The stages run in ascending bit order like everywhere else, so the fp32 sums are associated
// the same way and the result is the same bit for bit.  T = L / 64 threads per row.
__global__ __launch_bounds__(512) void fwht_f16_wide_kernel(const u32x4* __restrict__ x, uint32_t* __restrict__ y,
                                                           int L, int log2L, float scale) {
    extern __shared__ __attribute__((aligned(16))) float fbuf[];
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int chunks = L >> 3;
    const u32x4* xp = x + (size_t)blockIdx.x * chunks;
    uint32_t* yp = y + (size_t)blockIdx.x * (L >> 1);
    constexpr int kChunksPerThread = 8;  // chunks / nthreads = (L / 8) / (L / 64)
    u32x4 v[kChunksPerThread];
#pragma unroll
    for (int i = 0; i < kChunksPerThread; ++i) v[i] = xp[tid + i * nthreads];
#pragma unroll
    for (int i = 0; i < kChunksPerThread; ++i) {
        float f[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const h2 hv = bits_to_h2(v[i][p]);
            f[2 * p] = (float)hv.x;
            f[2 * p + 1] = (float)hv.y;
        }
#pragma unroll
        for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if ((e & h) == 0) {
                    const float p = f[e], q = f[e + h];
                    f[e] = p + q;
                    f[e + h] = p - q;
                }
            }
        }
        float* dst = fbuf + fwht_pad(8 * (tid + i * nthreads));
        *reinterpret_cast<f4*>(dst) = f4{f[0], f[1], f[2], f[3]};
        *reinterpret_cast<f4*>(dst + 4) = f4{f[4], f[5], f[6], f[7]};
    }
    __syncthreads();
    // index bits 3 .. log2L - 6 (log2L = 12 .. 15), then the top five bits in the final phase
    switch (log2L) {
        case 12: fwht_pass_fixed<4, 3>(fbuf, L, tid, nthreads); __syncthreads(); break;
        case 13: fwht_pass_fixed<5, 3>(fbuf, L, tid, nthreads); __syncthreads(); break;
        case 14:
            fwht_pass_fixed<5, 3>(fbuf, L, tid, nthreads);
            __syncthreads();
            fwht_pass_fixed<1, 8>(fbuf, L, tid, nthreads);
            __syncthreads();
            break;
        case 15:
            fwht_pass_fixed<5, 3>(fbuf, L, tid, nthreads);
            __syncthreads();
            fwht_pass_fixed<2, 8>(fbuf, L, tid, nthreads);
            __syncthreads();
            break;
        default: break;
    }
    // final phase: values 2 tid, 2 tid + 1 at the 32 strides of L / 32
    const int stride = L >> 5;
    float a[32], b[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        const float* src = fbuf + fwht_pad(2 * tid + j * stride);
        a[j] = src[0];
        b[j] = src[1];
    }
#pragma unroll
    for (int h = 1; h < 32; h <<= 1) {
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            if ((j & h) == 0) {
                const float p = a[j], q = a[j + h];
                a[j] = p + q;
                a[j + h] = p - q;
                const float r = b[j], t = b[j + h];
                b[j] = r + t;
                b[j + h] = r - t;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        h2 r;
        r.x = scaled_to_half(a[j], scale);
        r.y = scaled_to_half(b[j], scale);
        yp[tid + j * (stride >> 1)] = h2_to_bits(r);
    }
}

static int fwht_f16_launch(const void* x, void* y, int64_t pieces, int block, float scale, hipStream_t stream) {
    int log2L = 0;
    while ((1 << log2L) < block) ++log2L;
    const size_t shmem = (size_t)(block + (block >> 7) * 8) * sizeof(float);
    if (shmem > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&fwht_f16_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess ||
            hipFuncSetAttribute(reinterpret_cast<const void*>(&fwht_f16_wide_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
            return UNIQL_E_LAUNCH;
    }
    if (block >= 4096) {
        hipLaunchKernelGGL(fwht_f16_wide_kernel, dim3((unsigned)pieces), dim3(block / 64), shmem, stream,
                           reinterpret_cast<const u32x4*>(x), reinterpret_cast<uint32_t*>(y), block, log2L, scale);
        return UNIQL_OK;
    }
    const int threads = block / 8 < 1024 ? block / 8 : 1024;
    hipLaunchKernelGGL(fwht_f16_kernel, dim3((unsigned)pieces), dim3(threads), shmem, stream,
                       reinterpret_cast<const u32x4*>(x), reinterpret_cast<u32x4*>(y), block, log2L, scale);
    return UNIQL_OK;
}

// ---- composite widths: dim = BASE * P with P a power of two -----------------------------------
// The row is BASE chunks of P values: every chunk gets the P-point transform (LDS passes over
// the whole row touch only index bits below log2 P, so the chunks stay apart), then the BASE x BASE
// matrix combines the chunks: y[c P + i] = sum_c' z[c' P + i] H[c'][c], added in ascending c' in
// fp32; one rounding at the end.
template <typename T, int BASE>
__global__ __launch_bounds__(256) void fwht_composite_kernel(const T* __restrict__ x, T* __restrict__ y, int P,
                                                            int log2P, float scale) {
    extern __shared__ __attribute__((aligned(16))) float fbuf[];
    const uint64_t* table = BASE == 12 ? kHadamard12 : BASE == 20 ? kHadamard20 : BASE == 28 ? kHadamard28 : kHadamard40;
    const int tid = threadIdx.x;
    const int L = BASE * P;
    const T* xp = x + (size_t)blockIdx.x * L;
    T* yp = y + (size_t)blockIdx.x * L;
    for (int i = tid; i < L; i += 256) fbuf[i] = (float)xp[i];
    __syncthreads();
    int lo = 0;
    while (lo < log2P) {
        const int left = log2P - lo;
        if (left >= 3) {
            fwht_pass<3>(fbuf, L, lo, tid, 256);
            lo += 3;
        } else if (left == 2) {
            fwht_pass<2>(fbuf, L, lo, tid, 256);
            lo += 2;
        } else {
            fwht_pass<1>(fbuf, L, lo, tid, 256);
            lo += 1;
        }
        __syncthreads();
    }
    for (int i = tid; i < P; i += 256) {
        float z[BASE];
#pragma unroll
        for (int c = 0; c < BASE; ++c) z[c] = fbuf[c * P + i];
#pragma unroll
        for (int c = 0; c < BASE; ++c) {
            const uint64_t minus = table[c];
            float sum = 0.f;
#pragma unroll
            for (int cp = 0; cp < BASE; ++cp) sum += ((minus >> cp) & 1ull) ? -z[cp] : z[cp];
            float p = sum * scale;
            asm volatile("" : "+v"(p));  // see scaled_to_half: keep multiply and rounding separate
            yp[c * P + i] = (T)p;
        }
    }
}

template <typename T, int BASE>
static int fwht_composite_go(const void* x, void* y, int64_t rows, int P, float scale, hipStream_t stream) {
    int log2P = 0;
    while ((1 << log2P) < P) ++log2P;
    const size_t shmem = (size_t)BASE * P * sizeof(float);
    auto kern = &fwht_composite_kernel<T, BASE>;
    if (shmem > 64 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)shmem) != hipSuccess)
        return UNIQL_E_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(256), shmem, stream, reinterpret_cast<const T*>(x),
                       reinterpret_cast<T*>(y), P, log2P, scale);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

template <typename T>
static int fwht_composite_base(const void* x, void* y, int64_t rows, int base, int P, float scale, hipStream_t stream) {
    switch (base) {
        case 12: return fwht_composite_go<T, 12>(x, y, rows, P, scale, stream);
        case 20: return fwht_composite_go<T, 20>(x, y, rows, P, scale, stream);
        case 28: return fwht_composite_go<T, 28>(x, y, rows, P, scale, stream);
        case 40: return fwht_composite_go<T, 40>(x, y, rows, P, scale, stream);
        default: return UNIQL_E_UNSUPPORTED;
    }
}

int fwht_composite_launch(const void* x, void* y, int64_t rows, int dim, int base, float scale, int dtype,
                          hipStream_t stream) {
    if (rows == 0) return UNIQL_OK;
    if (rows > 0x7fffffffLL) return UNIQL_E_SHAPE;
    const int P = dim / base;
    if (dtype == UNIQL_DT_F16) return fwht_composite_base<half_t>(x, y, rows, base, P, scale, stream);
    if (dtype == UNIQL_DT_BF16) return fwht_composite_base<__bf16>(x, y, rows, base, P, scale, stream);
    return fwht_composite_base<float>(x, y, rows, base, P, scale, stream);
}

template <typename T>
static int fwht_lds_launch(const void* x, void* y, int64_t pieces, int block, float scale, hipStream_t stream) {
    int log2L = 0;
    while ((1 << log2L) < block) ++log2L;
    const size_t shmem = (size_t)block * sizeof(float);
    if (shmem > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&fwht_lds_kernel<T>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem) != hipSuccess)
            return UNIQL_E_LAUNCH;
    }
    hipLaunchKernelGGL((fwht_lds_kernel<T>), dim3((unsigned)pieces), dim3(256), shmem, stream,
                       reinterpret_cast<const T*>(x), reinterpret_cast<T*>(y), block, log2L, scale);
    return UNIQL_OK;
}

int fwht_launch(const void* x, void* y, int64_t rows, int dim, int block, float scale, int dtype,
                hipStream_t stream) {
    const int64_t pieces = rows * (dim / block);
    if (pieces == 0) return UNIQL_OK;
    if (block == 128 && dtype == UNIQL_DT_F16) {
        const int64_t grid = (pieces + 15) / 16;
        if (grid > 0x7fffffffLL) return UNIQL_E_SHAPE;
        hipLaunchKernelGGL(fwht128_kernel, dim3((unsigned)grid), dim3(256), 0, stream,
                           reinterpret_cast<const u32x4*>(x), reinterpret_cast<u32x4*>(y), pieces, scale);
    } else {
        if (pieces > 0x7fffffffLL) return UNIQL_E_SHAPE;
        int rc;
        if (dtype == UNIQL_DT_F16 && block >= 256) rc = fwht_f16_launch(x, y, pieces, block, scale, stream);
        else if (dtype == UNIQL_DT_F16) rc = fwht_lds_launch<half_t>(x, y, pieces, block, scale, stream);
        else if (dtype == UNIQL_DT_BF16) rc = fwht_lds_launch<__bf16>(x, y, pieces, block, scale, stream);
        else rc = fwht_lds_launch<float>(x, y, pieces, block, scale, stream);
        if (rc != UNIQL_OK) return rc;
    }
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
