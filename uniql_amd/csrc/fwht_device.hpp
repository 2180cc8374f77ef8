// Device-side pieces of the fp16 Walsh-Hadamard transform shared by the transform kernels and by
// the streaming GEMV kernel's fused full-row rotation.
#pragma once

#include "common.hpp"

namespace uniql {

// The fp32 image in LDS is padded by eight floats per 128: in the first LDS pass (bits 3..6)
// the lanes of a wave differ in bits 0..2 and 7.., and the padding moves each step of bit 7
// to another group of eight banks; the later passes walk consecutive addresses anyway.
__device__ __forceinline__ int fwht_pad(int idx) { return idx + ((idx >> 7) << 3); }

// A pass handles CNT consecutive index bits starting at bit `lo`: each task gathers
// 2^CNT values whose indices differ only in those bits, runs CNT butterfly stages in
// registers and scatters them back.
template <int CNT>
__device__ __forceinline__ void fwht_pass_padded(float* buf, int L, int lo, int tid, int nthreads) {
    constexpr int E = 1 << CNT;
    const int tasks = L >> CNT;
    const int lowmask = (1 << lo) - 1;
    for (int t = tid; t < tasks; t += nthreads) {
        const int base = ((t >> lo) << (lo + CNT)) | (t & lowmask);
        float v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) v[i] = buf[fwht_pad(base + (i << lo))];
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
        for (int i = 0; i < E; ++i) buf[fwht_pad(base + (i << lo))] = v[i];
    }
}

// The same with the first bit known at compile time: every address of a task is the first one
// plus a constant (the task's values lie (i << LO) apart and those bits of the first index are zero,
// so the padding term of value i is that of the first index plus ((i << LO) >> 7) << 3): the index
// arithmetic is done once per task instead of once per value.
template <int CNT, int LO>
__device__ __forceinline__ void fwht_pass_fixed(float* buf, int L, int tid, int nthreads) {
    constexpr int E = 1 << CNT;
    const int tasks = L >> CNT;
    constexpr int lowmask = (1 << LO) - 1;
    for (int t = tid; t < tasks; t += nthreads) {
        float* p0 = buf + fwht_pad(((t >> LO) << (LO + CNT)) | (t & lowmask));
        float v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) v[i] = p0[(i << LO) + (((i << LO) >> 7) << 3)];
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
        for (int i = 0; i < E; ++i) p0[(i << LO) + (((i << LO) >> 7) << 3)] = v[i];
    }
}

// index bits [LO, min(LO + 4, log2L)) of one row image
template <int LO>
__device__ __forceinline__ void fwht_pass_from(float* buf, int L, int log2L, int tid, int nthreads) {
    const int left = log2L - LO;
    if (left >= 4) fwht_pass_fixed<4, LO>(buf, L, tid, nthreads);
    else if (left == 3) fwht_pass_fixed<3, LO>(buf, L, tid, nthreads);
    else if (left == 2) fwht_pass_fixed<2, LO>(buf, L, tid, nthreads);
    else if (left == 1) fwht_pass_fixed<1, LO>(buf, L, tid, nthreads);
}

// index bits 3 .. log2L - 1 (log2L <= 19) of `rows` row images `row_floats` apart, four bits per
// pass, one workgroup barrier after each pass
__device__ __forceinline__ void fwht_passes_from_bit3(float* images, int rows, int row_floats, int L, int log2L, int tid,
                                                      int nthreads) {
    if (log2L > 3) {
        for (int m = 0; m < rows; ++m) fwht_pass_from<3>(images + (size_t)m * row_floats, L, log2L, tid, nthreads);
        __syncthreads();
    }
    if (log2L > 7) {
        for (int m = 0; m < rows; ++m) fwht_pass_from<7>(images + (size_t)m * row_floats, L, log2L, tid, nthreads);
        __syncthreads();
    }
    if (log2L > 11) {
        for (int m = 0; m < rows; ++m) fwht_pass_from<11>(images + (size_t)m * row_floats, L, log2L, tid, nthreads);
        __syncthreads();
    }
    if (log2L > 15) {
        for (int m = 0; m < rows; ++m) fwht_pass_from<15>(images + (size_t)m * row_floats, L, log2L, tid, nthreads);
        __syncthreads();
    }
}

// One fp16 row of L = 2^log2L values (L >= 8) -> its unscaled transform as a padded fp32 image in
// LDS (L + L/16 floats), by all `nthreads` threads of the workgroup together: 16-byte loads, index
// bits 0..2 in registers, then LDS passes of up to four bits, lowest bit first.  Ends with a
// workgroup barrier; every thread of the workgroup must call it.
__device__ __forceinline__ void fwht_row_to_lds(const u32x4* xp, float* fbuf, int L, int log2L, int tid, int nthreads) {
    const int chunks = L >> 3;
    for (int c = tid; c < chunks; c += nthreads) {
        const u32x4 v = xp[c];
        float f[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const h2 hv = bits_to_h2(v[p]);
            f[2 * p] = (float)hv.x;
            f[2 * p + 1] = (float)hv.y;
        }
#pragma unroll
        for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if ((i & h) == 0) {
                    const float p = f[i], q = f[i + h];
                    f[i] = p + q;
                    f[i + h] = p - q;
                }
            }
        }
        float* dst = fbuf + fwht_pad(8 * c);
        *reinterpret_cast<f4*>(dst) = f4{f[0], f[1], f[2], f[3]};
        *reinterpret_cast<f4*>(dst + 4) = f4{f[4], f[5], f[6], f[7]};
    }
    __syncthreads();
    fwht_passes_from_bit3(fbuf, 1, 0, L, log2L, tid, nthreads);
}

// ---- M rows at once, for a caller that has other memory requests to place between the loads and
// the first use of their data.  fwht_rows_load fetches the chunks (16 bytes) tid, tid + nthreads,
// ... of the M K / 8 chunks of all rows (at most MAXC per thread); fwht_rows_to_lds finishes the
// transforms into fp32 images of K + K/32 floats per row: eight floats of padding per 256, which
// keeps passes of FIVE index bits free of bank conflicts (a wave's 64 lanes differ in three low
// bits and, 256 + 8 floats apart, in three high ones), so K = 8192 takes two LDS passes after the
// three bits done in registers.  One barrier per pass for all rows together.
__device__ __forceinline__ int fwht_pad256(int idx) { return idx + ((idx >> 8) << 3); }

template <int CNT, int LO>
__device__ __forceinline__ void fwht_pass256(float* buf, int L, int tid, int nthreads) {
    constexpr int E = 1 << CNT;
    const int tasks = L >> CNT;
    constexpr int lowmask = (1 << LO) - 1;
    for (int t = tid; t < tasks; t += nthreads) {
        // the task's values lie (i << LO) apart; those bits of the first index are zero, so the
        // padding term of value i is that of the first index plus a constant
        float* p0 = buf + fwht_pad256(((t >> LO) << (LO + CNT)) | (t & lowmask));
        float v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) v[i] = p0[(i << LO) + (((i << LO) >> 8) << 3)];
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
        for (int i = 0; i < E; ++i) p0[(i << LO) + (((i << LO) >> 8) << 3)] = v[i];
    }
}

template <int MAXC>
__device__ __forceinline__ void fwht_rows_load(const half_t* X, int64_t ldx, int M, int log2K, int tid, int nthreads,
                                               u32x4 (&xin)[MAXC]) {
    const int per_row = 1 << (log2K - 3), total = M << (log2K - 3);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * nthreads;
        xin[i] = u32x4{0u, 0u, 0u, 0u};
        if (c < total)
            xin[i] = *reinterpret_cast<const u32x4*>(X + (size_t)(c >> (log2K - 3)) * ldx + 8 * (c & (per_row - 1)));
    }
}

__device__ __forceinline__ int fwht_rows_image_floats(int K) { return K + (K >> 5); }

// 256 <= K <= 32768
template <int MAXC>
__device__ __forceinline__ void fwht_rows_to_lds(const u32x4 (&xin)[MAXC], float* images, int M, int K, int log2K,
                                                 int tid, int nthreads) {
    const int per_row = 1 << (log2K - 3), total = M << (log2K - 3);
    const int row_floats = fwht_rows_image_floats(K);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * nthreads;
        if (c < total) {
            float f[8];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const h2 hv = bits_to_h2(xin[i][p]);
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
            float* dst = images + (size_t)(c >> (log2K - 3)) * row_floats + fwht_pad256(8 * (c & (per_row - 1)));
            *reinterpret_cast<f4*>(dst) = f4{f[0], f[1], f[2], f[3]};
            *reinterpret_cast<f4*>(dst + 4) = f4{f[4], f[5], f[6], f[7]};
        }
    }
    __syncthreads();
    // index bits 3 .. log2K - 1 in passes of at most five bits
#define UNIQL_FWHT_PASS(CNT_, LO_)                                                                         \
    do {                                                                                                   \
        for (int m = 0; m < M; ++m) fwht_pass256<CNT_, LO_>(images + (size_t)m * row_floats, K, tid, nthreads); \
        __syncthreads();                                                                                   \
    } while (0)
    switch (log2K) {
        case 8: UNIQL_FWHT_PASS(5, 3); break;
        case 9: UNIQL_FWHT_PASS(3, 3); UNIQL_FWHT_PASS(3, 6); break;
        case 10: UNIQL_FWHT_PASS(4, 3); UNIQL_FWHT_PASS(3, 7); break;
        case 11: UNIQL_FWHT_PASS(4, 3); UNIQL_FWHT_PASS(4, 7); break;
        case 12: UNIQL_FWHT_PASS(5, 3); UNIQL_FWHT_PASS(4, 8); break;
        case 13: UNIQL_FWHT_PASS(5, 3); UNIQL_FWHT_PASS(5, 8); break;
        case 14: UNIQL_FWHT_PASS(4, 3); UNIQL_FWHT_PASS(4, 7); UNIQL_FWHT_PASS(3, 11); break;
        case 15: UNIQL_FWHT_PASS(4, 3); UNIQL_FWHT_PASS(4, 7); UNIQL_FWHT_PASS(4, 11); break;
        default: break;
    }
#undef UNIQL_FWHT_PASS
}

}  // namespace uniql
