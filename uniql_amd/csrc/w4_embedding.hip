// int4 embedding gather: out[t, :] = fp16((code - 8) * scale[id_t]).
//
// A wavefront expands 256 consecutive packed words (2048 codes) of one table row: every lane
// takes four words 64 apart, so each of its four loads reads 256 contiguous bytes per wave
// and each of its four 16-byte stores writes 1 KiB of contiguous fp16.  The packer's nibble
// interleave [0,2,4,6,1,3,5,7] is exactly what the pairwise conversion undoes, so the four
// converted pairs of a word come out in natural element order.
#include "common.hpp"

namespace uniql {

constexpr int kEmbWordsPerWave = 256;

__global__ __launch_bounds__(256) void w4_embedding_kernel(const int64_t* __restrict__ ids,
                                                          const uint32_t* __restrict__ table,
                                                          const half_t* __restrict__ scales,
                                                          u32x4* __restrict__ out, int64_t ntokens,
                                                          int64_t vocab, int words /* dim / 8 */,
                                                          int chunks /* ceil(words / 256) */) {
    const int lane = threadIdx.x & 63;
    // The wave's number is uniform by construction; saying so makes everything derived from it
    // scalar, so the token's id and its scale, the first two of the three dependent loads in
    // front of the stores, come through the scalar cache (a quarter of the launch's time).
    const int64_t wave = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave >= ntokens * chunks) return;
    const int64_t t = wave / chunks;
    const int w0 = (int)(wave - t * chunks) * kEmbWordsPerWave + lane;
    // the reference narrows the id to a 32-bit int (quant_embedding_kernel.cuh:97)
    const int64_t id = (int64_t)(int)ids[t];
    const bool valid = id >= 0 && id < vocab;  // ids outside the table produce zeros instead of a wild read
    uint32_t q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int wd = w0 + 64 * j;
        q[j] = (valid && wd < words) ? __builtin_nontemporal_load(table + id * words + wd) : 0u;
    }
    // Scalar loads have no 16-bit form: the aligned 32-bit word that holds the scale is read where
    // that word lies inside the array (a 4-byte aligned `scales`; not the last entry of an odd-sized
    // table, whose word would end two bytes behind it), the 16 bits themselves otherwise.
    uint32_t scale_bits = 0u;
    if (valid) {  // uniform
        const bool word_ok = (reinterpret_cast<uintptr_t>(scales) & 3u) == 0 && ((id & 1) || id + 1 < vocab);
        if (word_ok) {
            const uint32_t scale_word = reinterpret_cast<const uint32_t*>(scales)[id >> 1];
            scale_bits = (id & 1) ? (scale_word >> 16) : (scale_word & 0xffffu);
        } else {
            scale_bits = reinterpret_cast<const uint16_t*>(scales)[id];
        }
    }
    const h2 sv = bits_to_h2(scale_bits | (scale_bits << 16));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int wd = w0 + 64 * j;
        if (wd < words) {
            u32x4 o = u32x4{0u, 0u, 0u, 0u};
            if (valid) {
                o[0] = h2_to_bits(code_pair_low(q[j]) * sv);
                o[1] = h2_to_bits(code_pair_high(q[j]) * sv);
                o[2] = h2_to_bits(code_pair_low(q[j] >> 8) * sv);
                o[3] = h2_to_bits(code_pair_high(q[j] >> 8) * sv);
            }
            __builtin_nontemporal_store(o, out + t * words + wd);
        }
    }
}

// Producer side: one workgroup quantises one table row.  scale = fp16(max|w| / 8),
// code = clamp(round(fp16(fp16(w / scale) + 8)), 0, 15): every operation rounded to fp16 as
// the tensor expression of the reference does on an fp16 table
// (quantize/quant_embedding_layers.py:35-37).  An all-zero row divides 0 by 0: the NaN
// becomes code 0 (the reference's NaN -> int32 -> uint32 conversion leaves the low nibble 0).
// Element 2 p + odd of every eight goes to nibble 4 odd + p of the word (:33,39-43).
__global__ __launch_bounds__(256) void w4_embedding_quantize_kernel(const half_t* __restrict__ W, int64_t ldw,
                                                                   uint32_t* __restrict__ packed,
                                                                   half_t* __restrict__ scales, int words) {
    __shared__ float wave_max[4];
    const int64_t row = blockIdx.x;
    const half_t* src = W + row * ldw;
    float amax = 0.f;
    for (int w = threadIdx.x; w < words; w += 256) {
        const h8 v = *reinterpret_cast<const h8*>(src + 8 * w);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float f = fabsf((float)v[i]);
            amax = (f > amax || f != f) ? f : amax;  // a NaN in the row makes the scale NaN, as amax() does
        }
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const float o = __shfl_xor(amax, d, kWave);
        amax = (o > amax || o != o) ? o : amax;
    }
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float o = wave_max[i];
        amax = (o > amax || o != o) ? o : amax;
    }
    const half_t scale = (half_t)(amax / 8.0f);
    if (threadIdx.x == 0) scales[row] = scale;
    for (int w = threadIdx.x; w < words; w += 256) {
        const h8 v = *reinterpret_cast<const h8*>(src + 8 * w);
        uint32_t word = 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const half_t q = (half_t)((float)v[i] / (float)scale);
            const half_t shifted = (half_t)((float)q + 8.0f);
            const float r = __builtin_rintf((float)shifted);
            const uint32_t code = (uint32_t)fminf(fmaxf(r, 0.0f), 15.0f);  // fmaxf(NaN, 0) = 0
            word |= code << (4 * (4 * (i & 1) + (i >> 1)));
        }
        packed[row * words + w] = word;
    }
}

int embedding_quantize_launch(const void* W, int64_t ldw, void* packed, void* scales, int64_t vocab, int dim,
                              hipStream_t stream) {
    if (vocab == 0) return UNIQL_OK;
    if (vocab > 0x7fffffffLL) return UNIQL_E_SHAPE;
    hipLaunchKernelGGL(w4_embedding_quantize_kernel, dim3((unsigned)vocab), dim3(256), 0, stream,
                       reinterpret_cast<const half_t*>(W), ldw, reinterpret_cast<uint32_t*>(packed),
                       reinterpret_cast<half_t*>(scales), dim / 8);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

int embedding_launch(const int64_t* ids, int64_t ntokens, const void* weight, const void* scales, void* out,
                     int64_t vocab, int dim, hipStream_t stream) {
    if (ntokens == 0) return UNIQL_OK;
    const int words = dim / 8;
    const int chunks = (words + kEmbWordsPerWave - 1) / kEmbWordsPerWave;
    const int64_t grid = (ntokens * chunks + 3) / 4;
    if (grid > 0x7fffffffLL) return UNIQL_E_SHAPE;
    hipLaunchKernelGGL(w4_embedding_kernel, dim3((unsigned)grid), dim3(256), 0, stream, ids,
                       reinterpret_cast<const uint32_t*>(weight), reinterpret_cast<const half_t*>(scales),
                       reinterpret_cast<u32x4*>(out), ntokens, vocab, words, chunks);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
