// Shared device helpers for the gfx950 W4A16 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "uniql_amd.h"

namespace uniql {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kGroup = 128;      // quantisation group along K
constexpr int kTileK = 16;       // K rows covered by one packed weight row
constexpr int kChunkN = 64;      // columns covered by 512 contiguous bytes of a packed row
constexpr int kWave = 64;

__device__ __forceinline__ h2 bits_to_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }
__device__ __forceinline__ uint32_t h2_to_bits(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// Two int4 codes -> two fp16 values (code - 8), exactly.
//   low form : codes sit in bits 0..3 and 16..19.  OR-ing 0x6400 into each half
//              makes the fp16 number 1024 + code; subtracting 1032 leaves code - 8.
//   high form: codes sit in bits 4..7 and 20..23, giving 1024 + 16*code;
//              (1024 + 16 c) / 16 - 72 = c - 8.  Every step is exact in fp16.
// The masks and the exponent pattern are kept in registers (not literals): gfx950's
// three-operand v_and_or_b32 cannot encode literals, and with literals the compiler
// falls back to a separate AND and OR.
struct NibbleMagic {
    uint32_t mask_low, mask_high, exponent;
    __device__ __forceinline__ void init() {
        mask_low = 0x000f000fu;
        mask_high = 0x00f000f0u;
        exponent = 0x64006400u;
        asm volatile("" : "+v"(mask_low), "+v"(mask_high));
        asm volatile("" : "+s"(exponent));
    }
    __device__ __forceinline__ h2 pair_low(uint32_t q) const {
        return bits_to_h2((q & mask_low) | exponent) - h2{(half_t)1032.0f, (half_t)1032.0f};
    }
    __device__ __forceinline__ h2 pair_high(uint32_t q) const {
        return bits_to_h2((q & mask_high) | exponent) * h2{(half_t)0.0625f, (half_t)0.0625f} -
               h2{(half_t)72.0f, (half_t)72.0f};
    }
};
__device__ __forceinline__ h2 code_pair_low(uint32_t q) {
    return bits_to_h2((q & 0x000f000fu) | 0x64006400u) - h2{(half_t)1032.0f, (half_t)1032.0f};
}
__device__ __forceinline__ h2 code_pair_high(uint32_t q) {
    return bits_to_h2((q & 0x00f000f0u) | 0x64006400u) * h2{(half_t)0.0625f, (half_t)0.0625f}
           - h2{(half_t)72.0f, (half_t)72.0f};
}

// fp16(v * s) with two roundings (fp32 product, then fp16), the result a separate
// multiply and conversion give.  Written as one expression the compiler selects
// v_fma_mixlo_f16, which rounds the exact product once and differs in rare cases; the
// empty asm keeps the product a plain fp32 value so that every kernel (and the
// fp32 host model of the transform) rounds the same way.
__device__ __forceinline__ half_t scaled_to_half(float v, float s) {
    float p = v * s;
    asm volatile("" : "+v"(p));
    return (half_t)p;
}

// Where each lane's eight scale values sit for a 16-byte load, grouped case:
// inside every 64-column block position 8*i + j holds column i + 8*j, so the 8
// fp16 at offset 8*col8 are the columns col8 + 8*jb, jb = 0..7.
//
// Per-column case (one scale row): inside every 32-column block position
// 8*i + jj holds column 2*i + {0,1,8,9,16,17,24,25}[jj].
__device__ __forceinline__ int single_scale_pos(int n) {
    const int blk = n & ~31, c = n & 31;
    return blk + 8 * ((c & 7) >> 1) + 2 * (c >> 3) + (c & 1);
}

// Butterflies of a 128-point Walsh-Hadamard transform on a row spread over 16
// consecutive lanes, 8 consecutive elements per lane (element e = 8*seg + i).
// In-lane stages handle index bits 0..2, lane exchanges handle bits 3..6.
__device__ __forceinline__ void wht128_row16(float (&v)[8], int seg) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((i & h) == 0) {
                const float a = v[i], b = v[i + h];
                v[i] = a + b;
                v[i + h] = a - b;
            }
        }
    }
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
        const bool upper = (seg & d) != 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float other = __shfl_xor(v[i], d, kWave);
            v[i] = upper ? (other - v[i]) : (v[i] + other);
        }
    }
}

}  // namespace uniql
