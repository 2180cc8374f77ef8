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

// ---- what happens to a finished output element --------------------------------------
// The reference's layer rounds the product to fp16, drops the padding columns, then adds the
// fp16 bias (second rounding); its MLP applies SiLU to the fp16 gate output (third rounding)
// and multiplies by the fp16 up output (fourth); its decoder layer adds the layer's fp16 output
// to the fp16 residual stream (one more rounding).  The same roundings are made here, in
// registers, so that the fused result equals the unfused sequence.
struct Epilogue {
    const half_t* bias;  // natural order [n_store] (gated: gate biases, then up biases), or nullptr
    const half_t* residual;  // [M][ldr], added to the rounded (and biased) product, or nullptr
    int64_t ldr;
    int64_t ldd;         // elements between output rows
    int n_store;         // output columns that exist; columns from here on are dropped
    int gated;           // 1: columns c and c + 64 of a 128-column strip are the gate and up values
                         //    of output column 64 strip + c; the output is silu(gate) * up
    int out_f32;         // D is float32 and receives the values before any rounding
    int vec_ok;          // ldd and D allow 16-byte stores of eight fp16 outputs
    int transpose;       // 1: D is [n_store][ldd] with the row index running along the inner axis
                         //    (the reference's output_transpose, "sequence length last")
    int relu2;           // 1: the stored value is relu(y)^2 of the rounded (and biased) product y

    __device__ __forceinline__ size_t offset(int m, int n) const {
        return transpose ? (size_t)n * ldd + m : (size_t)m * ldd + n;
    }
};

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + expf(-x)); }

// value of output column n (< n_store) from its fp32 product, and of a gated pair
__device__ __forceinline__ half_t finish_half(const Epilogue& e, int m, int n, float v) {
    half_t y = (half_t)v;
    if (e.bias) y = (half_t)((float)y + (float)e.bias[n]);
    if (e.relu2) {  // torch.square(relu(y)) on the fp16 tensor: one rounding of the exact square
        const float r = (float)y > 0.f ? (float)y : 0.f;
        y = (half_t)(r * r);
    }
    if (e.residual) y = (half_t)((float)e.residual[(size_t)m * e.ldr + n] + (float)y);
    return y;
}
__device__ __forceinline__ half_t finish_half_gated(const Epilogue& e, int n, float g, float u) {
    half_t g16 = (half_t)g;
    if (e.bias) g16 = (half_t)((float)g16 + (float)e.bias[n]);
    half_t u16 = (half_t)u;
    if (e.bias) u16 = (half_t)((float)u16 + (float)e.bias[e.n_store + n]);
    const half_t a16 = (half_t)silu_f32((float)g16);
    return (half_t)((float)a16 * (float)u16);
}

__device__ __forceinline__ void finish_store(const Epilogue& e, void* D, int m, int n, float v) {
    if (n >= e.n_store) return;
    const size_t o = e.offset(m, n);
    if (e.out_f32) {
        if (e.bias) v += (float)e.bias[n];
        if (e.relu2) v = v > 0.f ? v * v : 0.f;
        if (e.residual) v += (float)e.residual[(size_t)m * e.ldr + n];
        reinterpret_cast<float*>(D)[o] = v;
    } else {
        reinterpret_cast<half_t*>(D)[o] = finish_half(e, m, n, v);
    }
}

__device__ __forceinline__ void finish_store_gated(const Epilogue& e, void* D, int m, int n, float g, float u) {
    if (n >= e.n_store) return;
    const size_t o = e.offset(m, n);
    if (e.out_f32) {
        if (e.bias) {
            g += (float)e.bias[n];
            u += (float)e.bias[e.n_store + n];
        }
        reinterpret_cast<float*>(D)[o] = silu_f32(g) * u;
    } else {
        reinterpret_cast<half_t*>(D)[o] = finish_half_gated(e, n, g, u);
    }
}

// Eight consecutive fp16 values from p: one 16-byte load where the address allows it.
__device__ __forceinline__ void load_eight(const half_t* p, bool aligned16, float (&out)[8]) {
    if (aligned16) {
        const h8 v = *reinterpret_cast<const h8*>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (float)v[i];
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (float)p[i];
    }
}

// Eight consecutive outputs of row m starting at column n0 (a multiple of 8): one 16-byte
// store where the output's layout allows it, element stores otherwise.  Bias and residual come as
// 16-byte loads where they are aligned; the roundings are those of finish_half / finish_half_gated.
__device__ __forceinline__ void store_eight(const Epilogue& e, void* D, int m, int n0, f4 lo, f4 hi) {
    if (e.vec_ok && n0 + 8 <= e.n_store) {
        const size_t o = (size_t)m * e.ldd + n0;
        if (e.out_f32 && !e.bias && !e.residual && !e.relu2) {
            float* d = reinterpret_cast<float*>(D) + o;
            *reinterpret_cast<f4*>(d) = lo;
            *reinterpret_cast<f4*>(d + 4) = hi;
            return;
        }
        if (!e.out_f32 && !e.bias && !e.residual && !e.relu2) {
            const h2 r0 = h2{(half_t)lo[0], (half_t)lo[1]}, r1 = h2{(half_t)lo[2], (half_t)lo[3]};
            const h2 r2 = h2{(half_t)hi[0], (half_t)hi[1]}, r3 = h2{(half_t)hi[2], (half_t)hi[3]};
            *reinterpret_cast<u32x4*>(reinterpret_cast<half_t*>(D) + o) =
                u32x4{h2_to_bits(r0), h2_to_bits(r1), h2_to_bits(r2), h2_to_bits(r3)};
            return;
        }
        if (!e.out_f32) {
            half_t r[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                r[i] = (half_t)lo[i];
                r[4 + i] = (half_t)hi[i];
            }
            if (e.bias) {
                float b[8];
                load_eight(e.bias + n0, (reinterpret_cast<uintptr_t>(e.bias) & 15u) == 0, b);
#pragma unroll
                for (int i = 0; i < 8; ++i) r[i] = (half_t)((float)r[i] + b[i]);
            }
            if (e.relu2) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float p = (float)r[i] > 0.f ? (float)r[i] : 0.f;
                    r[i] = (half_t)(p * p);
                }
            }
            if (e.residual) {
                float q[8];
                load_eight(e.residual + (size_t)m * e.ldr + n0,
                           (reinterpret_cast<uintptr_t>(e.residual) & 15u) == 0 && (e.ldr & 7) == 0, q);
#pragma unroll
                for (int i = 0; i < 8; ++i) r[i] = (half_t)(q[i] + (float)r[i]);
            }
            *reinterpret_cast<h8*>(reinterpret_cast<half_t*>(D) + o) = h8{r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7]};
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        finish_store(e, D, m, n0 + i, lo[i]);
        finish_store(e, D, m, n0 + 4 + i, hi[i]);
    }
}
__device__ __forceinline__ void store_eight_gated(const Epilogue& e, void* D, int m, int n0, f4 glo, f4 ghi, f4 ulo,
                                                  f4 uhi) {
    if (e.vec_ok && !e.out_f32 && n0 + 8 <= e.n_store) {
        half_t r[8], g16[8], u16[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            g16[i] = (half_t)glo[i];
            g16[4 + i] = (half_t)ghi[i];
            u16[i] = (half_t)ulo[i];
            u16[4 + i] = (half_t)uhi[i];
        }
        if (e.bias) {
            float bg[8], bu[8];
            const bool al = (reinterpret_cast<uintptr_t>(e.bias) & 15u) == 0;
            load_eight(e.bias + n0, al, bg);
            load_eight(e.bias + e.n_store + n0, al && (e.n_store & 7) == 0, bu);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                g16[i] = (half_t)((float)g16[i] + bg[i]);
                u16[i] = (half_t)((float)u16[i] + bu[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const half_t a16 = (half_t)silu_f32((float)g16[i]);
            r[i] = (half_t)((float)a16 * (float)u16[i]);
        }
        *reinterpret_cast<h8*>(reinterpret_cast<half_t*>(D) + (size_t)m * e.ldd + n0) =
            h8{r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7]};
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        finish_store_gated(e, D, m, n0 + i, glo[i], ulo[i]);
        finish_store_gated(e, D, m, n0 + 4 + i, ghi[i], uhi[i]);
    }
}

// ---- exchange of partial sums between workgroups that split K ------------------------
// One 64-bit word per output element in a zero-initialised buffer:
//   bits 14..63  the running sum in units of 2^-24 (two's complement, 50 bits),
//   bits  7..13  the number of contributions that were NaN,
//   bits  0..6   the number of contributions.
// Integer adds commute, so the total does not depend on arrival order.  A contribution is
// clamped to +-2^18 (beyond the fp16 range of the output, so an infinite partial sum still
// gives an infinite fp16 result) and at most 127 contributions meet in a word: the sum
// field cannot overflow into nothing, the counts cannot carry into the sum.  A NaN partial
// sum adds nothing to the sum and one to the NaN count; the total then reads as NaN, as it
// would without a K split.
constexpr float kAccumScale = 16777216.0f;  // 2^24 fixed-point units per 1.0
constexpr float kAccumClamp = 262144.0f;    // 2^18
constexpr int kAccumMaxSplits = 127;

__device__ __forceinline__ unsigned long long accum_word(float v, unsigned count) {
    const bool is_nan = v != v;
    const float c = is_nan ? 0.f : fminf(fmaxf(v, -kAccumClamp), kAccumClamp);
    return ((unsigned long long)__float2ll_rn(c * kAccumScale) << 14) + (is_nan ? 128u : 0u) + count;
}
__device__ __forceinline__ float accum_value(unsigned long long word) {
    const float v = (float)((long long)word >> 14) * (1.0f / kAccumScale);
    return (word & 0x3f80ull) ? __builtin_nanf("") : v;
}
// Adds one contribution.  True for the last of `splits` arrivals, which gets the total and
// must put the word back to zero (accum_reset) after using it.
__device__ __forceinline__ bool accum_add(unsigned long long* p, float v, int splits, float& total) {
    const unsigned long long word = accum_word(v, 1u);
    const unsigned long long old = __hip_atomic_fetch_add(p, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((int)(old & 0x7full) != splits - 1) return false;
    total = accum_value(old + word);
    return true;
}
__device__ __forceinline__ void accum_reset(unsigned long long* p) {
    __hip_atomic_store(p, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Gated pair: the up value is added first (its word carries no count); the gate word's add is
// issued only after the up add has returned, i.e. has been performed.  Whoever completes the
// gate word's count therefore finds every up contribution in place and takes it with an
// exchange, which also leaves that word zero.
__device__ __forceinline__ bool accum_add_pair(unsigned long long* pg, unsigned long long* pu, float g, float u,
                                               int splits, float& total_g, float& total_u) {
    const unsigned long long old_u =
        __hip_atomic_fetch_add(pu, accum_word(u, 0u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned long long word = accum_word(g, 1u);
    uint32_t lo = (uint32_t)word;
    const uint32_t returned = (uint32_t)old_u;
    asm volatile("" : "+v"(lo) : "v"(returned));  // the gate word now depends on the up add's return value
    word = (word & 0xffffffff00000000ull) | lo;
    const unsigned long long old = __hip_atomic_fetch_add(pg, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((int)(old & 0x7full) != splits - 1) return false;
    total_g = accum_value(old + word);
    total_u = accum_value(__hip_atomic_exchange(pu, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    return true;
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
