// Rotary position embedding with per-head gathered frequencies, in place on the projections'
// outputs.  Attention heads pruned to fewer than the original head_dim columns keep, per
// key/value head, the list of the original columns they retained; column j of such a head is
// rotated with the frequency of original column indices[head][j].
//
// One thread rotates up to eight neighbouring column pairs (j, j + d/2) of one head of one token
// with 16-byte loads and stores (4- or 2-byte ones when the head width does not allow more),
// consecutive lanes on consecutive columns.  Every value is read once and written once; cos /
// sin rows are shared by all heads of a token and stay in cache.
//
// Arithmetic: out = x * cos_g + rotate_half(x) * sin_g with both products and the sum rounded to
// fp16 one after the other, which is what the tensor expression of the reference computes on
// fp16 tensors.
#include "common.hpp"

namespace uniql {

struct RopeArgs {
    half_t* q;
    half_t* k;
    const half_t* cos;
    const half_t* sin;
    const void* indices;  // [n_kh][hd], index_bytes wide
    int64_t q_row_stride, k_row_stride, cos_row_stride;
    int seq_len, cos_batch, n_qh, n_kh, hd, index_bytes;
};

__device__ __forceinline__ int load_index(const void* base, int index_bytes, int pos) {
    if (index_bytes == 1) return (int)reinterpret_cast<const uint8_t*>(base)[pos];
    if (index_bytes == 4) return reinterpret_cast<const int32_t*>(base)[pos];
    return (int)reinterpret_cast<const int64_t*>(base)[pos];
}

// one column pair: (lo, hi) = (x[j], x[j + d/2]) with their own table columns
__device__ __forceinline__ void rotate_pair(half_t& lo, half_t& hi, half_t c_lo, half_t s_lo, half_t c_hi,
                                            half_t s_hi) {
    // no fused multiply-add: the reference rounds each product before the sum
#pragma clang fp contract(off)
    const float x1 = (float)lo, x2 = (float)hi;
    const half_t a_lo = (half_t)(x1 * (float)c_lo), r_lo = (half_t)(-x2 * (float)s_lo);
    const half_t a_hi = (half_t)(x2 * (float)c_hi), r_hi = (half_t)(x1 * (float)s_hi);
    lo = (half_t)((float)a_lo + (float)r_lo);
    hi = (half_t)((float)a_hi + (float)r_hi);
}

template <int VEC>
struct HalfVec;  // VEC fp16 values moved with one access
template <>
struct HalfVec<8> { typedef h8 type; };
template <>
struct HalfVec<2> { typedef h2 type; };
template <>
struct HalfVec<1> { typedef half_t type; };

// VEC columns per thread and half of the head: 8 (16-byte accesses), 2 or 1.  A block covers
// 256 consecutive work items of one token, so the only divisions are 32-bit ones.
template <int VEC>
__global__ __launch_bounds__(256) void rope_indices_kernel(const RopeArgs a) {
    typedef typename HalfVec<VEC>::type vec_t;
    const int half = a.hd >> 1;
    const int per_head = half / VEC;
    const int per_row = (a.n_qh + a.n_kh) * per_head;
    const int blocks_per_row = (per_row + 255) >> 8;
    const int64_t row = blockIdx.x / blocks_per_row;
    const int t = (int)(blockIdx.x % blocks_per_row) * 256 + threadIdx.x;
    if (t >= per_row) return;
    const int head = t / per_head;
    const int j = (t - head * per_head) * VEC;

    const bool is_q = head < a.n_qh;
    const int kv_head = is_q ? head / (a.n_qh / a.n_kh) : head - a.n_qh;
    half_t* x = is_q ? a.q + row * a.q_row_stride + (int64_t)head * a.hd
                     : a.k + row * a.k_row_stride + (int64_t)(head - a.n_qh) * a.hd;
    const int64_t table_row = a.cos_batch == 1 ? row % a.seq_len : row;
    const half_t* cos_row = a.cos + table_row * a.cos_row_stride;
    const half_t* sin_row = a.sin + table_row * a.cos_row_stride;

    vec_t lo_v = *reinterpret_cast<const vec_t*>(x + j), hi_v = *reinterpret_cast<const vec_t*>(x + half + j);
    half_t lo[VEC], hi[VEC];
    if constexpr (VEC == 1) {
        lo[0] = lo_v;
        hi[0] = hi_v;
    } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            lo[v] = lo_v[v];
            hi[v] = hi_v[v];
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const int i_lo = load_index(a.indices, a.index_bytes, kv_head * a.hd + j + v);
        const int i_hi = load_index(a.indices, a.index_bytes, kv_head * a.hd + half + j + v);
        rotate_pair(lo[v], hi[v], cos_row[i_lo], sin_row[i_lo], cos_row[i_hi], sin_row[i_hi]);
    }
    if constexpr (VEC == 1) {
        lo_v = lo[0];
        hi_v = hi[0];
    } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            lo_v[v] = lo[v];
            hi_v[v] = hi[v];
        }
    }
    *reinterpret_cast<vec_t*>(x + j) = lo_v;
    *reinterpret_cast<vec_t*>(x + half + j) = hi_v;
}

// Many tokens: one workgroup per token builds the token's gathered (cos, sin) pairs once per
// key/value head in LDS (n_kv_heads x head_dim entries of 4 bytes) and every query head of the
// group reads them from there, instead of every element gathering from the tables in memory.
template <int VEC>
__global__ __launch_bounds__(256) void rope_indices_lds_kernel(const RopeArgs a, int cos_dim) {
    typedef typename HalfVec<VEC>::type vec_t;
    extern __shared__ __attribute__((aligned(16))) uint32_t rope_lds[];
    uint16_t* trow = reinterpret_cast<uint16_t*>(rope_lds);  // the token's cos row, then its sin row
    // gathered tables: entry (kv head, column) of the cosines, then the same of the sines, as fp16
    uint16_t* tab_cos = reinterpret_cast<uint16_t*>(rope_lds + ((cos_dim + 3) & ~3));
    uint16_t* tab_sin = tab_cos + a.n_kh * a.hd;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t table_row = a.cos_batch == 1 ? row % a.seq_len : row;
    const uint16_t* cos_row = reinterpret_cast<const uint16_t*>(a.cos + table_row * a.cos_row_stride);
    const uint16_t* sin_row = reinterpret_cast<const uint16_t*>(a.sin + table_row * a.cos_row_stride);
    // Everything the token needs from memory is requested before the first barrier: the (cos, sin)
    // row, the thread's first four index entries and its first two work items' q / k values are three
    // independent loads, and issued one behind a barrier behind the other they would cost three
    // memory round trips in a launch that lasts little longer than that.
    const int entries = a.n_kh * a.hd;
    const int half = a.hd >> 1;
    const int per_head = half / VEC;
    const int per_row = (a.n_qh + a.n_kh) * per_head;
    constexpr int kIdxAhead = 4;
    int idx_ahead[kIdxAhead];
#pragma unroll
    for (int i = 0; i < kIdxAhead; ++i) {
        const int e = tid + 256 * i;
        idx_ahead[i] = e < entries ? load_index(a.indices, a.index_bytes, e) : 0;
    }
    auto item = [&](int t, half_t*& x, int& kv_head, int& j) __attribute__((always_inline)) {
        const int head = t / per_head;
        j = (t - head * per_head) * VEC;
        const bool is_q = head < a.n_qh;
        kv_head = is_q ? head / (a.n_qh / a.n_kh) : head - a.n_qh;
        x = is_q ? a.q + row * a.q_row_stride + (int64_t)head * a.hd
                 : a.k + row * a.k_row_stride + (int64_t)(head - a.n_qh) * a.hd;
    };
    constexpr int kItemsAhead = 2;  // 32 + 8 heads of 128 are 320 work items of eight column pairs: two per thread at most
    half_t* x0[kItemsAhead];
    int kv0[kItemsAhead], j0[kItemsAhead];
    vec_t lo0[kItemsAhead], hi0[kItemsAhead];
#pragma unroll
    for (int i = 0; i < kItemsAhead; ++i) {
        x0[i] = nullptr;
        kv0[i] = j0[i] = 0;
        lo0[i] = hi0[i] = vec_t();
        if (tid + 256 * i < per_row) {
            item(tid + 256 * i, x0[i], kv0[i], j0[i]);
            lo0[i] = *reinterpret_cast<const vec_t*>(x0[i] + j0[i]);
            hi0[i] = *reinterpret_cast<const vec_t*>(x0[i] + half + j0[i]);
        }
    }
    for (int i = tid; i < cos_dim; i += 256) {
        trow[i] = cos_row[i];
        trow[cos_dim + i] = sin_row[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kIdxAhead; ++i) {
        const int e = tid + 256 * i;
        if (e < entries) {
            tab_cos[e] = trow[idx_ahead[i]];
            tab_sin[e] = trow[cos_dim + idx_ahead[i]];
        }
    }
    for (int e = tid + 256 * kIdxAhead; e < entries; e += 256) {
        const int i = load_index(a.indices, a.index_bytes, e);
        tab_cos[e] = trow[i];
        tab_sin[e] = trow[cos_dim + i];
    }
    __syncthreads();
    auto rotate_item = [&](half_t* x, int kv_head, int j, vec_t lo_v, vec_t hi_v) __attribute__((always_inline)) {
        const int e0 = kv_head * a.hd + j;
        if constexpr (VEC > 1) {
            // All of the item's column pairs at once in packed fp16 arithmetic.  An fp16 product or sum
            // computed in fp32 and rounded to fp16 equals the fp16 operation's own single rounding
            // (fp32's 24 bits are at least 2 x 11 + 2), so these are the values of rotate_pair bit for
            // bit, at a fifth of its instructions: the conversions made this kernel compute-bound.
#pragma clang fp contract(off)
            const vec_t c_lo = *reinterpret_cast<const vec_t*>(tab_cos + e0), s_lo = *reinterpret_cast<const vec_t*>(tab_sin + e0);
            const vec_t c_hi = *reinterpret_cast<const vec_t*>(tab_cos + e0 + half);
            const vec_t s_hi = *reinterpret_cast<const vec_t*>(tab_sin + e0 + half);
            const vec_t a_lo = lo_v * c_lo, r_lo = (-hi_v) * s_lo;
            const vec_t a_hi = hi_v * c_hi, r_hi = lo_v * s_hi;
            *reinterpret_cast<vec_t*>(x + j) = a_lo + r_lo;
            *reinterpret_cast<vec_t*>(x + half + j) = a_hi + r_hi;
        } else {
            half_t lo = lo_v, hi = hi_v;
            rotate_pair(lo, hi, __builtin_bit_cast(half_t, tab_cos[e0]), __builtin_bit_cast(half_t, tab_sin[e0]),
                        __builtin_bit_cast(half_t, tab_cos[e0 + half]), __builtin_bit_cast(half_t, tab_sin[e0 + half]));
            *reinterpret_cast<vec_t*>(x + j) = lo;
            *reinterpret_cast<vec_t*>(x + half + j) = hi;
        }
    };
#pragma unroll
    for (int i = 0; i < kItemsAhead; ++i)
        if (tid + 256 * i < per_row) rotate_item(x0[i], kv0[i], j0[i], lo0[i], hi0[i]);
    for (int t = tid + 256 * kItemsAhead; t < per_row; t += 256) {
        half_t* x;
        int kv_head, j;
        item(t, x, kv_head, j);
        const vec_t lo_v = *reinterpret_cast<const vec_t*>(x + j), hi_v = *reinterpret_cast<const vec_t*>(x + half + j);
        rotate_item(x, kv_head, j, lo_v, hi_v);
    }
}

int rope_indices_launch(void* q, int64_t q_row_stride, void* k, int64_t k_row_stride, const void* cos, const void* sin,
                        int64_t cos_row_stride, const void* indices, int index_bytes, int64_t rows, int seq_len,
                        int cos_batch, int n_qh, int n_kh, int hd, int cos_dim, hipStream_t stream) {
    RopeArgs a;
    a.q = reinterpret_cast<half_t*>(q);
    a.k = reinterpret_cast<half_t*>(k);
    a.cos = reinterpret_cast<const half_t*>(cos);
    a.sin = reinterpret_cast<const half_t*>(sin);
    a.indices = indices;
    a.q_row_stride = q_row_stride;
    a.k_row_stride = k_row_stride;
    a.cos_row_stride = cos_row_stride;
    a.seq_len = seq_len;
    a.cos_batch = cos_batch;
    a.n_qh = n_qh;
    a.n_kh = n_kh;
    a.hd = hd;
    a.index_bytes = index_bytes;
    if (rows == 0) return UNIQL_OK;
    const int half = hd / 2;
    // the widest access every offset (head start, half-head start, row start) is aligned for
    const uintptr_t bases = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k);
    int vec = 1;
    if (half % 8 == 0 && q_row_stride % 8 == 0 && k_row_stride % 8 == 0 && (bases & 15u) == 0) vec = 8;
    else if (half % 2 == 0 && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 && (bases & 3u) == 0) vec = 2;
    // enough tokens to fill the chip with one workgroup each, and tables that fit LDS
    const size_t lds_bytes = ((size_t)((cos_dim + 3) & ~3) + (size_t)n_kh * hd) * 4;
    if (rows >= 64 && lds_bytes <= 32 * 1024 && rows <= 0x7fffffffLL) {
        if (vec == 8)
            hipLaunchKernelGGL(rope_indices_lds_kernel<8>, dim3((unsigned)rows), dim3(256), lds_bytes, stream, a, cos_dim);
        else if (vec == 2)
            hipLaunchKernelGGL(rope_indices_lds_kernel<2>, dim3((unsigned)rows), dim3(256), lds_bytes, stream, a, cos_dim);
        else
            hipLaunchKernelGGL(rope_indices_lds_kernel<1>, dim3((unsigned)rows), dim3(256), lds_bytes, stream, a, cos_dim);
        return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
    }
    // few tokens: the direct gather, narrow accesses (more threads in flight hide the dependent
    // index -> table loads better than wide accesses do)
    if (vec == 8) vec = 2;
    const int per_row = (n_qh + n_kh) * (half / vec);
    const int64_t blocks = rows * ((per_row + 255) / 256);
    if (blocks > 0x7fffffffLL) return UNIQL_E_SHAPE;
    if (vec == 8)
        hipLaunchKernelGGL(rope_indices_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else if (vec == 2)
        hipLaunchKernelGGL(rope_indices_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL(rope_indices_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
