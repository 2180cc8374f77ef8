// Rotary position embedding with per-head gathered frequencies, in place on the projections'
// outputs.  Attention heads pruned to fewer than the original head_dim columns keep, per
// key/value head, the list of the original columns they retained; column j of such a head is
// rotated with the frequency of original column indices[head][j].
//
// One thread rotates two neighbouring column pairs (j, j + d/2), (j+1, j+1 + d/2) of one head of
// one token: 4-byte loads and stores, consecutive lanes on consecutive columns.  Every value is
// read once and written once; cos / sin rows are shared by all heads of a token and stay in cache.
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
    int64_t work;         // rows * (n_qh + n_kh) * (hd / 2 / VEC)
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

template <int VEC>  // columns per thread and half: 2 (4-byte accesses) or 1
__global__ __launch_bounds__(256) void rope_indices_kernel(const RopeArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= a.work) return;
    const int half = a.hd >> 1;
    const int per_head = half / VEC;
    const int heads = a.n_qh + a.n_kh;
    const int j = (int)(idx % per_head) * VEC;
    const int head = (int)((idx / per_head) % heads);
    const int64_t row = idx / ((int64_t)per_head * heads);

    const bool is_q = head < a.n_qh;
    const int kv_head = is_q ? head / (a.n_qh / a.n_kh) : head - a.n_qh;
    half_t* x = is_q ? a.q + row * a.q_row_stride + (int64_t)head * a.hd
                     : a.k + row * a.k_row_stride + (int64_t)(head - a.n_qh) * a.hd;
    const int64_t table_row = a.cos_batch == 1 ? row % a.seq_len : row;
    const half_t* cos_row = a.cos + table_row * a.cos_row_stride;
    const half_t* sin_row = a.sin + table_row * a.cos_row_stride;

    half_t lo[VEC], hi[VEC];
    if (VEC == 2) {
        const h2 l = *reinterpret_cast<const h2*>(x + j), h = *reinterpret_cast<const h2*>(x + half + j);
        lo[0] = l.x;
        lo[VEC - 1] = l.y;
        hi[0] = h.x;
        hi[VEC - 1] = h.y;
    } else {
        lo[0] = x[j];
        hi[0] = x[half + j];
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const int i_lo = load_index(a.indices, a.index_bytes, kv_head * a.hd + j + v);
        const int i_hi = load_index(a.indices, a.index_bytes, kv_head * a.hd + half + j + v);
        rotate_pair(lo[v], hi[v], cos_row[i_lo], sin_row[i_lo], cos_row[i_hi], sin_row[i_hi]);
    }
    if (VEC == 2) {
        *reinterpret_cast<h2*>(x + j) = h2{lo[0], lo[VEC - 1]};
        *reinterpret_cast<h2*>(x + half + j) = h2{hi[0], hi[VEC - 1]};
    } else {
        x[j] = lo[0];
        x[half + j] = hi[0];
    }
}

int rope_indices_launch(void* q, int64_t q_row_stride, void* k, int64_t k_row_stride, const void* cos, const void* sin,
                        int64_t cos_row_stride, const void* indices, int index_bytes, int64_t rows, int seq_len,
                        int cos_batch, int n_qh, int n_kh, int hd, hipStream_t stream) {
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
    const int half = hd / 2;
    // 4-byte accesses need even offsets everywhere
    const bool vec2 = half % 2 == 0 && q_row_stride % 2 == 0 && k_row_stride % 2 == 0 &&
                      (reinterpret_cast<uintptr_t>(q) & 3u) == 0 && (reinterpret_cast<uintptr_t>(k) & 3u) == 0;
    const int vec = vec2 ? 2 : 1;
    a.work = rows * (int64_t)(n_qh + n_kh) * (half / vec);
    if (a.work == 0) return UNIQL_OK;
    const int64_t blocks = (a.work + 255) / 256;
    if (blocks > 0x7fffffffLL) return UNIQL_E_SHAPE;
    if (vec2)
        hipLaunchKernelGGL(rope_indices_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    else
        hipLaunchKernelGGL(rope_indices_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
