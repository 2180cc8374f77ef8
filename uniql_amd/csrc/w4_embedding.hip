// int4 embedding gather: out[t, :] = fp16((code - 8) * scale[id_t]).
//
// One lane per packed 32-bit word (8 codes): a wave reads 256 contiguous bytes of
// the table row and writes 1 KiB of contiguous fp16 with 16-byte stores.  The
// packer's nibble interleave [0,2,4,6,1,3,5,7] is exactly what the pairwise
// conversion undoes, so the four converted pairs come out in natural element order.
#include "common.hpp"

namespace uniql {

__global__ __launch_bounds__(256) void w4_embedding_kernel(const int64_t* __restrict__ ids,
                                                          const uint32_t* __restrict__ table,
                                                          const half_t* __restrict__ scales,
                                                          u32x4* __restrict__ out, int64_t ntokens,
                                                          int64_t vocab, int words /* dim / 8 */) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= ntokens * words) return;
    const int64_t t = idx / words;
    const int wd = (int)(idx - t * words);
    // the reference narrows the id to a 32-bit int (quant_embedding_kernel.cuh:97)
    const int64_t id = (int64_t)(int)ids[t];
    u32x4 o = u32x4{0u, 0u, 0u, 0u};
    if (id >= 0 && id < vocab) {  // ids outside the table produce zeros instead of a wild read
        const uint32_t q = __builtin_nontemporal_load(table + id * words + wd);
        const half_t s = scales[id];
        const h2 sv = h2{s, s};
        o[0] = h2_to_bits(code_pair_low(q) * sv);
        o[1] = h2_to_bits(code_pair_high(q) * sv);
        o[2] = h2_to_bits(code_pair_low(q >> 8) * sv);
        o[3] = h2_to_bits(code_pair_high(q >> 8) * sv);
    }
    __builtin_nontemporal_store(o, out + idx);
}

int embedding_launch(const int64_t* ids, int64_t ntokens, const void* weight, const void* scales, void* out,
                     int64_t vocab, int dim, hipStream_t stream) {
    if (ntokens == 0) return UNIQL_OK;
    const int words = dim / 8;
    const int64_t total = ntokens * words;
    const int64_t grid = (total + 255) / 256;
    if (grid > 0x7fffffffLL) return UNIQL_E_SHAPE;
    hipLaunchKernelGGL(w4_embedding_kernel, dim3((unsigned)grid), dim3(256), 0, stream, ids,
                       reinterpret_cast<const uint32_t*>(weight), reinterpret_cast<const half_t*>(scales),
                       reinterpret_cast<u32x4*>(out), ntokens, vocab, words);
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
