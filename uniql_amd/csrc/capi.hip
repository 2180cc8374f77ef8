// extern "C" surface: argument checks and dispatch.  Nothing here allocates,
// synchronises or throws.
#include "common.hpp"

namespace uniql {
int stream_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, void* accum, int m, int n,
                  int k, int groups, bool had128, float had_scale, bool out_f32, unsigned tune,
                  hipStream_t stream);
size_t stream_accum_bytes(int m, int n, int k);
int tile_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, void* accum, size_t accum_bytes,
                int m, int n, int k, int groups, bool out_f32, unsigned tune, hipStream_t stream);
size_t tile_accum_bytes(int m, int n, int k);
int dequant_launch(const void* B, const void* S, void* W, uint8_t* codes, int n, int k, int groups,
                   hipStream_t stream);
int embedding_launch(const int64_t* ids, int64_t ntokens, const void* weight, const void* scales, void* out,
                     int64_t vocab, int dim, hipStream_t stream);
int fwht_launch(const void* x, void* y, int64_t rows, int dim, int block, float scale, int dtype,
                hipStream_t stream);
int quantize_launch(const void* W, int64_t ldw, const void* given_scales, void* B, void* S, int out_features,
                    int in_features, int n_pad, int k_pad, hipStream_t stream);
int pack_launch(const uint8_t* codes, const void* scales, void* B, void* S, int n, int k, int n_pad, int k_pad,
                hipStream_t stream);
}  // namespace uniql

using namespace uniql;

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
static inline size_t round256(size_t v) { return (v + 255) & ~(size_t)255; }

static int check_linear_shape(int m, int n, int k, int groups) {
    if (m < 0 || n <= 0 || k <= 0) return UNIQL_E_SHAPE;
    if (n % 128 != 0 || k % 128 != 0) return UNIQL_E_SHAPE;
    if (!(groups == 1 || groups == k / 128)) return UNIQL_E_SHAPE;
    return UNIQL_OK;
}

extern "C" {

int uniql_abi_version(void) { return UNIQL_ABI_VERSION; }

const char* uniql_status_string(int code) {
    switch (code) {
        case UNIQL_OK: return "ok";
        case UNIQL_E_NULL: return "a required pointer is NULL";
        case UNIQL_E_SHAPE: return "sizes violate the packed layout (k % 128, n % 128, groups, dim, block)";
        case UNIQL_E_ALIGN: return "pointer or leading dimension not 16-byte aligned";
        case UNIQL_E_WORKSPACE: return "workspace, accum or temp buffer too small";
        case UNIQL_E_UNSUPPORTED: return "request not supported by this build";
        case UNIQL_E_LAUNCH: return "HIP runtime rejected the kernel launch";
        default: return "unknown status";
    }
}

// rows up to this many take the weight-streaming kernel, more take the tiled one
static constexpr int kStreamMaxM = 16;

size_t uniql_w4a16_gemm_accum_bytes(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0 || n % 128 != 0 || k % 128 != 0) return 0;
    // enough for either kernel, so that the forcing flags never need a bigger buffer
    const size_t a = stream_accum_bytes(m, n, k), b = tile_accum_bytes(m, n, k);
    return round256(a > b ? a : b);
}

size_t uniql_w4a16_gemm_temp_bytes(int m, int n, int k, int had_block) {
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    // rotated activations: every block width except the 128 fused into the streaming kernel,
    // and 128 too once the tiled kernel may take the call
    if (had_block != 0) return round256((size_t)m * k * sizeof(half_t));
    return 0;
}

int uniql_w4a16_gemm(const void* A, int64_t lda, const void* B, const void* S, void* D, const int32_t* workspace,
                     int64_t workspace_len, void* accum, size_t accum_bytes, void* temp, size_t temp_bytes, int m,
                     int n, int k, int groups, int had_block, float had_scale, unsigned flags, void* stream) {
    const int rc = check_linear_shape(m, n, k, groups);
    if (rc != UNIQL_OK) return rc;
    if (flags & UNIQL_F_TRANSPOSE_OUT) return UNIQL_E_UNSUPPORTED;
    if (m == 0) return UNIQL_OK;
    if (!A || !B || !S || !D) return UNIQL_E_NULL;
    if (lda < k || (lda % 8) != 0) return UNIQL_E_ALIGN;
    if (!aligned16(A) || !aligned16(B) || !aligned16(S) || !aligned16(D)) return UNIQL_E_ALIGN;
    if (workspace && workspace_len < n / 128) return UNIQL_E_WORKSPACE;
    if (had_block != 0 && (!is_pow2(had_block) || had_block < 2 || had_block > 32768 || k % had_block != 0))
        return UNIQL_E_SHAPE;
    const size_t need_accum = uniql_w4a16_gemm_accum_bytes(m, n, k);
    if (need_accum > 0 && (!accum || accum_bytes < need_accum)) return UNIQL_E_WORKSPACE;
    const size_t need_temp = uniql_w4a16_gemm_temp_bytes(m, n, k, had_block);
    if (need_temp > 0 && (!temp || temp_bytes < need_temp)) return UNIQL_E_WORKSPACE;
    if ((accum && !aligned16(accum)) || (temp && !aligned16(temp))) return UNIQL_E_ALIGN;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);

    bool use_stream = m <= kStreamMaxM;
    if (flags & UNIQL_F_FORCE_SKINNY) use_stream = true;
    if (flags & UNIQL_F_FORCE_TILED) use_stream = false;

    const void* Ain = A;
    int64_t ld = lda;
    const bool had128 = (had_block == 128) && use_stream;
    if (had_block != 0 && !had128) {
        // rotate into the temporary buffer, then run the plain product on it
        if (lda != k) {
            for (int r = 0; r < m; ++r) {
                const int e = fwht_launch(reinterpret_cast<const half_t*>(A) + (size_t)r * lda,
                                          reinterpret_cast<half_t*>(temp) + (size_t)r * k, 1, k, had_block, had_scale,
                                          UNIQL_DT_F16, st);
                if (e != UNIQL_OK) return e;
            }
        } else {
            const int e = fwht_launch(A, temp, m, k, had_block, had_scale, UNIQL_DT_F16, st);
            if (e != UNIQL_OK) return e;
        }
        Ain = temp;
        ld = k;
    }
    const unsigned tune = flags >> 8;  // tuning fields, see the header
    if (use_stream)
        return stream_launch(Ain, ld, B, S, D, accum, m, n, k, groups, had128, had_scale,
                             (flags & UNIQL_F_OUT_F32) != 0, tune, st);
    return tile_launch(Ain, ld, B, S, D, accum, accum_bytes, m, n, k, groups, (flags & UNIQL_F_OUT_F32) != 0, tune,
                       st);
}

int uniql_w4a16_dequant(const void* B, const void* S, void* W, uint8_t* codes, int n, int k, int groups,
                        void* stream) {
    const int rc = check_linear_shape(1, n, k, groups);
    if (rc != UNIQL_OK) return rc;
    if (!B || !S || (!W && !codes)) return UNIQL_E_NULL;
    if (!aligned16(B)) return UNIQL_E_ALIGN;
    return dequant_launch(B, S, W, codes, n, k, groups, reinterpret_cast<hipStream_t>(stream));
}

int uniql_w4a16_quantize(const void* W, int64_t ldw, const void* given_scales, void* B, void* S, int out_features,
                         int in_features, int n_pad, int k_pad, void* stream) {
    if (!W || !B || !S) return UNIQL_E_NULL;
    if (out_features <= 0 || in_features <= 0 || ldw < in_features) return UNIQL_E_SHAPE;
    if (k_pad != (in_features + 127) / 128 * 128 || n_pad < out_features || n_pad % 128 != 0) return UNIQL_E_SHAPE;
    if (in_features <= 128) return UNIQL_E_UNSUPPORTED;
    if ((int64_t)(k_pad / 16) * 2 * n_pad > 0x7fffffffLL * 256) return UNIQL_E_SHAPE;
    return quantize_launch(W, ldw, given_scales, B, S, out_features, in_features, n_pad, k_pad,
                           reinterpret_cast<hipStream_t>(stream));
}

int uniql_w4a16_pack(const uint8_t* codes, const void* scales, void* B, void* S, int n, int k, int n_pad,
                     void* stream) {
    if (!codes || !scales || !B || !S) return UNIQL_E_NULL;
    if (n <= 0 || k <= 0 || k % 128 != 0 || n_pad < n || n_pad % 128 != 0) return UNIQL_E_SHAPE;
    if ((int64_t)(k / 16) * 2 * n_pad > 0x7fffffffLL * 256) return UNIQL_E_SHAPE;
    return pack_launch(codes, scales, B, S, n, k, n_pad, k, reinterpret_cast<hipStream_t>(stream));
}

int uniql_w4_embedding_lookup(const int64_t* ids, int64_t ntokens, const void* weight, const void* scales,
                              void* out, int64_t vocab, int dim, void* stream) {
    if (ntokens < 0 || vocab <= 0 || dim <= 0 || dim % 8 != 0) return UNIQL_E_SHAPE;
    if (ntokens == 0) return UNIQL_OK;
    if (!ids || !weight || !scales || !out) return UNIQL_E_NULL;
    if (!aligned16(out) || (reinterpret_cast<uintptr_t>(weight) & 3u)) return UNIQL_E_ALIGN;
    return embedding_launch(ids, ntokens, weight, scales, out, vocab, dim, reinterpret_cast<hipStream_t>(stream));
}

int uniql_fwht(const void* x, void* y, int64_t rows, int dim, int block, float scale, int dtype, void* stream) {
    if (dtype != UNIQL_DT_F16 && dtype != UNIQL_DT_BF16 && dtype != UNIQL_DT_F32) return UNIQL_E_UNSUPPORTED;
    if (rows < 0 || dim <= 0 || !is_pow2(block) || block < 2 || block > 32768 || dim % block != 0)
        return UNIQL_E_SHAPE;
    if (rows == 0) return UNIQL_OK;
    if (!x || !y) return UNIQL_E_NULL;
    if (block == 128 && dtype == UNIQL_DT_F16 && (!aligned16(x) || !aligned16(y))) return UNIQL_E_ALIGN;
    return fwht_launch(x, y, rows, dim, block, scale, dtype, reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
