// extern "C" surface: argument checks and dispatch.  Nothing here allocates,
// synchronises or throws.
#include <mutex>

#include "common.hpp"
#include "uniql_amd_diag.h"

namespace uniql {
int stream_launch(const void* A, int64_t lda, int k_valid, const void* B, const void* S, void* D,
                  const Epilogue& epi, void* accum, int m, int n, int k, int groups, int had_mode, float had_scale,
                  unsigned tune, hipStream_t stream);
bool stream_rotates_rows(int m, int k);
size_t stream_accum_bytes(int m, int n, int k);
bool stream_shape_ok(int k, int64_t lda);
int read_floor_launch(const void* B, const void* S, void* sink, int m, int n, int k, unsigned tune, hipStream_t stream);
size_t read_floor_sink_bytes(int m, int n, int k, unsigned tune);
int tile_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, const Epilogue& epi, void* accum,
                size_t accum_bytes, void* part, size_t part_bytes, int m, int n, int k, int groups, unsigned tune,
                hipStream_t stream);
size_t tile_part_bytes(int m, int n, int k, unsigned tune);
bool tile_shape_ok(int m, int n, int k, int64_t ldx, unsigned tune);
int pad_rows_launch(const void* A, int64_t lda, int k_in, void* dst, int k, int m, hipStream_t stream);
size_t tile_accum_bytes(int m, int n, int k, unsigned tune = 0);
int wide_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, const Epilogue& epi, int m, int n,
                int k, int groups, hipStream_t stream);
bool wide_shape_ok(int m, int n, int k, int groups, int64_t ldx);
bool wide_preferred(int m, int n, int k, unsigned tune);
int dequant_launch(const void* B, const void* S, void* W, uint8_t* codes, int n, int k, int groups,
                   hipStream_t stream);
int embedding_launch(const int64_t* ids, int64_t ntokens, const void* weight, const void* scales, void* out,
                     int64_t vocab, int dim, hipStream_t stream);
int embedding_quantize_launch(const void* W, int64_t ldw, void* packed, void* scales, int64_t vocab, int dim,
                              hipStream_t stream);
int rope_indices_launch(void* q, int64_t q_row_stride, void* k, int64_t k_row_stride, const void* cos, const void* sin,
                        int64_t cos_row_stride, const void* indices, int index_bytes, int64_t rows, int seq_len,
                        int cos_batch, int n_qh, int n_kh, int hd, int cos_dim, hipStream_t stream);
int fwht_launch(const void* x, void* y, int64_t rows, int dim, int block, float scale, int dtype,
                hipStream_t stream);
int fwht_composite_launch(const void* x, void* y, int64_t rows, int dim, int base, float scale, int dtype,
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

int uniql_stream_capture_id(void* stream, unsigned long long* id) {
    if (!id) return UNIQL_E_NULL;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long capture = 0;
    if (hipStreamGetCaptureInfo(reinterpret_cast<hipStream_t>(stream), &status, &capture) != hipSuccess)
        return UNIQL_E_LAUNCH;
    *id = status == hipStreamCaptureStatusActive ? capture : 0;
    return UNIQL_OK;
}

const char* uniql_status_string(int code) {
    switch (code) {
        case UNIQL_OK: return "ok";
        case UNIQL_E_NULL: return "a required pointer is NULL";
        case UNIQL_E_SHAPE: return "sizes violate the packed layout (k % 128, n % 128, groups, dim, block)";
        case UNIQL_E_ALIGN: return "pointer or leading dimension not 16-byte aligned";
        case UNIQL_E_WORKSPACE: return "workspace, accum or temp buffer too small";
        case UNIQL_E_UNSUPPORTED: return "request not supported by this build";
        case UNIQL_E_LAUNCH: return "HIP runtime rejected the kernel launch";
        case UNIQL_E_STATIC_LIMIT:
            return "the call needs more scratch memory than the library's static buffer holds "
                   "(uniql_w4a16_gemm_static_limit); use uniql_w4a16_gemm with caller-provided buffers";
        default: return "unknown status";
    }
}

// rows up to this many take the weight-streaming kernel, more take the tiled one
static constexpr int kStreamMaxM = 16;

// which kernel takes a call
static bool takes_stream_kernel(int m, unsigned flags) {
    bool use_stream = m <= kStreamMaxM;
    if (flags & UNIQL_F_FORCE_SKINNY) use_stream = true;
    if (flags & UNIQL_F_FORCE_TILED) use_stream = false;
    return use_stream;
}

// How the streaming kernel itself applies a rotation: 1 the 128-block one while staging, 2 whole
// rows (block = k, a power of two, few rows, input not shorter than k), 0 not at all: then the
// transform kernel runs first, into `temp`.
static int fused_rotation(int m, int k, int k_in, int had_block, bool use_stream, unsigned flags) {
    if (!use_stream || had_block == 0) return 0;
    if (had_block == 128) return 1;
    if (flags & UNIQL_F_SEPARATE_ROTATION) return 0;
    return (had_block == k && k_in == k && stream_rotates_rows(m, k)) ? 2 : 0;
}

// bytes of the rotated or zero-padded copy of the activations at the start of `temp`: every
// rotation that is not fused into the streaming kernel, and padding whenever the
// kernel cannot guard its own loads (tiled kernel) or a rotation comes first
static size_t activation_copy_bytes(int m, int k, int k_in, int had_block, bool use_stream, unsigned flags) {
    const bool rotate_first = had_block != 0 && fused_rotation(m, k, k_in, had_block, use_stream, flags) == 0;
    const bool pad_first = k_in != k && (rotate_first || !use_stream);
    return (rotate_first || pad_first) ? round256((size_t)m * k * sizeof(half_t)) : 0;
}

// What one layer call needs, decided in ONE place for the argument checks, the launch and the
// entry point that brings its own scratch memory: which kernel takes the call, whether the
// activations are copied (rotated / zero-padded) into `temp` first, and the bytes of `accum` and
// `temp` that follow from that.  The 256 x 256 kernel needs neither buffer.
struct LinearNeeds {
    bool use_stream, use_wide, rotate_first, pad_first;
    int had_mode;
    int64_t ld_kernel;   // row stride the product kernel will see
    size_t accum_bytes;  // rounded to 256
    size_t act_bytes;    // copy of the activations at the start of temp (rounded to 256), or 0
    size_t part_bytes;   // the tiled kernel's partial tiles behind it, or 0
};
static LinearNeeds linear_needs(int m, int n, int k, int k_in, int64_t lda, int groups, int had_block, unsigned flags) {
    LinearNeeds q;
    const unsigned tune = flags >> 8;
    q.use_stream = takes_stream_kernel(m, flags);
    q.had_mode = fused_rotation(m, k, k_in, had_block, q.use_stream, flags);
    q.rotate_first = had_block != 0 && q.had_mode == 0;
    // the transform kernel reads dense rows of k values: a strided or short input is first copied
    // (and zero-padded) into the temporary buffer, then rotated there in place
    q.pad_first = q.rotate_first ? (k_in != k || lda != k) : (k_in != k && !q.use_stream);
    q.ld_kernel = (q.rotate_first || q.pad_first) ? (int64_t)k : lda;
    // large M: the 256 x 256 kernel where it is the faster one and can take the call
    q.use_wide = !q.use_stream && wide_preferred(m, n, k, tune) && wide_shape_ok(m, n, k, groups, q.ld_kernel);
    q.accum_bytes = round256(q.use_stream ? stream_accum_bytes(m, n, k) : q.use_wide ? 0 : tile_accum_bytes(m, n, k, tune));
    q.act_bytes = (q.rotate_first || q.pad_first) ? round256((size_t)m * k * sizeof(half_t)) : 0;
    q.part_bytes = (q.use_stream || q.use_wide) ? 0 : tile_part_bytes(m, n, k, tune);
    return q;
}

int uniql_w4a16_linear_workspace(int m, int n, int k, int k_in, int had_block, unsigned flags, size_t* accum_bytes,
                                 size_t* temp_bytes) {
    if (!accum_bytes || !temp_bytes) return UNIQL_E_NULL;
    *accum_bytes = *temp_bytes = 0;
    if (m < 0 || n <= 0 || k <= 0 || n % 128 != 0 || k % 128 != 0) return UNIQL_E_SHAPE;
    if (m == 0) return UNIQL_OK;
    const bool use_stream = takes_stream_kernel(m, flags);
    const unsigned tune = flags >> 8;
    // (the 256 x 256 kernel needs neither buffer; the sizes are the 128 x 128 kernel's, which takes
    // the call when the scales are per column)
    *accum_bytes = round256(use_stream ? stream_accum_bytes(m, n, k) : tile_accum_bytes(m, n, k, tune));
    // a strided input ahead of a separate rotation is compacted into the copy as well: count it
    const size_t act = had_block != 0 && fused_rotation(m, k, k_in, had_block, use_stream, flags) == 0
                           ? round256((size_t)m * k * sizeof(half_t))
                           : activation_copy_bytes(m, k, k_in, had_block, use_stream, flags);
    *temp_bytes = act + (use_stream ? 0 : round256(tile_part_bytes(m, n, k, tune)));
    return UNIQL_OK;
}

size_t uniql_w4a16_gemm_accum_bytes(int m, int n, int k) {
    if (m <= 0 || n <= 0 || k <= 0 || n % 128 != 0 || k % 128 != 0) return 0;
    // enough for either kernel with its own plan (forced tuning fields: uniql_w4a16_linear_workspace)
    const size_t a = stream_accum_bytes(m, n, k), b = tile_accum_bytes(m, n, k);
    return round256(a > b ? a : b);
}

size_t uniql_w4a16_linear_temp_bytes(int m, int n, int k, int k_in, int had_block) {
    if (m <= 0 || n <= 0 || k <= 0 || n % 128 != 0 || k % 128 != 0) return 0;
    // the copy of the activations (as if the tiled kernel took the call: the larger case) and the
    // partial tiles of the tiled kernel's own plan
    const size_t act = (had_block != 0 || k_in != k) ? round256((size_t)m * k * sizeof(half_t)) : 0;
    return act + (takes_stream_kernel(m, 0) ? 0 : round256(tile_part_bytes(m, n, k, 0)));
}

size_t uniql_w4a16_gemm_temp_bytes(int m, int n, int k, int had_block) {
    return uniql_w4a16_linear_temp_bytes(m, n, k, k, had_block);
}

// check_only: every argument check, then return before the first kernel is enqueued
static int linear_impl(const void* A, int64_t lda, int k_in, const void* B, const void* S, const void* bias,
                       const void* residual, int64_t ldr, void* D, int64_t ldd, int n_out, int epilogue,
                       const int32_t* workspace,
                       int64_t workspace_len, void* accum, size_t accum_bytes, void* temp, size_t temp_bytes, int m,
                       int n, int k, int groups, int had_block, float had_scale, unsigned flags, void* stream,
                       bool check_only) {
    const int rc = check_linear_shape(m, n, k, groups);
    if (rc != UNIQL_OK) return rc;
    const bool transpose = (flags & UNIQL_F_TRANSPOSE_OUT) != 0;
    if (epilogue != UNIQL_EPI_NONE && epilogue != UNIQL_EPI_SILU_MUL && epilogue != UNIQL_EPI_RELU2)
        return UNIQL_E_UNSUPPORTED;
    const bool gated = epilogue == UNIQL_EPI_SILU_MUL;
    if (k_in <= 0 || k_in > k || k - k_in >= 128 || (k_in % 8) != 0) return UNIQL_E_SHAPE;
    if (n_out <= 0 || n_out > (gated ? n / 2 : n) || ldd < (transpose ? m : n_out)) return UNIQL_E_SHAPE;
    if (m == 0) return UNIQL_OK;
    if (!A || !B || !S || !D) return UNIQL_E_NULL;
    if (lda < k_in || (lda % 8) != 0) return UNIQL_E_ALIGN;
    const bool out_f32 = (flags & UNIQL_F_OUT_F32) != 0;
    if (!aligned16(A) || !aligned16(B) || !aligned16(S)) return UNIQL_E_ALIGN;
    if (reinterpret_cast<uintptr_t>(D) % (out_f32 ? 4 : 2) != 0) return UNIQL_E_ALIGN;
    if (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)) return UNIQL_E_ALIGN;
    if (residual) {
        if (epilogue != UNIQL_EPI_NONE) return UNIQL_E_UNSUPPORTED;  // activations feed the next layer, not the residual stream
        if (ldr < n_out) return UNIQL_E_SHAPE;
        if (reinterpret_cast<uintptr_t>(residual) & 1u) return UNIQL_E_ALIGN;
    }
    if (workspace && workspace_len < n / 128) return UNIQL_E_WORKSPACE;
    if (had_block != 0 && (!is_pow2(had_block) || had_block < 2 || had_block > 32768 || k % had_block != 0))
        return UNIQL_E_SHAPE;
    if ((accum && !aligned16(accum)) || (temp && !aligned16(temp))) return UNIQL_E_ALIGN;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const unsigned tune = flags >> 8;  // tuning fields, see the header
    const LinearNeeds q = linear_needs(m, n, k, k_in, lda, groups, had_block, flags);
    const bool use_stream = q.use_stream, use_wide = q.use_wide, rotate_first = q.rotate_first, pad_first = q.pad_first;
    const int had_mode = q.had_mode;
    const int64_t ld_kernel = q.ld_kernel;
    const void* Ain = A;
    int64_t ld = lda;
    int k_valid = k_in;
    const size_t need_accum = q.accum_bytes;
    if (need_accum > 0 && (!accum || accum_bytes < need_accum)) return UNIQL_E_WORKSPACE;
    // temp: the copy of the activations, then the tiled kernel's partial tiles when it splits K
    const size_t act_bytes = q.act_bytes, part_bytes = q.part_bytes;
    if (act_bytes + part_bytes > 0 && (!temp || temp_bytes < act_bytes + part_bytes)) return UNIQL_E_WORKSPACE;
    void* part = part_bytes ? reinterpret_cast<char*>(temp) + act_bytes : nullptr;
    // last check before the first kernel is enqueued: whether the tiled kernel can take the shape
    if (!use_stream && !use_wide && !tile_shape_ok(m, n, k, ld_kernel, tune)) return UNIQL_E_SHAPE;
    if (use_stream && !stream_shape_ok(k, ld_kernel)) return UNIQL_E_SHAPE;
    if (check_only) return UNIQL_OK;
    if (pad_first) {
        const int e = pad_rows_launch(A, lda, k_in, temp, k, m, st);
        if (e != UNIQL_OK) return e;
        Ain = temp;
        ld = k;
        k_valid = k;
    }
    if (rotate_first) {
        const int e = fwht_launch(Ain, temp, m, k, had_block, had_scale, UNIQL_DT_F16, st);
        if (e != UNIQL_OK) return e;
        Ain = temp;
        ld = k;
    }
    Epilogue epi;
    epi.bias = reinterpret_cast<const half_t*>(bias);
    epi.residual = reinterpret_cast<const half_t*>(residual);
    epi.ldr = ldr;
    epi.ldd = ldd;
    epi.n_store = n_out;
    epi.gated = gated ? 1 : 0;
    epi.out_f32 = out_f32 ? 1 : 0;
    epi.transpose = transpose ? 1 : 0;
    epi.relu2 = epilogue == UNIQL_EPI_RELU2 ? 1 : 0;
    epi.vec_ok = (!transpose && ldd % 8 == 0 && aligned16(D)) ? 1 : 0;
    if (use_stream)
        return stream_launch(Ain, ld, k_valid, B, S, D, epi, accum, m, n, k, groups, had_mode, had_scale, tune, st);
    if (use_wide) return wide_launch(Ain, ld, B, S, D, epi, m, n, k, groups, st);
    return tile_launch(Ain, ld, B, S, D, epi, accum, accum_bytes, part, part_bytes, m, n, k, groups, tune, st);
}

int uniql_w4a16_linear(const void* A, int64_t lda, int k_in, const void* B, const void* S, const void* bias,
                       const void* residual, int64_t ldr, void* D, int64_t ldd, int n_out, int epilogue,
                       const int32_t* workspace,
                       int64_t workspace_len, void* accum, size_t accum_bytes, void* temp, size_t temp_bytes, int m,
                       int n, int k, int groups, int had_block, float had_scale, unsigned flags, void* stream) {
    return linear_impl(A, lda, k_in, B, S, bias, residual, ldr, D, ldd, n_out, epilogue, workspace, workspace_len, accum,
                       accum_bytes, temp, temp_bytes, m, n, k, groups, had_block, had_scale, flags, stream, false);
}

static int gemm_impl(const void* A, int64_t lda, const void* B, const void* S, void* D, const int32_t* workspace,
                     int64_t workspace_len, void* accum, size_t accum_bytes, void* temp, size_t temp_bytes, int m,
                     int n, int k, int groups, int had_block, float had_scale, unsigned flags, void* stream,
                     bool check_only) {
    if (D && !aligned16(D)) return UNIQL_E_ALIGN;
    // transposed: D is [n, m8] with m8 = m rounded up to 8, as the reference allocates it
    // (marlin_gemm_kernel.cuh:1023-1026)
    const int64_t ldd = (flags & UNIQL_F_TRANSPOSE_OUT) ? (int64_t)((m + 7) / 8) * 8 : n;
    return linear_impl(A, lda, k, B, S, nullptr, nullptr, 0, D, ldd, n, UNIQL_EPI_NONE, workspace, workspace_len, accum,
                       accum_bytes, temp, temp_bytes, m, n, k, groups, had_block, had_scale, flags, stream, check_only);
}

int uniql_w4a16_gemm(const void* A, int64_t lda, const void* B, const void* S, void* D, const int32_t* workspace,
                     int64_t workspace_len, void* accum, size_t accum_bytes, void* temp, size_t temp_bytes, int m,
                     int n, int k, int groups, int had_block, float had_scale, unsigned flags, void* stream) {
    return gemm_impl(A, lda, B, S, D, workspace, workspace_len, accum, accum_bytes, temp, temp_bytes, m, n, k, groups,
                     had_block, had_scale, flags, stream, false);
}

// ---- the entry point that allocates nothing --------------------------------------------------
// All the scratch memory a product needs (the zero-in / zero-out exchange words first, then the
// temporary area) lives in one array in this library's device image.  Each GPU holds its own copy
// at its own address; the name below is only a host-side handle for hipGetSymbolAddress, never a
// device address, so every use goes through the per-device pointer looked up once.
static constexpr size_t kStaticAccumBytes = (size_t)4 << 20;   // exchange words: 16 rows x 32768 columns
static constexpr size_t kStaticTempBytes = (size_t)12 << 20;   // rotated rows / partial tiles
static __device__ __align__(256) unsigned char scratch[kStaticAccumBytes + kStaticTempBytes];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[kMaxDevices];  // zero-initialised: not looked up yet

// the current device's copy of the array, or nullptr
static unsigned char* static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = reinterpret_cast<unsigned char*>(p);
    }
    return g_scratch_ptr[dev];
}

size_t uniql_w4a16_gemm_static_limit(int which) {
    return which == 0 ? kStaticAccumBytes : (which == 1 ? kStaticTempBytes : 0);
}

int uniql_w4a16_gemm_static(const void* A, int64_t lda, const void* B, const void* S, void* D,
                            const int32_t* workspace, int64_t workspace_len, int m, int n, int k, int groups,
                            int had_block, float had_scale, unsigned flags, void* stream) {
    const int rc = check_linear_shape(m, n, k, groups);
    if (rc != UNIQL_OK) return rc;
    if (m == 0) return UNIQL_OK;
    // (the sizes of the kernel that will really take the call: a long prefill on the 256 x 256 kernel needs
    // no scratch at all, whatever the 128-column kernel would have asked for)
    const LinearNeeds q = linear_needs(m, n, k, k, lda, groups, had_block, flags);
    const size_t need_accum = q.accum_bytes, need_temp = q.act_bytes + round256(q.part_bytes);
    if (need_accum > kStaticAccumBytes || need_temp > kStaticTempBytes) return UNIQL_E_STATIC_LIMIT;
    if (!A || !B || !S || !D) return UNIQL_E_NULL;
    unsigned char* base = static_scratch();
    if (!base) return UNIQL_E_LAUNCH;
    void* accum = need_accum ? base : nullptr;
    void* temp = need_temp ? base + kStaticAccumBytes : nullptr;
    // every argument check of the product first: nothing is enqueued for a call that will be refused
    const int crc = gemm_impl(A, lda, B, S, D, workspace, workspace_len, accum, need_accum, temp, need_temp, m, n, k,
                              groups, had_block, had_scale, flags, stream, true);
    if (crc != UNIQL_OK) return crc;
    // The exchange words must be zero on entry.  The kernels leave them zero, but the array is
    // shared by every call on this GPU, so the part this call uses is cleared by a small kernel
    // (a kernel, not a memset node: the call may be recorded into a graph).
    if (need_accum > 0) {
        const int e = uniql_clear(base, need_accum, stream);
        if (e != UNIQL_OK) return e;
    }
    return gemm_impl(A, lda, B, S, D, workspace, workspace_len, accum, need_accum, temp, need_temp, m, n, k, groups,
                     had_block, had_scale, flags, stream, false);
}

int uniql_w4a16_read_floor(const void* B, const void* S, void* sink, size_t sink_bytes, int m, int n, int k,
                           unsigned flags, void* stream) {
    const int rc = check_linear_shape(m, n, k, k / 128);
    if (rc != UNIQL_OK) return rc;
    if (m <= 0) return UNIQL_E_SHAPE;
    if (!B || !S || !sink) return UNIQL_E_NULL;
    if (!aligned16(B) || !aligned16(S)) return UNIQL_E_ALIGN;
    if (sink_bytes < read_floor_sink_bytes(m, n, k, flags >> 8)) return UNIQL_E_WORKSPACE;
    return read_floor_launch(B, S, sink, m, n, k, flags >> 8, reinterpret_cast<hipStream_t>(stream));
}

size_t uniql_w4a16_read_floor_sink_bytes(int m, int n, int k, unsigned flags) {
    if (m <= 0 || n <= 0 || k <= 0 || n % 128 != 0 || k % 128 != 0) return 0;
    return read_floor_sink_bytes(m, n, k, flags >> 8);
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

int uniql_w4_embedding_quantize(const void* W, int64_t ldw, void* packed, void* scales, int64_t vocab, int dim,
                                void* stream) {
    if (vocab < 0 || dim <= 0 || dim % 8 != 0 || ldw < dim || ldw % 8 != 0) return UNIQL_E_SHAPE;
    if (vocab == 0) return UNIQL_OK;
    if (!W || !packed || !scales) return UNIQL_E_NULL;
    if (!aligned16(W) || (reinterpret_cast<uintptr_t>(packed) & 3u)) return UNIQL_E_ALIGN;
    return embedding_quantize_launch(W, ldw, packed, scales, vocab, dim, reinterpret_cast<hipStream_t>(stream));
}

int uniql_rope_indices(void* q, int64_t q_row_stride, void* k, int64_t k_row_stride, const void* cos,
                       const void* sin, int64_t cos_row_stride, const void* indices, int index_bytes, int64_t rows,
                       int seq_len, int cos_batch, int n_q_heads, int n_kv_heads, int head_dim, int cos_dim,
                       void* stream) {
    if (rows < 0 || seq_len < 0 || n_q_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || cos_dim <= 0)
        return UNIQL_E_SHAPE;
    if (seq_len == 0) return rows == 0 ? UNIQL_OK : UNIQL_E_SHAPE;  // no tokens: nothing to rotate
    if (head_dim % 2 != 0 || n_q_heads % n_kv_heads != 0) return UNIQL_E_SHAPE;
    if (index_bytes != 1 && index_bytes != 4 && index_bytes != 8) return UNIQL_E_UNSUPPORTED;
    if (index_bytes == 1 && cos_dim > 256) return UNIQL_E_SHAPE;
    if (cos_batch != 1 && (cos_batch <= 0 || rows != (int64_t)cos_batch * seq_len)) return UNIQL_E_SHAPE;
    if (cos_batch == 1 && rows % seq_len != 0) return UNIQL_E_SHAPE;
    if (q_row_stride < (int64_t)n_q_heads * head_dim || k_row_stride < (int64_t)n_kv_heads * head_dim ||
        cos_row_stride < cos_dim)
        return UNIQL_E_SHAPE;
    if (rows == 0) return UNIQL_OK;
    if (!q || !k || !cos || !sin || !indices) return UNIQL_E_NULL;
    return rope_indices_launch(q, q_row_stride, k, k_row_stride, cos, sin, cos_row_stride, indices, index_bytes,
                               rows, seq_len, cos_batch, n_q_heads, n_kv_heads, head_dim, cos_dim,
                               reinterpret_cast<hipStream_t>(stream));
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

int uniql_fwht_composite(const void* x, void* y, int64_t rows, int dim, int base, float scale, int dtype, void* stream) {
    if (dtype != UNIQL_DT_F16 && dtype != UNIQL_DT_BF16 && dtype != UNIQL_DT_F32) return UNIQL_E_UNSUPPORTED;
    if (base != 12 && base != 20 && base != 28 && base != 40) return UNIQL_E_UNSUPPORTED;
    if (rows < 0 || dim <= 0 || dim % base != 0 || !is_pow2(dim / base) || dim > 40960) return UNIQL_E_SHAPE;
    if (rows == 0) return UNIQL_OK;
    if (!x || !y) return UNIQL_E_NULL;
    return fwht_composite_launch(x, y, rows, dim, base, scale, dtype, reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
