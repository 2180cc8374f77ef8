/*
 * uniql_amd.h - C ABI of the MI355X (gfx950) W4A16 kernels.
 *
 * Plain pointers and sizes only.  All pointers named "device" are HIP device
 * addresses on the current device.  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  No entry point synchronises the stream
 * or frees memory; every call only enqueues kernels, so all of them can be
 * recorded into a HIP graph.  Return value: 0 on success, a negative
 * UNIQL_E_* code otherwise (nothing was launched then).
 *
 * Paths in the comments are files of the reference (enyac-group/UniQL).
 */
#ifndef UNIQL_AMD_H
#define UNIQL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define UNIQL_ABI_VERSION 1

enum {
    UNIQL_OK = 0,
    UNIQL_E_NULL = -1,        /* a required pointer is NULL                        */
    UNIQL_E_SHAPE = -2,       /* m/n/k/groups violate the layout's divisibility    */
    UNIQL_E_ALIGN = -3,       /* a pointer or leading dimension is not 16-byte aligned */
    UNIQL_E_WORKSPACE = -4,   /* workspace, accum or temp buffer too small         */
    UNIQL_E_UNSUPPORTED = -5, /* valid request this build does not implement       */
    UNIQL_E_LAUNCH = -6,      /* the HIP runtime rejected a launch                 */
    UNIQL_E_STATIC_LIMIT = -7 /* uniql_w4a16_gemm_static: the call needs more scratch than the static buffer holds */
};

/* flags of uniql_w4a16_gemm / uniql_w4a16_linear.  Bits 1, 2, 4 and 8..21 select kernels and plans
 * for tests and measurements; they are described in uniql_amd_diag.h and are zero in production. */
enum {
    UNIQL_F_OUT_F32 = 1 << 0,      /* D is float32 [m, n] instead of fp16: the value before the final rounding */
    UNIQL_F_TRANSPOSE_OUT = 1 << 3 /* the reference's output_transpose ("sequence length last",
                                      csrc/linear/marlin_gemm_kernel.cuh:574-606,1023-1026): D is [n, ldd]
                                      with D[j, i] = product[i, j]; uniql_w4a16_gemm uses ldd = m rounded up
                                      to a multiple of 8 as the reference does and leaves the padding columns
                                      untouched; uniql_w4a16_linear takes ldd >= m from the caller */
};

int uniql_abi_version(void);
const char* uniql_status_string(int code);

/* The identifier of the graph capture `stream` is recording into, 0 when it is not capturing.
 * No counterpart in the reference (its wrapper allocates its scratch with torch on every call,
 * csrc/linear/marlin_gemm_kernel.cuh:1018); a host shim that caches the zero-in / zero-out `accum`
 * buffer needs it: a buffer allocated and zero-filled while capturing is only zero when that
 * graph replays, so it must not serve another capture or eager calls. */
int uniql_stream_capture_id(void* stream, unsigned long long* id);

/* Fills `bytes` bytes at device address `p` (both multiples of 16) with zeros, with a kernel.  No
 * counterpart in the reference.  For the host shim's `accum` buffers: a clear that may be recorded
 * into a graph must be a kernel node, not a memset node (memset nodes have given wrong results on
 * replays after the first on this platform), and what an allocator's zero fill records is not
 * under the caller's control. */
int uniql_clear(void* p, size_t bytes, void* stream);

/*
 * D[m, n] = A[m, k] . dequant(B)[k, n],  fp16 in, fp32 accumulate, fp16 out.
 * Replaces quant_linear_cuda.w4a16o16_gemm (csrc/linear/quant_linear.cpp:6-24,
 * host wrapper csrc/linear/marlin_gemm_kernel.cuh:991-1052).
 *
 *   A          device, fp16 [m, k] row-major, row stride lda elements (lda >= k, lda % 8 == 0)
 *   B          device, int32 [k/16, 2 n]: the packed layout written by
 *              quantize/quantize_helpers.py:66-84 with the table of :144-165
 *   S          device, fp16 [groups, n], permuted by quantize_helpers.py:168-180;
 *              groups == k/128 (group-128 scales) or groups == 1 (one scale per column)
 *   D          device, fp16 [m, n] row-major (float32 with UNIQL_F_OUT_F32)
 *   workspace  device, int32 [workspace_len] or NULL: the module's `workspace` buffer
 *              (quantize/quant_linear_layers.py:33-35; the reference's inter-block
 *              lock array).  Only its length is checked (>= n/128, as the reference
 *              checks it); it is never read or written, so it stays zero.
 *   accum      device, uniql_w4a16_gemm_accum_bytes(m, n, k) bytes, ALL ZERO on entry
 *              and all zero again when the kernels have finished: the words through
 *              which workgroups that share output columns combine their partial sums
 *              (streaming kernel: a 64-bit sum|count word per output element of up to
 *              16 rows; tiled kernel: an arrival count per output tile).  Replaces the
 *              reference's per-call fp16 `C` buffer and its locks
 *              (marlin_gemm_kernel.cuh:515-570,1018).  A caller clears it once and
 *              reuses it for every call on the same stream; two calls that may run
 *              concurrently need separate buffers.  May be NULL when the size is 0.
 *   temp       device, uniql_w4a16_gemm_temp_bytes(m, n, k, had_block) bytes, contents
 *              irrelevant: rotated activations whenever the rotation is not fused, and
 *              the fp32 partial tiles of the tiled kernel when its plan splits K over
 *              workgroups; may be NULL when that size is 0.  Two calls that may run
 *              concurrently need separate buffers.
 *   had_block  0: none.  Otherwise the activations are rotated first,
 *              A <- fp16(A . H_had_block * had_scale) on consecutive
 *              had_block-wide pieces of each row.  Inside the streaming kernel (m <= 16,
 *              no extra memory traffic): 128, and had_block == k for a power-of-two k
 *              with min(m, 16) * k <= 16384 (every workgroup transforms the rows into LDS
 *              while its first weights are on their way).  Any other power of two
 *              (<= 32768, dividing k), and every rotation for larger m, runs the
 *              transform kernel into `temp` first.  Same values either way.
 *   k % 128 == 0, n % 128 == 0 (the module pads n to 256).
 *
 * Partial sums that meet in the streaming kernel's `accum` words are rounded to multiples of
 * 2^-24 and clamped to +-2^18 (beyond the fp16 range of D, so an infinite partial sum still
 * gives an infinite fp16 result; with UNIQL_F_OUT_F32 the clamp itself is visible).  A NaN
 * partial sum makes the result NaN, as without a K split.  The one difference from a launch
 * that does not split K: +inf and -inf that meet from DIFFERENT workgroups cancel to a finite
 * value instead of NaN.  Either kernel's result is the same from run to run: integer additions
 * in the first, partial tiles added in split order in the second.
 */
size_t uniql_w4a16_gemm_accum_bytes(int m, int n, int k);
size_t uniql_w4a16_gemm_temp_bytes(int m, int n, int k, int had_block);

int uniql_w4a16_gemm(const void* A, int64_t lda, const void* B, const void* S, void* D,
                     const int32_t* workspace, int64_t workspace_len,
                     void* accum, size_t accum_bytes, void* temp, size_t temp_bytes,
                     int m, int n, int k, int groups,
                     int had_block, float had_scale,
                     unsigned flags, void* stream);

/*
 * uniql_w4a16_gemm for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * wrapper allocates its reduction buffer on every call (csrc/linear/marlin_gemm_kernel.cuh:1018).
 * Same arguments and results as uniql_w4a16_gemm without `accum` and `temp`: both come from a
 * 16 MiB array inside the library's device image (one copy per GPU, held until the process ends):
 * uniql_w4a16_gemm_static_limit(0) bytes of exchange words (4 MiB: the streaming kernel's 16-row
 * slab up to n = 32768) and uniql_w4a16_gemm_static_limit(1) bytes of temporary area (12 MiB:
 * rotated activations, the tiled kernel's partial tiles).  A call whose plan needs more of either
 * returns UNIQL_E_STATIC_LIMIT and launches nothing (the needs are those of the kernel that takes
 * the call: at most what uniql_w4a16_linear_workspace reports, nothing at all for a long prefill
 * on the 256 x 256 tiles).  The
 * call itself allocates and frees nothing; it enqueues one small clearing kernel for the
 * exchange words it will use, then the kernels of uniql_w4a16_gemm.
 * Every call on a GPU shares that GPU's array: calls that may overlap on one GPU (different
 * streams, or graphs replayed concurrently) race and must use uniql_w4a16_gemm with separate
 * buffers instead.
 * Before a call is recorded into a graph, one call with the same m class (1, 2, 3..4, 5..8, 9..16,
 * more), flags and rotation must have run eagerly on that device: the first call per device
 * resolves the array's address (hipGetSymbolAddress) and the first launch of a kernel that uses
 * more than 64 KiB of LDS sets a function attribute, neither of which may happen while a stream
 * is capturing.
 */
size_t uniql_w4a16_gemm_static_limit(int which);
int uniql_w4a16_gemm_static(const void* A, int64_t lda, const void* B, const void* S, void* D,
                            const int32_t* workspace, int64_t workspace_len,
                            int m, int n, int k, int groups,
                            int had_block, float had_scale,
                            unsigned flags, void* stream);

/*
 * The whole forward of the reference's layer in one call, with the work around the product
 * done inside the kernels instead of by separate tensor operations:
 * W4A16B16O16Linear.forward (quantize/quant_linear_layers.py:92-114: pad the input to k,
 * product, drop the padded output columns, add the bias), the decoder layer's
 * `residual + layer(x)` (modeling/llama/llama_qblocks.py:182,188) and, with UNIQL_EPI_SILU_MUL,
 * the MLP's act_fn(gate_proj(x)) * up_proj(x) (modeling/llama/llama_qblocks.py:48-51) or, with
 * UNIQL_EPI_RELU2, the un-gated act_fn(up_proj(x)) with the squared ReLU
 * (modeling/nemotron_h/nemotron_h_qblocks.py:577,588; mlp_hidden_act "relu2",
 * modeling/nemotron_h/configuration_nemotron_h.py:145).
 * Arguments as uniql_w4a16_gemm, plus:
 *   k_in      columns of A that exist (lda >= k_in, k_in % 8 == 0, k - 128 < k_in <= k); K rows
 *             from k_in on count as zero activations (the module's pad_in)
 *   bias      device, fp16 [n_out] in natural column order, or NULL; added to the fp16-rounded
 *             product and rounded again, as the reference's `y + self.bias` does.  With
 *             UNIQL_EPI_SILU_MUL: [2 n_out], the gate biases followed by the up biases
 *   residual  device, fp16 [m, ldr] (ldr >= n_out) or NULL: added to the rounded (and biased)
 *             product and rounded again; may be the same memory as D (every element is read
 *             by the thread that writes it); only with UNIQL_EPI_NONE
 *   D, ldd    output rows of ldd elements (ldd >= n_out); 16-byte stores are used when
 *             ldd % 8 == 0 and D is 16-byte aligned
 *   n_out     output columns that exist (the module's out_features); the rest of n is dropped
 *   epilogue  UNIQL_EPI_NONE: n_out <= n.
 *             UNIQL_EPI_SILU_MUL: B and S hold the gate and the up projection interleaved in
 *             blocks of 64 columns (block 2c = columns 64c.. of gate, block 2c+1 = the same
 *             columns of up; packed words and permuted scales of a 64-column block are
 *             contiguous, so this is a concatenation of slices of the two layers' tensors), n is
 *             twice the padded width of one projection, n_out <= n/2, and
 *             D[m, j] = fp16(fp16(silu(g)) * u) with g, u the fp16-rounded (and biased) gate and
 *             up outputs of column j: the reference's sequence of roundings.
 *             UNIQL_EPI_RELU2: D[m, j] = fp16(max(y, 0)^2) with y the fp16-rounded (and biased)
 *             output: torch.square(relu(y)) on the fp16 tensor.
 *   temp      uniql_w4a16_linear_temp_bytes(m, n, k, k_in, had_block) bytes
 * With UNIQL_F_OUT_F32 D is float32 and no intermediate rounding is applied.
 */
enum { UNIQL_EPI_NONE = 0, UNIQL_EPI_SILU_MUL = 1, UNIQL_EPI_RELU2 = 2 };

size_t uniql_w4a16_linear_temp_bytes(int m, int n, int k, int k_in, int had_block);

/* Sizes of `accum` and `temp` for one call with these flags (the two functions above and
 * uniql_w4a16_gemm_accum_bytes answer for flags = 0; forced kernels or tuning fields can need
 * more).  `temp` holds the rotated or zero-padded copy of the activations and, when the tiled
 * kernel splits K over workgroups, one fp32 partial tile per (output tile, split); `accum` then
 * holds one arrival count per output tile.  No counterpart in the reference, whose wrapper
 * allocates its reduction buffer itself (csrc/linear/marlin_gemm_kernel.cuh:1018). */
int uniql_w4a16_linear_workspace(int m, int n, int k, int k_in, int had_block, unsigned flags,
                                 size_t* accum_bytes, size_t* temp_bytes);


int uniql_w4a16_linear(const void* A, int64_t lda, int k_in, const void* B, const void* S, const void* bias,
                       const void* residual, int64_t ldr,
                       void* D, int64_t ldd, int n_out, int epilogue,
                       const int32_t* workspace, int64_t workspace_len,
                       void* accum, size_t accum_bytes, void* temp, size_t temp_bytes,
                       int m, int n, int k, int groups,
                       int had_block, float had_scale,
                       unsigned flags, void* stream);

/*
 * W[k, n] fp16 = fp16_rn((code - 8) * scale), natural (un-permuted) order.
 * The value csrc/linear/marlin_gemm_kernel.cuh:118-146 builds in registers and
 * quantize/quantize_helpers.py:118 calls w_ref.  Also writes the raw codes
 * (uint8 [k, n]) when `codes` is not NULL: the inverse of
 * quantize_helpers.py:303-328 on the device.
 */
int uniql_w4a16_dequant(const void* B, const void* S, void* W, uint8_t* codes,
                        int n, int k, int groups, void* stream);

/*
 * Group-128 quantisation of an fp16 weight matrix on the device, straight into the packed
 * layout.  Replaces the host arithmetic of W4A16B16O16Linear.from_fp16
 * (quantize/quant_linear_layers.py:50-89 -> quantize/quantize_helpers.py:87-141,183-241: fp16
 * tensors on the CPU, every operation rounded to fp16) with the same results bit for bit.
 *   W             device, fp16 [out_features, in_features] row-major (nn.Linear.weight), row
 *                 stride ldw elements
 *   given_scales  NULL: scale = fp16(max|w| * 2/15) per (group of 128 K, column), code =
 *                 clamp(round(w / scale) + 8, 0, 15).  Otherwise device fp16
 *                 [k_pad/128, out_features], natural order: the GPTQ hand-over
 *                 (quantize_helpers.py:205-218), code = clamp(round(w / scale + 8), 0, 15)
 *   B             device out, int32 [k_pad/16, 2 n_pad]
 *   S             device out, fp16 [k_pad/128, n_pad], permuted
 *   k_pad = in_features rounded up to 128 (rows past in_features count as zero weights),
 *   n_pad >= out_features, n_pad % 128 == 0 (columns past out_features get code 0, scale 0);
 *   in_features > 128 (the one-scale-per-column case of the reference is not produced).
 */
int uniql_w4a16_quantize(const void* W, int64_t ldw, const void* given_scales, void* B, void* S,
                         int out_features, int in_features, int n_pad, int k_pad, void* stream);

/*
 * Packs ready codes and natural-order scales: the inverse of uniql_w4a16_dequant's `codes`
 * output.  Replaces get_w4a16_permute_weights + w4a16_permute_scales
 * (quantize/quantize_helpers.py:66-84,168-180) as the slicing functions of
 * modeling/modeling_helpers.py:235-867 use them after cutting the unpacked tensors.
 *   codes   device, uint8 [k, n] (values 0..15)
 *   scales  device, fp16 [k/128, n], natural order
 *   B       device out, int32 [k/16, 2 n_pad];  S  device out, fp16 [k/128, n_pad], permuted
 *   k % 128 == 0, n_pad >= n, n_pad % 128 == 0 (padding columns: code 0, scale 0)
 */
int uniql_w4a16_pack(const uint8_t* codes, const void* scales, void* B, void* S, int n, int k, int n_pad,
                     void* stream);

/*
 * out[t, :] = fp16_rn((code - 8) * scales[ids[t]]) for t < ntokens.
 * Replaces quant_embedding_cuda.w4a16_embedding_lookup
 * (csrc/embedding/quant_embedding_kernel.cuh:80-166).
 *   ids     device, int64 [ntokens]; each id must be in [0, vocab)
 *   weight  device, int32 [vocab, dim/8], packing of quantize/quant_embedding_layers.py:33-43
 *   scales  device, fp16 [vocab]
 *   out     device, fp16 [ntokens, dim];  dim % 8 == 0
 */
int uniql_w4_embedding_lookup(const int64_t* ids, int64_t ntokens,
                              const void* weight, const void* scales, void* out,
                              int64_t vocab, int dim, void* stream);

/*
 * Quantises an fp16 embedding table on the device: scales[v] = fp16(max|W[v, :]| / 8),
 * code = clamp(round(W / scale + 8), 0, 15) with every operation rounded to fp16, eight codes
 * per word in nibble order [0, 2, 4, 6, 1, 3, 5, 7].  Replaces the tensor arithmetic and the
 * host packing loop of W4O16Embedding.from_fp16 (quantize/quant_embedding_layers.py:26-48)
 * with the same results bit for bit.
 *   W       device, fp16 [vocab, dim], row stride ldw elements (ldw % 8 == 0), 16-byte aligned
 *   packed  device out, int32 [vocab, dim/8];  scales  device out, fp16 [vocab];  dim % 8 == 0
 */
int uniql_w4_embedding_quantize(const void* W, int64_t ldw, void* packed, void* scales,
                                int64_t vocab, int dim, void* stream);

/*
 * Rotary position embedding with gathered frequencies, in place:
 *   x[.., j] <- fp16(fp16(x[.., j] * cos[t, i(j)]) + fp16(rot(x)[.., j] * sin[t, i(j)]))
 * with rot(x) = (-x[d/2:], x[:d/2]) and i(j) = indices[kv head of the head][j].  Replaces
 * apply_rotary_pos_emb_indices_triton (modeling/rope_triton.py:10-177) with the arithmetic of
 * the tensor version it stands in for (modeling/llama/llama_rope.py:38-96; the same function
 * in modeling/qwen/qwen2_rope.py:37).
 *   q        device, fp16 [rows, n_q_heads, head_dim], token-major (the projections' output
 *            layout), rows = batch * seq_len, row stride q_row_stride elements; modified
 *   k        device, fp16 [rows, n_kv_heads, head_dim], row stride k_row_stride; modified
 *   cos,sin  device, fp16 [cos_batch, seq_len, cos_dim], row stride cos_row_stride;
 *            cos_batch is 1 (all batches share the table) or the batch size
 *   indices  device, [n_kv_heads, head_dim] integers of index_bytes (1: uint8 as the module
 *            stores them, 4: int32, 8: int64), each < cos_dim; query head h uses row
 *            h / (n_q_heads / n_kv_heads)
 * rows = 0 (with any seq_len >= 0) is a valid call that does nothing.
 */
int uniql_rope_indices(void* q, int64_t q_row_stride, void* k, int64_t k_row_stride,
                       const void* cos, const void* sin, int64_t cos_row_stride,
                       const void* indices, int index_bytes,
                       int64_t rows, int seq_len, int cos_batch,
                       int n_q_heads, int n_kv_heads, int head_dim, int cos_dim, void* stream);

/*
 * y[r, :] = round((x[r, :] . H) * scale), H = Sylvester Hadamard matrix applied
 * to consecutive `block`-wide pieces of each row (block == dim: the whole row);
 * butterflies in fp32, one rounding to the element type at the end.
 * Replaces fast_hadamard_transform_cuda.fast_hadamard_transform(x, scale) as
 * called by quantize/hadamard_helpers.py:22-48 (power-of-two case).
 *   x, y   device, [rows, dim] contiguous, element type `dtype` (UNIQL_DT_*); y may equal x
 *   block  power of two, 2 <= block <= 32768, dim % block == 0
 */
enum { UNIQL_DT_F16 = 0, UNIQL_DT_BF16 = 1, UNIQL_DT_F32 = 2 };

int uniql_fwht(const void* x, void* y, int64_t rows, int dim, int block,
               float scale, int dtype, void* stream);

/*
 * y[r, :] = round((x[r, :] . (H_base (x) H_P)) * scale) for dim = base * P, base in {12, 20, 28, 40}, P a power
 * of two: the row is `base` chunks of P values, every chunk gets the P-point transform, then the
 * base x base Hadamard matrix combines the chunks (y[c P + i] = sum_c' z[c' P + i] H[c'][c]); fp32
 * throughout, one rounding at the end.  Replaces fast_hadamard_transform_cuda.fast_hadamard_transform_{12,20,28,40}N
 * as selected by quantize/hadamard_helpers.py:20-31 (Qwen2's 3584 = 28 * 128, Llama's 14336 = 28 * 512).
 * The base matrices of that third-party package are not part of the reference tree; the ones used here
 * (Sloane's 12 x 12, Paley's constructions for 20 and 28, the doubled 20 for 40) satisfy H H^T = base I,
 * which is all that HadLinear and the Hadamard module need as long as both sides of a layer use this
 * library; results are NOT guaranteed to match weights rotated offline with the reference's tables.
 *   x, y   device, [rows, dim] contiguous, element type `dtype`; y may equal x;  dim <= 40960
 */
int uniql_fwht_composite(const void* x, void* y, int64_t rows, int dim, int base,
                         float scale, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* UNIQL_AMD_H */
