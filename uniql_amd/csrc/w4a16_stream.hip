// Weight-streaming W4A16 kernel for small M (decode): D[M,N] = X[M,K] . dequant(B)[K,N].
//
// The packed weight row r (16 K-rows) stores, per 64-column chunk, 32 sixteen-byte
// pieces; piece 4*c8 + kq holds K-rows {2kq, 2kq+1, 2kq+8, 2kq+9} of the eight
// columns c8 + 8*jb (jb = 0..7) of that chunk.  A wavefront reads one 128-column
// strip (two chunks) of a row with a single 16-byte load per lane, choosing the
// piece so that the registers ARE the B operand of v_mfma_f32_16x16x32_f16:
//
//     lane l :  slot = l % 16  ->  chunk = 2*strip + slot/8,  c8 = slot % 8
//               kq   = l / 16  ->  piece 4*c8 + kq
//
// Every byte of the 1 KiB row segment is fetched once and sixteen MFMAs (per jb one for the
// low and one for the high code pairs of the words) consume four packed rows (64 K values) at
// a time.  The activations are the A operand:
// rows of X (up to 16 per launch) staged through LDS in the same K order.  MFMA is
// used purely as a wide dot-product unit: its cost does not depend on M, so
// M = 1..16 all run at the weight-streaming rate.
//
// Every weight is expanded to the reference's fp16 value fp16_rn((code - 8) * scale)
// (csrc/linear/marlin_gemm_kernel.cuh:118-146) before it enters the matrix unit; the products are
// exact in the MFMA and accumulate in fp32, so the result equals the reference's value up to the
// order of the fp32 additions, for every M.  Two expansions give that value (see process()):
//   * short, 9 vector instructions per packed word (a shift, four ANDs, four fused multiply-adds
//     whose first operand is the masked code read as an fp16 subnormal), exact while every scale of
//     the wave's unit lies in [2^-10, 2^-4); the weights from the low code position come out
//     divided by 16 and are summed apart;
//   * long, 13 instructions (a shift, four mask-and-or into [1024, 1040), two subtractions, two
//     fused multiply-adds, four multiplications by the scale), exact for every scale; a wave takes
//     it for a unit in which any lane's check of its scales fails.
// (Feeding the raw codes to the matrix unit and scaling each group's fp32 dot product instead
// would need 5 instructions, but leaves out the fp16 rounding of the scaled weights: up to 5e-3
// away from the reference's value at K = 14336, which an fp16 output between 16 and 32 cannot
// absorb inside a max-abs tolerance of 1e-2.)
//
// Work split: unit = (strip of 128 columns) x (group of 128 K).  A wave owns `upw`
// consecutive groups of a strip, the four or eight waves of a workgroup own consecutive
// group ranges, partial sums meet in LDS.  When K is split over several workgroups,
// each output element has a 64-bit word in a zero-initialised accumulator: bits 14..63
// hold the running sum as a fixed-point integer (2^-24 units), bits 7..13 the number of NaN
// contributions, bits 0..6 the number of contributions.  A workgroup adds (value << 14) + 1 with ONE device-scope atomic and
// looks at the returned old word: whoever sees count == splits - 1 was last, owns the
// total (old + own), stores the output and writes the word back to zero.  Integer adds
// commute, so the result does not depend on arrival order, and nobody waits for anyone.
#include <atomic>

#include "common.hpp"
#include "fwht_device.hpp"

namespace uniql {

constexpr int kXsStride = 68;  // dwords per staged activation row: 64 + 4, keeps the 64 lanes on distinct banks

struct StreamArgs {
    const u32x4* B;       // packed weights, [K/16][N/2] 16-byte pieces
    const half_t* S;      // permuted scales [groups][N]
    const half_t* X;      // activations [M][ldx]
    void* D;              // fp16 or fp32 [M][epi.ldd]
    unsigned long long* accum;  // [M][N] fixed-point sum | count words, zero on entry and on exit (splits > 1)
    int64_t ldx;
    int M, N, K;
    int G;                // number of 128-wide K groups = K/128
    int per_column;       // 1: a single scale row (per-column scales)
    int upw;              // groups per wave
    int splits;           // workgroups along K per strip
    int xrows;            // activation rows staged per wave: M rounded up to a multiple of 4
    int k_valid;          // columns of X that exist (multiple of 8); the rest of K counts as zeros
    unsigned x_bytes;     // bytes from X to the end of its last row (< 2 GiB: buffer addressing)
    float had_scale;
    int log2K;            // full-row rotation: K = 2^log2K
    int fwht_lds;         // full-row rotation: dword offset of the rows' fp32 images in LDS
    Epilogue epi;
};

// One launch covers up to 16 rows of X (the rows of one MFMA tile); more rows run as further
// launches over the same weights, which only the forcing flag asks for: from 17 rows on the
// tiled kernel is faster.  RC: row class, an upper bound of M
// (1, 2, 4, 8, 16): it fixes NV, how many of the four output rows of a lane's accumulator
// quad are real, and XQ, how many quads of activation rows are loaded and staged.  WAVES:
// wavefronts per workgroup (4 or 8); with 8 a workgroup can cover all of K for shapes with
// many strips, which removes the exchange of partial sums between workgroups.  EXT: the call
// uses something beyond the plain product (input shorter than K, output cut, strided or fp32, bias,
// gated pairs); the plain instantiation leaves all of that code out, which at a few
// microseconds per launch is measurable (instruction fetch).
// HAD: 0 no rotation; 1 every 128-block of the activations is rotated in registers while it is
// staged (zero extra memory traffic); 2 the rows are rotated as a whole (block = K, a power of
// two): every workgroup transforms the (few) rows once, into fp32 images in LDS, while its first
// weights are on their way, and the staging reads its 128 values from there.  Same butterfly
// order and the same single rounding as the transform kernel: the same values bit for bit.
template <int RC, int HAD, int WAVES, bool EXT>
__global__ __launch_bounds__(64 * WAVES, 2)
void w4a16_stream_kernel(const StreamArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr int NV = RC < 4 ? RC : 4;
    constexpr int XQ = (RC + 3) / 4;
    constexpr int RPW = 4;  // row pairs (32 K values each) per group

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps address math scalar
    const int slot = lane & 15;
    const int kq = lane >> 4;
    const int c8 = slot & 7;

    const int strip = blockIdx.x;
    const int split = blockIdx.y;

    const int N4 = a.N >> 1;  // 16-byte pieces per packed row
    const int g_begin = (split * WAVES + w) * a.upw;
    const int g_end = (g_begin + a.upw < a.G) ? (g_begin + a.upw) : a.G;

    // per-lane offsets inside the strip (32-bit), everything else is uniform
    const uint32_t piece_off = (uint32_t)((slot >> 3) * 32 + 4 * c8 + kq);  // 16-byte pieces
    const uint32_t scale_off = (uint32_t)((slot >> 3) * 64 + 8 * c8);       // halves
    const u32x4* strip_w = a.B + (size_t)strip * 64;
    const half_t* strip_s = a.S + (size_t)strip * 128;

    // acc[jb][v]: output row 4 kq + v, column slot jb of this lane; acc_low collects the products of
    // the weights that the short expansion leaves divided by 16 (see process)
    f4 acc[8], acc_low[8];
#pragma unroll
    for (int jb = 0; jb < 8; ++jb) acc[jb] = acc_low[jb] = f4{0.f, 0.f, 0.f, 0.f};

    uint32_t* xs = lds + (size_t)w * a.xrows * kXsStride;  // this wave's staging rows
    // Staged row layout (dwords): the pair of K values 2d, 2d+1 of the group, d = 32 rq + 8 i + kq' + 4 c
    // (packed row 4 rq + i of the group, K rows 2 kq', 2 kq' + 1 for c = 0 or 2 kq' + 8, 2 kq' + 9 for
    // c = 1), sits at dword 32 rq + 16 c + 4 kq' + i, so that the A operand of lane (row, kq') for
    // the low (c = 0) or high (c = 1) code pairs of the four packed rows of quad rq is one 16-byte read.
    // MFMA row `slot` reads staged row min(slot, xrows - 1): rows past M only feed output rows
    // that are never stored.
    const int xrow_of = (slot < a.xrows ? slot : a.xrows - 1) * kXsStride + 4 * kq;
    // where this lane's staged quad goes: lane `slot` holds pairs d = 4 slot + p, written 4 p apart
    const int stage_off = 32 * (slot >> 3) + 16 * (slot & 1) + ((slot & 7) >> 1);
    NibbleMagic magic;
    magic.init();

    // Everything a group needs from memory, held in registers: two sets, so that the loads of the
    // wave's next group are in flight while the current one is expanded and multiplied (the
    // expansion is about as long as the memory latency it would otherwise leave uncovered).
    struct GroupRegs {
        u32x4 wq[2 * RPW];
        u32x4 sc;
        u32x4 xv[XQ];
    };
    GroupRegs set_a, set_b;
    // Activation rows are read through a buffer descriptor: a lane whose row does not exist (or,
    // with a short input, whose columns do not) uses an offset beyond the descriptor and gets zeros.
    // No branch around a load: the code from the kernel's entry to the first group's loads is one
    // block, so the kernel arguments are fetched together and the loads leave as early as possible.
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.X), 0, a.x_bytes, 0x00020000);
    uint32_t x_off[XQ];
#pragma unroll
    for (int i = 0; i < XQ; ++i) {
        const int m = 4 * i + kq;
        x_off[i] = m < a.M ? (uint32_t)m * (uint32_t)a.ldx * 2u + 16u * (uint32_t)slot : 0x80000000u;
    }
    // activations first (small, they gate the LDS staging), then scales, then the eight packed rows
    auto issue_loads = [&](int g, GroupRegs& r) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XQ; ++i) {
            if (HAD == 2) {  // the rotated rows come from LDS
                r.xv[i] = u32x4{0u, 0u, 0u, 0u};
                continue;
            }
            uint32_t off = x_off[i];
            if (EXT) off = 128 * g + 8 * slot < a.k_valid ? off : 0x80000000u;
            r.xv[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, off, 256u * (uint32_t)g, 0));
        }
        // (one scale row: the load of row 0 is not used, see sc_fixed)
        r.sc = *reinterpret_cast<const u32x4*>(strip_s + (size_t)(a.per_column ? 0 : g) * a.N + scale_off);
        const u32x4* rowp = strip_w + (size_t)(8 * g) * N4;  // uniform
#pragma unroll
        for (int rr = 0; rr < 2 * RPW; ++rr) r.wq[rr] = __builtin_nontemporal_load(rowp + (size_t)rr * N4 + piece_off);
    };

    u32x4 sc_fixed = u32x4{0u, 0u, 0u, 0u};  // one scale per column: the same eight scales for every group
    const int fwht_row_floats = fwht_rows_image_floats(a.K);  // HAD == 2: padded fp32 image of one row
    auto process = [&](const GroupRegs& r, int g) __attribute__((always_inline)) {
        const u32x4 scales = a.per_column ? sc_fixed : r.sc;
        // ---- rotate (optionally) and stage the activations in LDS ------------------
#pragma unroll
        for (int i = 0; i < XQ; ++i) {
            const int mrow = i * 4;
            if (mrow < a.xrows) {  // uniform
                u32x4 v = r.xv[i];
                if (HAD == 2) {
                    v = u32x4{0u, 0u, 0u, 0u};
                    if (mrow + kq < a.M) {
                        const float* src = reinterpret_cast<const float*>(lds + a.fwht_lds) +
                                           (size_t)(mrow + kq) * fwht_row_floats + fwht_pad256(128 * g + 8 * slot);
                        const f4 lo4 = *reinterpret_cast<const f4*>(src), hi4 = *reinterpret_cast<const f4*>(src + 4);
#pragma unroll
                        for (int p = 0; p < 2; ++p) {
                            h2 hv;
                            hv.x = scaled_to_half(lo4[2 * p], a.had_scale);
                            hv.y = scaled_to_half(lo4[2 * p + 1], a.had_scale);
                            v[p] = h2_to_bits(hv);
                            hv.x = scaled_to_half(hi4[2 * p], a.had_scale);
                            hv.y = scaled_to_half(hi4[2 * p + 1], a.had_scale);
                            v[2 + p] = h2_to_bits(hv);
                        }
                    }
                }
                if (HAD == 1) {
                    float f[8];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const h2 hv = bits_to_h2(v[p]);
                        f[2 * p] = (float)hv.x;
                        f[2 * p + 1] = (float)hv.y;
                    }
                    wht128_row16(f, slot);
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        h2 hv;
                        hv.x = scaled_to_half(f[2 * p], a.had_scale);
                        hv.y = scaled_to_half(f[2 * p + 1], a.had_scale);
                        v[p] = h2_to_bits(hv);
                    }
                }
                uint32_t* row = xs + (size_t)(mrow + kq) * kXsStride;
#pragma unroll
                for (int p = 0; p < 4; ++p) row[stage_off + 4 * p] = v[p];
            }
        }
        // LDS operations of one wave complete in issue order: the reads below see
        // the writes above without a workgroup barrier (each wave has its own rows).
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // Quad rq (packed rows 4 rq .. 4 rq + 3 = 64 K values) against the eight column slots
        // jb = 2 j + blk of this lane.  Word j of a packed row holds, for blk 0 and (after >> 8) for
        // blk 1, a LOW code pair (bits 0..3 and 16..19: K rows 2 kq, 2 kq + 1) and a HIGH code pair
        // (bits 4..7 and 20..23: K rows 2 kq + 8, 2 kq + 9).  One MFMA takes the low pairs of the
        // quad's four rows, the next the high pairs; the scale of column slot jb is half jb of the
        // 16-byte scale load.
        //
        // Short expansion.  A code c left where it is, everything else masked away, IS an fp16
        // number: c 2^-20 in the high position, c 2^-24 in the low one (subnormals, exact).  With
        // S = s 2^20 one fused multiply-add gives
        //     high:  fma(c 2^-20, S, -8 s)  = fp16_rn((c - 8) s)
        //     low:   fma(c 2^-24, S, -s/2)  = fp16_rn((c - 8) s / 16) = fp16_rn((c - 8) s) / 16
        // exactly (one rounding of the exact value, as the reference's multiplication makes), PROVIDED
        // S, 8 s and s / 2 are exact and the low form's result is a normal number whenever it is not
        // zero: 2^-10 <= s < 2^-4.  The low pairs' products are summed apart (acc_low) and enter the
        // result times 16 at the end: a power of two, exact in fp32.  9 vector instructions per packed
        // word (a shift, four ANDs, four FMAs) instead of 13.  A lane checks its eight scales; if any
        // lane of the wave finds one outside the range (or zero: padding columns, empty groups), the
        // whole wave expands this unit the long way (mask-and-or into [1024, 1040), subtract, multiply:
        // exact for every scale), into the same accumulators.
        //
        // Range check on both halves of a scale word at once: t = bits - 0x1400 must lie below 0x1800,
        // i.e. neither t nor t + 0x0800 may have one of its three top bits set (a borrow or carry
        // between the halves only happens next to a half that fails anyway)
        uint32_t out_of_range = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t t = scales[j] - 0x14001400u;
            out_of_range |= t | (t + 0x08000800u);
        }
        const bool lane_ok = (out_of_range & 0xE000E000u) == 0;
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(!lane_ok) == 0ull, 1)) {
            h2 s20[4], c_high[4], c_low[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const h2 pr = bits_to_h2(scales[j]);
                s20[j] = bits_to_h2(scales[j] + 0x50005000u);  // exponents + 20 (both are normal and stay in range)
                c_high[j] = pr * h2{(half_t)-8.0f, (half_t)-8.0f};
                c_low[j] = pr * h2{(half_t)-0.5f, (half_t)-0.5f};
            }
#pragma unroll
            for (int rq = 0; rq < RPW / 2; ++rq) {
                const h8 xa_low = __builtin_bit_cast(h8, *reinterpret_cast<const u32x4*>(xs + xrow_of + 32 * rq));
                const h8 xa_high = __builtin_bit_cast(h8, *reinterpret_cast<const u32x4*>(xs + xrow_of + 32 * rq + 16));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
#pragma unroll
                    for (int blk = 0; blk < 2; ++blk) {
                        const h2 sv = blk ? h2{s20[j].y, s20[j].y} : h2{s20[j].x, s20[j].x};
                        const h2 ch = blk ? h2{c_high[j].y, c_high[j].y} : h2{c_high[j].x, c_high[j].x};
                        const h2 cl = blk ? h2{c_low[j].y, c_low[j].y} : h2{c_low[j].x, c_low[j].x};
                        h2 el[4], eh[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t q = r.wq[4 * rq + i][j];
                            const uint32_t pq = blk ? (q >> 8) : q;
                            el[i] = __builtin_elementwise_fma(bits_to_h2(pq & magic.mask_low), sv, cl);
                            eh[i] = __builtin_elementwise_fma(bits_to_h2(pq & magic.mask_high), sv, ch);
                        }
                        const h8 bl = h8{el[0].x, el[0].y, el[1].x, el[1].y, el[2].x, el[2].y, el[3].x, el[3].y};
                        const h8 bh = h8{eh[0].x, eh[0].y, eh[1].x, eh[1].y, eh[2].x, eh[2].y, eh[3].x, eh[3].y};
                        acc_low[2 * j + blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa_low, bl, acc_low[2 * j + blk], 0, 0, 0);
                        acc[2 * j + blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa_high, bh, acc[2 * j + blk], 0, 0, 0);
                    }
                }
            }
        } else {
#pragma unroll
            for (int rq = 0; rq < RPW / 2; ++rq) {
                const h8 xa_low = __builtin_bit_cast(h8, *reinterpret_cast<const u32x4*>(xs + xrow_of + 32 * rq));
                const h8 xa_high = __builtin_bit_cast(h8, *reinterpret_cast<const u32x4*>(xs + xrow_of + 32 * rq + 16));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const h2 pr = bits_to_h2(scales[j]);
#pragma unroll
                    for (int blk = 0; blk < 2; ++blk) {
                        const h2 sv = blk ? h2{pr.y, pr.y} : h2{pr.x, pr.x};
                        h2 el[4], eh[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t q = r.wq[4 * rq + i][j];
                            const uint32_t pq = blk ? (q >> 8) : q;
                            el[i] = magic.pair_low(pq) * sv;
                            eh[i] = magic.pair_high(pq) * sv;
                        }
                        const h8 bl = h8{el[0].x, el[0].y, el[1].x, el[1].y, el[2].x, el[2].y, el[3].x, el[3].y};
                        const h8 bh = h8{eh[0].x, eh[0].y, eh[1].x, eh[1].y, eh[2].x, eh[2].y, eh[3].x, eh[3].y};
                        acc[2 * j + blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa_low, bl, acc[2 * j + blk], 0, 0, 0);
                        acc[2 * j + blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa_high, bh, acc[2 * j + blk], 0, 0, 0);
                    }
                }
            }
        }
        // the next group's staging must not overtake this group's operand reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // Wave-uniform trip counts throughout.  Every process() call sits on a path with a fixed
    // sequence of loads before it, so that the wait the compiler places ahead of the first use
    // of a set leaves exactly the other set's loads outstanding (a process() reached both with
    // and without a prefetch behind it would have to wait for everything).
    // whole-row rotation: this thread's share of the activation rows is requested first (it comes
    // from cache: every workgroup reads the same rows), so that the transform can run while the
    // first weights, requested right behind, are still on their way
    constexpr int kRowChunks = HAD == 2 ? 16384 / 8 / (64 * WAVES) : 1;  // 16-byte chunks of the rows per thread
    u32x4 xin[kRowChunks];
    if (HAD == 2) fwht_rows_load<kRowChunks>(a.X, a.ldx, a.M, a.log2K, tid, 64 * WAVES, xin);
    // the first group's loads leave before anything else is decided (a wave without groups asks
    // for the last group and ignores it)
    issue_loads(g_begin < a.G ? g_begin : a.G - 1, set_a);
    if (a.per_column) {  // uniform, rare
        uint32_t t[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int n0 = strip * 128 + (slot >> 3) * 64 + c8 + 8 * (2 * p), n1 = n0 + 8;
            const uint16_t lo = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n0));
            const uint16_t hi = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n1));
            t[p] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        sc_fixed = u32x4{t[0], t[1], t[2], t[3]};
    }
    if (HAD == 2)  // all waves, also those without groups: the transform has workgroup barriers
        fwht_rows_to_lds<kRowChunks>(xin, reinterpret_cast<float*>(lds + a.fwht_lds), a.M, a.K, a.log2K, tid, 64 * WAVES);
    auto finish = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int jb = 0; jb < 8; ++jb) acc[jb] += acc_low[jb] * 16.0f;
    // The output stage's kernel arguments are fetched here, under the exchange of the partial sums
    // (left to itself the compiler loads each of them in front of its first use: a scalar load and
    // its wait in front of every row's atomic and again in front of its store).
    const int n_splits = a.splits, n_cols = a.N, m_rows = a.M;
    unsigned long long* const accum_base = a.accum;
    void* const d_base = a.D;
    asm volatile("" ::"s"(n_splits), "s"(n_cols), "s"(m_rows), "s"(accum_base), "s"(d_base));
    // ---- combine the waves (fixed order), then the K splits ------------------------------
    // acc[jb][v] on lane l is row m = 4 (l/16) + v, column
    // 128 strip + 64 (slot/8) + 16 (jb/2) + 8 (jb%2) + slot%8.
    // The exchange area follows the staging rows, so no barrier is needed before the first
    // round.
    float* red = reinterpret_cast<float*>(lds + (size_t)WAVES * a.xrows * kXsStride);
    // the exchange area holds 64 rows of 128 floats: all waves at once up to 8 activation rows
    // (the row class fixes both: the staged rows are M rounded up to a multiple of four)
    constexpr int rr_rows = RC <= 4 ? 4 : RC;                            // rows per wave in the exchange area
    constexpr int wpr = 64 / rr_rows < WAVES ? 64 / rr_rows : WAVES;     // waves per round
    constexpr int RPT = WAVES / 2;                  // output rows covered per pass of the workgroup
    constexpr int NI = (RC + RPT - 1) / RPT;        // passes needed for the rows of this row class
    const int ncol_lane = 64 * (slot >> 3) + c8;
    const int col_out = tid & 127;
    const int n_out = 128 * strip + col_out;
    const bool gated = EXT && a.epi.gated != 0;  // uniform
    const int col_pair = col_out ^ 64;    // the other half of a (gate, up) pair
    bool first_round = true;
    float tot[NI], oth[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) tot[i] = oth[i] = 0.f;
    for (int round = 0; round < WAVES / wpr; ++round) {
        if (!first_round) __syncthreads();
        first_round = false;
        // (one condition around all of a lane's writes: rows from M up to the area's rr_rows per wave
        // are written too and never read; a condition per write would put every write behind a branch)
        if (w / wpr == round && 4 * kq < rr_rows) {
#pragma unroll
            for (int jb = 0; jb < 8; ++jb) {
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    const int ml = 4 * kq + v;
                    red[((w % wpr) * rr_rows + ml) * 128 + ncol_lane + 16 * (jb >> 1) + 8 * (jb & 1)] = acc[jb][v];
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int ml = (tid >> 7) + RPT * i;
            if (ml < m_rows) {
#pragma unroll
                for (int ww = 0; ww < wpr; ++ww) {
                    tot[i] += red[(ww * rr_rows + ml) * 128 + col_out];
                    if (gated) oth[i] += red[(ww * rr_rows + ml) * 128 + col_pair];
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int m = (tid >> 7) + RPT * i;
        if (m >= m_rows) continue;
        unsigned long long* word = accum_base + (size_t)m * n_cols + n_out;
        if (!gated) {
            float total = tot[i];
            const bool mine = n_splits == 1 || accum_add(word, tot[i], n_splits, total);
            if (mine) {
                if constexpr (EXT) {
                    finish_store(a.epi, d_base, m, n_out, total);
                } else {  // (fp32 output is one of the extended instantiation's cases)
                    reinterpret_cast<half_t*>(d_base)[(size_t)m * n_cols + n_out] = (half_t)total;
                }
                if (n_splits != 1) accum_reset(word);
            }
        } else if (col_out < 64) {
            const int n_pair = 64 * strip + col_out;
            if (n_splits == 1) {
                finish_store_gated(a.epi, d_base, m, n_pair, tot[i], oth[i]);
            } else {
                float total_g, total_u;
                if (accum_add_pair(word, word + 64, tot[i], oth[i], n_splits, total_g, total_u)) {
                    finish_store_gated(a.epi, d_base, m, n_pair, total_g, total_u);
                    accum_reset(word);
                }
            }
        }
    }
    };

    // The short cases come first in the code: a wave with one or two groups runs through the kernel
    // once, on instructions that arrive from memory as it goes, and should meet them in fetch order.
    if (g_begin + 1 >= g_end) {
        if (g_begin < g_end) process(set_a, g_begin);
        finish();
    } else if (g_begin + 2 >= g_end) {
        issue_loads(g_begin + 1, set_b);
        process(set_a, g_begin);
        process(set_b, g_begin + 1);
        finish();
    } else {
        int g = g_begin;
        while (g + 2 < g_end) {
            issue_loads(g + 1, set_b);
            process(set_a, g);
            issue_loads(g + 2, set_a);
            process(set_b, g + 1);
            g += 2;
        }
        if (g + 1 < g_end) {
            issue_loads(g + 1, set_b);
            process(set_a, g);
            process(set_b, g + 1);
        } else {
            process(set_a, g);
        }
        finish();
    }
}

// ---------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------
static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct StreamPlan {
    int waves;  // 4 or 8
    int upw;    // groups per wave
    int splits;
};

// Heuristic (from sweeps over waves x groups per wave on the Llama, pruned-Llama and Mamba2 shapes
// at 1, 2, 4 and 8 rows):
//   * enough strips to occupy most of the chip on their own (>= 144): one workgroup owns a whole
//     strip, so no partial sums are exchanged between workgroups; four waves with eight groups each
//     when K allows it (long streams per wave, two register sets in flight), else eight waves;
//   * otherwise K is split over workgroups.  One or two rows: as many groups per workgroup as it
//     takes to stay within about 288 workgroups, on 4 waves, or, from four groups per wave on, on 8
//     waves with half as many each (two waves per SIMD cover each other's waits: 14336 -> 4096 at
//     one row 8.2 against 8.6 us).  More rows: every split costs a 64-bit atomic per output element,
//     so 8 waves (4 for small problems: below 1536 units, from 8 rows on below 768) and at most 256
//     workgroups.
static StreamPlan stream_plan(int m, int n, int k, int upw_override, int waves_override) {
    const int nstrips = n / 128, G = k / 128;
    const int64_t units = (int64_t)nstrips * G;
    StreamPlan p;
    const bool whole_strip = m <= 16 && nstrips >= 144 && G >= 16 && G <= 64;
    int max_wgs = 288;
    if (waves_override) {
        p.waves = waves_override;
    } else if (whole_strip) {
        p.waves = G <= 32 ? 4 : 8;
    } else if (m <= 2) {
        p.waves = 4;
    } else {
        p.waves = (m <= 16 && units >= (m >= 8 ? 768 : 1536)) ? 8 : 4;
        max_wgs = 256;
    }
    if (upw_override > 0) {
        p.upw = upw_override;
    } else if (whole_strip && !waves_override) {
        p.upw = ceil_div(G, p.waves);
    } else {
        p.upw = 1;
        while (p.upw < 8 && (int64_t)nstrips * ceil_div(G, p.waves * p.upw) > max_wgs) ++p.upw;
        if (m <= 2 && !waves_override && p.waves == 4 && p.upw >= 4 && p.upw % 2 == 0) {
            p.waves = 8;
            p.upw /= 2;
        }
    }
    p.splits = ceil_div(G, p.waves * p.upw);
    while (p.splits > kAccumMaxSplits) {  // the contribution count has 7 bits
        p.upw *= 2;
        p.splits = ceil_div(G, p.waves * p.upw);
    }
    return p;
}

size_t stream_accum_bytes(int m, int n, int k) {
    // one 64-bit word per output element of a 16-row slab, whenever some plan splits K
    const int G = k / 128;
    if (G <= 4) return 0;
    const int mrows = m < 16 ? m : 16;
    return (size_t)mrows * n * sizeof(unsigned long long);
}

template <int RC, int HAD, int WAVES, bool EXT>
static hipError_t launch_one(StreamArgs a, hipStream_t stream) {
    const size_t stage = (size_t)WAVES * a.xrows * kXsStride * 4;
    constexpr int rr_rows = RC <= 4 ? 4 : RC;  // as in the kernel
    constexpr int wpr = 64 / rr_rows < WAVES ? 64 / rr_rows : WAVES;
    const size_t red = (size_t)wpr * rr_rows * 128 * 4;
    size_t shmem = stage + red;
    if (HAD == 2) {  // one padded fp32 image per activation row behind the staging and exchange areas
        a.fwht_lds = (int)(shmem / 4);
        shmem += (size_t)a.M * (a.K + (a.K >> 5)) * 4;
    }
    auto kern = &w4a16_stream_kernel<RC, HAD, WAVES, EXT>;
    if (shmem > 64 * 1024) {
        static std::atomic<unsigned long long> attribute_set{0};  // a bit per device, once per instantiation
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
        if (!((attribute_set.load(std::memory_order_acquire) >> dev) & 1ull)) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            attribute_set.fetch_or(1ull << dev, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL(kern, dim3(a.N / 128, a.splits), dim3(64 * WAVES), shmem, stream, a);
    return hipGetLastError();
}

template <int RC, int HAD>
static hipError_t launch_waves(const StreamArgs& a, int waves, bool ext, hipStream_t stream) {
    if (waves == 8)
        return ext ? launch_one<RC, HAD, 8, true>(a, stream) : launch_one<RC, HAD, 8, false>(a, stream);
    return ext ? launch_one<RC, HAD, 4, true>(a, stream) : launch_one<RC, HAD, 4, false>(a, stream);
}

template <int HAD>
static hipError_t launch_rows(const StreamArgs& a, int waves, hipStream_t stream) {
    const Epilogue& e = a.epi;
    const bool ext = e.gated || e.bias || e.residual || e.relu2 || e.transpose || e.n_store != a.N ||
                     e.ldd != a.N || a.k_valid != a.K || e.out_f32;
    if (a.M == 1) return launch_waves<1, HAD>(a, waves, ext, stream);
    if (a.M == 2) return launch_waves<2, HAD>(a, waves, ext, stream);
    if (a.M <= 4) return launch_waves<4, HAD>(a, waves, ext, stream);
    if (a.M <= 8) return launch_waves<8, HAD>(a, waves, ext, stream);
    return launch_waves<16, HAD>(a, waves, ext, stream);
}

// the activation rows of a 16-row slab are addressed with 32-bit byte offsets
bool stream_shape_ok(int k, int64_t lda) { return (15 * lda + k) * 2 < ((int64_t)1 << 31); }

// Whether the full-row rotation (block = k) of an m-row call runs inside the streaming kernel:
// k a power of two and the rows' fp32 images (k + k/16 floats each, per 16-row slab) small enough
// to leave room for several workgroups per compute unit.
bool stream_rotates_rows(int m, int k) {
    const int mm = m < 16 ? m : 16;
    return k >= 256 && (k & (k - 1)) == 0 && (int64_t)mm * k <= 16384;
}

// Rows are processed in slabs of at most 16; every slab re-streams the weights.
// had_mode: 0 no rotation, 1 128-blocks, 2 whole rows (stream_rotates_rows must hold, k_valid = k).
// tune: bits 0..7 groups per wave, bits 8..12 waves per workgroup (4 or 8); zero fields mean
// "choose".
int stream_launch(const void* A, int64_t lda, int k_valid, const void* B, const void* S, void* D,
                  const Epilogue& epi, void* accum, int m, int n, int k, int groups, int had_mode, float had_scale,
                  unsigned tune, hipStream_t stream) {
    if (!stream_shape_ok(k, lda)) return UNIQL_E_SHAPE;
    StreamArgs a;
    a.B = reinterpret_cast<const u32x4*>(B);
    a.S = reinterpret_cast<const half_t*>(S);
    a.accum = reinterpret_cast<unsigned long long*>(accum);
    a.ldx = lda;
    a.N = n;
    a.K = k;
    a.G = k / 128;
    a.per_column = (groups == 1) ? 1 : 0;
    a.k_valid = k_valid;
    a.epi = epi;
    a.had_scale = had_scale;
    a.fwht_lds = 0;
    a.log2K = 0;
    while ((1 << a.log2K) < k) ++a.log2K;
    int waves_override = (int)((tune >> 8) & 0x1fu);
    if (waves_override != 4 && waves_override != 8) waves_override = 0;
    const size_t out_elt = epi.out_f32 ? 4 : 2;
    for (int m0 = 0; m0 < m; m0 += 16) {
        const int mm = (m - m0) < 16 ? (m - m0) : 16;
        const StreamPlan plan = stream_plan(mm, n, k, (int)(tune & 0xffu), waves_override);
        a.upw = plan.upw;
        a.splits = plan.splits;
        a.M = mm;
        a.x_bytes = (unsigned)(((int64_t)(mm - 1) * lda + k_valid) * 2);
        a.xrows = ((mm + 3) / 4) * 4;
        a.X = reinterpret_cast<const half_t*>(A) + (size_t)m0 * lda;
        a.D = reinterpret_cast<char*>(D) + (size_t)m0 * (epi.transpose ? 1 : epi.ldd) * out_elt;
        if (epi.residual) a.epi.residual = epi.residual + (size_t)m0 * epi.ldr;
        const hipError_t e = had_mode == 1   ? launch_rows<1>(a, plan.waves, stream)
                             : had_mode == 2 ? launch_rows<2>(a, plan.waves, stream)
                                             : launch_rows<0>(a, plan.waves, stream);
        if (e != hipSuccess) return UNIQL_E_LAUNCH;
    }
    return UNIQL_OK;
}

// ---------------------------------------------------------------------------------
// Measurement aid: what the memory system alone allows for a streaming launch.  Same grid,
// same wave count, same strip / split / group walk and the same 16-byte nontemporal loads of
// packed rows and scales as w4a16_stream_kernel, but the data is only XOR-ed together (36
// instructions per unit) and nothing is staged, expanded, multiplied, reduced or exchanged;
// one dword per wave is stored if the XOR hits a value that random data practically never
// produces, so the loads cannot be dropped.  DEPTH units are requested before the first is
// consumed.
template <int WAVES, int DEPTH>
__global__ __launch_bounds__(64 * WAVES, 2)
void w4a16_read_floor_kernel(const u32x4* B, const half_t* S, int N, int G, int upw, uint32_t* sink) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15, kq = lane >> 4, c8 = slot & 7;
    const int strip = blockIdx.x;
    const int split = blockIdx.y;
    const int N4 = N >> 1;
    const int g_begin = (split * WAVES + w) * upw;
    const int g_end = (g_begin + upw < G) ? (g_begin + upw) : G;
    const uint32_t piece_off = (uint32_t)((slot >> 3) * 32 + 4 * c8 + kq);
    const uint32_t scale_off = (uint32_t)((slot >> 3) * 64 + 8 * c8);
    const u32x4* strip_w = B + (size_t)strip * 64;
    const half_t* strip_s = S + (size_t)strip * 128;
    u32x4 x = u32x4{0u, 0u, 0u, 0u};
    for (int g0 = g_begin; g0 < g_end; g0 += DEPTH) {
        u32x4 wq[DEPTH][8], sc[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int g = g0 + d < g_end ? g0 + d : g_end - 1;  // past the end: the last unit again (depth > 1 only)
            sc[d] = *reinterpret_cast<const u32x4*>(strip_s + (size_t)g * N + scale_off);
            const u32x4* rowp = strip_w + (size_t)(8 * g) * N4;
#pragma unroll
            for (int rr = 0; rr < 8; ++rr) wq[d][rr] = __builtin_nontemporal_load(rowp + (size_t)rr * N4 + piece_off);
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            x ^= sc[d];
#pragma unroll
            for (int rr = 0; rr < 8; ++rr) x ^= wq[d][rr];
        }
    }
    if ((x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u) sink[(blockIdx.y * gridDim.x + blockIdx.x) * WAVES + w] = x[0];
}

template <int WAVES>
static void read_floor_depth(int depth, dim3 grid, hipStream_t stream, const u32x4* B, const half_t* S, int N, int G,
                             int upw, uint32_t* sink) {
    if (depth >= 4)
        hipLaunchKernelGGL((w4a16_read_floor_kernel<WAVES, 4>), grid, dim3(64 * WAVES), 0, stream, B, S, N, G, upw, sink);
    else if (depth >= 2)
        hipLaunchKernelGGL((w4a16_read_floor_kernel<WAVES, 2>), grid, dim3(64 * WAVES), 0, stream, B, S, N, G, upw, sink);
    else
        hipLaunchKernelGGL((w4a16_read_floor_kernel<WAVES, 1>), grid, dim3(64 * WAVES), 0, stream, B, S, N, G, upw, sink);
}

// tune: as stream_launch (bits 0..7 groups per wave, bits 8..12 waves per workgroup), plus bits
// 13..15 the number of units a wave requests before it consumes the first (0 = 1)
int read_floor_launch(const void* B, const void* S, void* sink, int m, int n, int k, unsigned tune, hipStream_t stream) {
    int waves_override = (int)((tune >> 8) & 0x1fu);
    if (waves_override != 4 && waves_override != 8) waves_override = 0;
    const StreamPlan plan = stream_plan(m < 16 ? m : 16, n, k, (int)(tune & 0xffu), waves_override);
    const int depth = (int)((tune >> 13) & 7u);
    const dim3 grid(n / 128, plan.splits);
    if (plan.waves == 8)
        read_floor_depth<8>(depth, grid, stream, reinterpret_cast<const u32x4*>(B), reinterpret_cast<const half_t*>(S), n,
                            k / 128, plan.upw, reinterpret_cast<uint32_t*>(sink));
    else
        read_floor_depth<4>(depth, grid, stream, reinterpret_cast<const u32x4*>(B), reinterpret_cast<const half_t*>(S), n,
                            k / 128, plan.upw, reinterpret_cast<uint32_t*>(sink));
    return hipGetLastError() == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

size_t read_floor_sink_bytes(int m, int n, int k, unsigned tune) {
    int waves_override = (int)((tune >> 8) & 0x1fu);
    if (waves_override != 4 && waves_override != 8) waves_override = 0;
    const StreamPlan plan = stream_plan(m < 16 ? m : 16, n, k, (int)(tune & 0xffu), waves_override);
    return (size_t)(n / 128) * plan.splits * plan.waves * sizeof(uint32_t);
}

}  // namespace uniql
