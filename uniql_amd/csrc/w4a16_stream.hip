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
// Every byte of the 1 KiB row segment is fetched once and eight MFMAs (one per jb)
// consume two packed rows (32 K values) at a time.  The activations are the A operand:
// rows of X (up to 16 per launch) staged through LDS in the same K order.  MFMA is
// used purely as a wide dot-product unit: its cost does not depend on M, so
// M = 1..16 all run at the weight-streaming rate.
//
// Every weight is expanded to the reference's fp16 value fp16_rn((code - 8) * scale)
// (csrc/linear/marlin_gemm_kernel.cuh:118-146) before it enters the matrix unit: 13 vector
// instructions per packed word (one shift, four mask-and-or, two fp16 subtractions, two fp16
// fused multiply-adds, four fp16 multiplications by the scale), all exact except the final
// multiplication, which rounds once as the reference's does.  The products are exact in the
// MFMA and accumulate in fp32, so the result equals the reference's value up to the order of
// the fp32 additions, for every M.  (Feeding the raw codes as fp16 subnormals and scaling each
// group's fp32 dot product instead saves 8 of the 13 instructions, but leaves out the fp16
// rounding of the scaled weights: up to 5e-3 away from the reference's value at K = 14336,
// which an fp16 output between 16 and 32 cannot absorb inside a max-abs tolerance of 1e-2.)
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

    f4 acc[8];  // acc[jb][v]: output row 4 kq + v, column slot jb of this lane
#pragma unroll
    for (int jb = 0; jb < 8; ++jb) acc[jb] = f4{0.f, 0.f, 0.f, 0.f};

    uint32_t* xs = lds + (size_t)w * a.xrows * kXsStride;  // this wave's staging rows
    // Staged row layout (dwords): the pair of K values 2d, 2d+1 of the group, d = 16 rp + kq' + 4 t,
    // sits at dword 16 rp + 4 kq' + t, so that the A operand of lane (row, kq') for row pair rp
    // is one 16-byte read.
    // MFMA row `slot` reads staged row min(slot, xrows - 1): rows past M only feed output rows
    // that are never stored.
    const int xrow_of = (slot < a.xrows ? slot : a.xrows - 1) * kXsStride + 4 * kq;
    // where this lane's staged quad goes: lane `slot` holds pairs d = 4 slot + i
    const int stage_off = 16 * (slot >> 2) + (slot & 3);
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

        // Row pair rp (packed rows 2rp, 2rp+1 = 32 K values) against the eight column slots
        // jb = 2j + blk of this lane: the B operand is the four code pairs of words j of both
        // packed rows (low byte pair for blk 0, after >> 8 for blk 1), expanded and scaled; the
        // scale of column slot jb is half jb of the 16-byte scale load.  Consecutive MFMAs go to
        // different accumulators.
#pragma unroll
        for (int rp = 0; rp < RPW; ++rp) {
            const h8 xa = __builtin_bit_cast(h8, *reinterpret_cast<const u32x4*>(xs + xrow_of + 16 * rp));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t q0 = r.wq[2 * rp][j], q1 = r.wq[2 * rp + 1][j];
                const h2 pr = bits_to_h2(scales[j]);
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const uint32_t p0 = blk ? (q0 >> 8) : q0;
                    const uint32_t p1 = blk ? (q1 >> 8) : q1;
                    const h2 sv = blk ? h2{pr.y, pr.y} : h2{pr.x, pr.x};
                    const h2 e0 = magic.pair_low(p0) * sv, e1 = magic.pair_high(p0) * sv;
                    const h2 e2 = magic.pair_low(p1) * sv, e3 = magic.pair_high(p1) * sv;
                    const h8 bw = h8{e0.x, e0.y, e1.x, e1.y, e2.x, e2.y, e3.x, e3.y};
                    acc[2 * j + blk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, bw, acc[2 * j + blk], 0, 0, 0);
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
            if (ml < a.M) {
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
        if (m >= a.M) continue;
        unsigned long long* word = a.accum + (size_t)m * a.N + n_out;
        if (!gated) {
            float total = tot[i];
            const bool mine = a.splits == 1 || accum_add(word, tot[i], a.splits, total);
            if (mine) {
                if constexpr (EXT) {
                    finish_store(a.epi, a.D, m, n_out, total);
                } else {  // (fp32 output is one of the extended instantiation's cases)
                    reinterpret_cast<half_t*>(a.D)[(size_t)m * a.N + n_out] = (half_t)total;
                }
                if (a.splits != 1) accum_reset(word);
            }
        } else if (col_out < 64) {
            const int n_pair = 64 * strip + col_out;
            if (a.splits == 1) {
                finish_store_gated(a.epi, a.D, m, n_pair, tot[i], oth[i]);
            } else {
                float total_g, total_u;
                if (accum_add_pair(word, word + 64, tot[i], oth[i], a.splits, total_g, total_u)) {
                    finish_store_gated(a.epi, a.D, m, n_pair, total_g, total_u);
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
//   * enough strips to occupy the chip on their own (>= 176): one workgroup owns a whole strip, so
//     no partial sums are exchanged between workgroups; four waves with eight groups each when K
//     allows it (long streams per wave, two register sets in flight), else eight waves;
//   * otherwise K is split over workgroups.  One or two rows: 4 waves, and as many groups per wave
//     as it takes to stay within about 288 workgroups.  More rows: every split costs a 64-bit
//     atomic per output element, so 8 waves (4 for small problems: below 1536 units, from 8 rows on
//     below 768) and at most 256 workgroups.
static StreamPlan stream_plan(int m, int n, int k, int upw_override, int waves_override) {
    const int nstrips = n / 128, G = k / 128;
    const int64_t units = (int64_t)nstrips * G;
    StreamPlan p;
    const bool whole_strip = m <= 16 && nstrips >= 176 && G >= 16 && G <= 64;
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
        // one or two rows and a strip count that lands well below the chip's 256 compute units once
        // the grid is inside the limit (146 strips: 292 workgroups are too many, 146 too few): one
        // group per wave and many short workgroups instead (4096 -> 18688 at one row: 10.5 against 11.3 us)
        if (m <= 2 && p.upw > 1 && (int64_t)nstrips * ceil_div(G, p.waves * p.upw) < 176) p.upw = 1;
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
