// Wide-tile W4A16 kernel for large M (long prefill): D[M,N] = X[M,K] . dequant(B)[K,N].
//
// A workgroup of four wavefronts owns a 256 x 256 output tile; wave (wm, wn) owns the 128 x 128
// quarter (rows 128 wm.., columns 128 wn..) as 4 x 4 accumulators of v_mfma_f32_32x32x16_f16 and
// keeps it for the whole of K, so there is no exchange of partial tiles at the end.  K advances in
// blocks of 32 (two packed rows).  Per block
//   * the X tile (256 rows x 32 K) travels global -> LDS as buffer loads into LDS, two blocks at a
//     time (64 K = whole 128-byte lines of every row, 32 KiB),
//   * the block's codes (2 packed rows x 256 columns, 4 KiB) travel the same way, the scales once
//     per K group,
//   * every weight of the block is expanded to the reference's fp16 value (code - 8) * scale ONCE
//     per workgroup (one thread: the 32 codes of two columns x 16 K) and written to LDS as fp16,
//     16 KiB, in MFMA operand order,
//   * each wave reads 4 weight operands and 4 activation operands (16 bytes per lane each) per
//     16 K and issues 16 MFMAs on them.
// At the end every wave sends its quarter through LDS, 32 rows at a time, to the store code it shares with
// the 128-column kernel (all epilogues of the layer call).
// Against the 128 x 128 tiles of w4a16_tile_kernel (whose four waves split K and expand their own
// weights) a weight is expanded once per 256 rows instead of once per 128, an X element is loaded
// once per 256 columns instead of once per 128, and the weights no longer pass through the vector
// ALU of the wave that multiplies them.  The price is the 256 x 256 granularity: the kernel is
// chosen only where the grid still fills the chip (see wide_preferred).
//
// LDS operand layout.  Weights: element (column x, k) of a block lives in 16-byte unit
// 4 x + ((k / 8) ^ sw(x)); activations: element (row x, k) of a pair of blocks in unit
// 8 x + ((k / 8) ^ sw8(x)).  The XOR swizzles are chosen so that neither an MFMA operand read
// (32 consecutive x, one K eighth per half-wave) nor a 16-byte write of the expansion meets a bank
// conflict (checked with a probe of 16-byte LDS accesses on the hardware).
//
// Pipeline.  Rings: X two slots (a pair of blocks each), codes four slots, scales three slots (one
// per K group), expanded weights two buffers.  Iteration kb multiplies block kb; meanwhile it
// expands the codes of block kb+1 (fetched from LDS into registers during iteration kb-1) into
// the other weight buffer and, after the one barrier of the iteration, reads the first operands
// of block kb+1, fetches the codes of block kb+2 and requests the codes of block kb+5.  The X
// blocks of pair p are requested in two halves: the lower rows behind the barrier of iteration
// 2p-3 (which frees the slot), the upper rows during the first half of iteration 2p-2; they are
// first read behind the barrier of iteration 2p-1.  The loop is unrolled four times (one K
// group), so every ring slot and with it every LDS address is a constant, and the scales are
// requested and fetched once per group.  A wave that has a SIMD to itself issues one instruction
// every four clocks, whatever the instruction: the matrix pipe (32 clocks per MFMA) stays busy
// only while the loop needs fewer than eight instructions per MFMA, so the instruction count is
// what the code is written for (about 4.6 per MFMA).  vmcnt is counted by hand: nothing but the
// loop's own loads uses the counter, and their number and order per iteration are fixed.  The
// last group runs a copy of the loop body that requests nothing but the last upper rows.
#include <atomic>

#include "common.hpp"

namespace uniql {

// ---- the K loop's load schedule, as numbers -------------------------------------------------
// An iteration (one block of 32 K values; J = block index mod 4) issues: in its first half, when J
// is even, the kWideXRowLoads loads of the upper rows of a pair of X blocks; in its second half one
// load of codes, in a group's first iteration (J = 0) one load of scales, and, when J is odd, the
// kWideXRowLoads loads of the lower rows of the next pair.  The issue sites are written with these
// functions' constants and the waits are computed from them.
constexpr int kWideXRowLoads = 4;
constexpr int wide_loads_first_half(int j) { return (j & 1) == 0 ? kWideXRowLoads : 0; }
constexpr int wide_loads_second_half(int j) { return 1 + (j == 0 ? 1 : 0) + ((j & 1) ? kWideXRowLoads : 0); }
constexpr int wide_loads(int j) { return wide_loads_first_half(j) + wide_loads_second_half(j); }
// loads that may still be outstanding at the barrier in the second half of iteration j (see the
// comment at the kernel's `iteration`)
constexpr int wide_vmcnt_at_barrier(int j) {
    return (j & 1) ? wide_loads_second_half((j + 3) & 3)
                   : wide_loads((j + 2) & 3) + wide_loads((j + 3) & 3) + wide_loads_first_half(j);
}

struct WideArgs {
    const u32x4* B;
    const half_t* S;
    const half_t* X;
    void* D;
    int64_t ldx;
    int M, N, K;
    int mblocks;  // ceil(M / 256)
    Epilogue epi;
};

typedef __attribute__((address_space(3))) void* wide_lptr_t;

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding)
#define UNIQL_WIDE_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)
// s_waitcnt lgkmcnt(0) with the other counters left alone
#define UNIQL_WIDE_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

constexpr int kWideXBytes = 256 * 128;  // one X slot: 256 rows x 64 K (a pair of blocks) x 2 bytes
constexpr int kWideCBytes = 4096;       // one block of codes: 4 waves x 1 KiB
constexpr int kWideSBytes = 4096;       // one group's scales: 4 waves x 1 KiB (256 bytes used per wave)
constexpr int kWideWBytes = 256 * 64;   // one block of expanded weights: 256 columns x 32 K x 2 bytes
constexpr int kWideXBase = 0;
constexpr int kWideCBase = kWideXBase + 2 * kWideXBytes;
constexpr int kWideSBase = kWideCBase + 4 * kWideCBytes;
constexpr int kWideWBase = kWideSBase + 3 * kWideSBytes;
constexpr int kWideLdsBytes = kWideWBase + 2 * kWideWBytes;  // 126976

// bit 0 = x2 ^ x4, bit 1 = x2 ^ x5: of the XOR swizzles of this form the one (with a few equals)
// for which a probe of 16-byte LDS accesses showed no extra passes for either access pattern
__device__ __forceinline__ int wide_sw(int x) { return (((x >> 2) ^ (x >> 4)) & 1) | ((((x >> 2) ^ (x >> 5)) & 1) << 1); }

// X rows are 128 bytes (eight 16-byte chunks): chunk c of row x sits at position c ^ sw8(x)
__device__ __forceinline__ int wide_sw8(int x) { return (x >> 1) & 7; }

template <int V>
struct WideInt {
    static constexpr int value = V;
};

__global__ __launch_bounds__(256, 1) void w4a16_wide_kernel(const WideArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    char* const ldsb = reinterpret_cast<char*>(lds);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = w >> 1, wn = w & 1;

    // the M blocks of one column block are neighbours in launch order: they run together and the
    // column block's codes are fetched from memory once
    const int mblock = blockIdx.x % a.mblocks;
    const int nblock = blockIdx.x / a.mblocks;
    const int m0 = mblock * 256, n0 = nblock * 256;
    const int ngroups = a.K >> 7;
    const int N4 = a.N >> 1;  // 16-byte pieces per packed row

    // ---- loads -------------------------------------------------------------------------
    // Every load is a buffer load into LDS: a descriptor (uniform base), a 32-bit lane offset that
    // never changes, and a uniform 32-bit offset that advances with K.  No vector instruction and
    // one scalar addition per advance go into addresses.
    // X: wave w brings rows 64 w .. 64 w + 63 of a pair of blocks (64 K = whole 128-byte lines),
    // 8 rows per operation; lane l lands in unit l of the operation's KiB, i.e. row l / 8,
    // position l % 8, and fetches the K eighth that belongs there.  Rows past M re-read the last
    // row (never stored).
    uint32_t xsrc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = 64 * w + 8 * i + (lane >> 3);
        const int c = (lane & 7) ^ wide_sw8(row);
        const int rc = m0 + row < a.M ? row : a.M - 1 - m0;
        xsrc[i] = (uint32_t)(((size_t)rc * a.ldx + 8 * c) * sizeof(half_t));
    }
    // codes: wave w brings packed row w / 2 of the block, column chunks 2 (w % 2), 2 (w % 2) + 1
    // of the tile: one contiguous KiB, which the same wave expands
    const uint32_t c_lane = 16u * lane;
    // scales of the same 128 columns: lanes 0..15 fetch the 256 bytes, the others repeat them
    const uint32_t s_lane = 16u * (lane & 15);
    const uint32_t c_block_bytes = 16u * (uint32_t)a.N, s_group_bytes = 2u * (uint32_t)a.N;
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.X + (size_t)m0 * a.ldx), 0, 0xffffffffu, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<u32x4*>(a.B + (size_t)(w >> 1) * N4 + (size_t)(n0 / 64 + 2 * (w & 1)) * 32), 0, 0xffffffffu, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t s_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.S + n0 + 128 * (w & 1)), 0, 0xffffffffu, kRsrcFlags);
    // the next pair of X blocks / block of codes / group of scales to request: byte offsets, advanced after use
    uint32_t x_next = 0, c_next = 0, s_next = 0;
    const int wave_x = w * 8192, wave_kib = w * 1024;  // the wave's share of an X slot / of a codes or scales slot

    auto load_x = [&](int slot, int i) __attribute__((always_inline)) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (wide_lptr_t)(ldsb + kWideXBase + slot * kWideXBytes + i * 1024 + wave_x),
                                                 16, xsrc[i], x_next, 0, 0);
    };
    auto load_c = [&](int slot) __attribute__((always_inline)) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(c_rsrc, (wide_lptr_t)(ldsb + kWideCBase + slot * kWideCBytes + wave_kib), 16,
                                                 c_lane, c_next, 0, 0);
    };
    auto load_s = [&](int slot_bytes) __attribute__((always_inline)) {  // slot_bytes: uniform, 0 / 4096 / 8192
        __builtin_amdgcn_raw_ptr_buffer_load_lds(s_rsrc, (wide_lptr_t)(ldsb + kWideSBase + slot_bytes + wave_kib), 16, s_lane,
                                                 s_next, 0, 0);
    };

    // ---- expansion ---------------------------------------------------------------------
    // Lane (cl, c8, j) of wave w takes the four words q = 0..3 at 128 cl + 16 c8 + 4 q + j of the
    // wave's KiB: codes of columns 16 j + 8 blk + c8 (blk = 0, 1) of chunk 2 wn + cl, K values
    // 8 hi + 2 q + lo of packed row w / 2.  Per (blk, hi) that is one 16-byte operand piece
    // (eight consecutive K of one column).
    const int cl = lane >> 5, c8 = (lane >> 2) & 7, j = lane & 3;
    const int code_off = kWideCBase + wave_kib + 4 * (128 * cl + 16 * c8 + j);    // + slot * kWideCBytes + 16 q
    const int scale_off = kWideSBase + wave_kib + 4 * (32 * cl + 4 * c8 + j);     // + slot bytes: halves (blk = 0, 1) at 64 cl + 8 c8 + 2 j
    int wdst[2][2];  // byte offsets of the four pieces in weight buffer 0
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int hi = 0; hi < 2; ++hi) {
            const int col = 64 * (2 * wn + cl) + 16 * j + 8 * blk + c8;
            const int c = 2 * (w >> 1) + hi;
            wdst[blk][hi] = kWideWBase + 16 * (4 * col + (c ^ wide_sw(col)));
        }
    NibbleMagic magic;
    magic.init();
    // The expansion of a block in pieces, so that the loop can spread it between its MFMAs:
    // expand_fetch reads the lane's four words, expand_begin(e) / expand_end(e) make two of the 32
    // values (e = 8 blk + 4 hi + q: word q, column blk, K values 8 hi + 2 q + {0, 1}; begin: the
    // exact code - 8, end: the rounding multiplication by the scale), expand_store(blk, hi) writes
    // one finished operand piece.  begin and end of a piece sit in different slots of the loop: a
    // packed instruction right behind the one it depends on costs an idle issue slot.
    uint32_t word[4], piece[16];
    h2 scale_pair = h2{(half_t)0.f, (half_t)0.f};
    auto expand_fetch = [&](int cslot) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < 4; ++q) word[q] = *reinterpret_cast<const uint32_t*>(ldsb + code_off + cslot * kWideCBytes + 16 * q);
    };
    auto scale_fetch = [&](int slot_bytes) __attribute__((always_inline)) {
        scale_pair = bits_to_h2(*reinterpret_cast<const uint32_t*>(ldsb + scale_off + slot_bytes));
    };
    auto expand_begin = [&](int e) __attribute__((always_inline)) {
        const int blk = e >> 3, hi = (e >> 2) & 1, q = e & 3;
        const uint32_t qq = blk ? (word[q] >> 8) : word[q];
        uint32_t bits = h2_to_bits(hi ? magic.pair_high(qq) : magic.pair_low(qq));
        asm volatile("" : "+v"(bits));  // pins the step to the place in the schedule where it is asked for
        piece[e] = bits;
    };
    auto expand_end = [&](int e) __attribute__((always_inline)) {
        const int blk = e >> 3;
        const h2 sv = blk ? h2{scale_pair.y, scale_pair.y} : h2{scale_pair.x, scale_pair.x};
        uint32_t bits = h2_to_bits(bits_to_h2(piece[e]) * sv);
        asm volatile("" : "+v"(bits));
        piece[e] = bits;
    };
    auto expand_store = [&](int buf, int blk, int hi) __attribute__((always_inline)) {
        const int e = 8 * blk + 4 * hi;
        *reinterpret_cast<u32x4*>(ldsb + wdst[blk][hi] + buf * kWideWBytes) = u32x4{piece[e], piece[e + 1], piece[e + 2], piece[e + 3]};
    };

    // ---- MFMA operands -------------------------------------------------------------------
    // Operand t of K sixteenth s of a block: x = 128 wq + 32 t + r (r = lane % 32), K eighth
    // 2 s + h of the block (h = lane / 32).
    // Weights (64 bytes per column): unit 4 x + ((2 s + h) ^ sw(x)), and sw(x) = sw(r) ^ 2 (t % 2):
    // with u0 = 4 r + (h ^ (sw(r) & 1)) + (sw(r) & 2) the unit is 512 wq + 128 t + ((s ^ t) % 2 ? u0 ^ 2 : u0).
    // Activations (128 bytes per row, block b of the pair): unit 8 x + ((4 b + 2 s + h) ^ sw8(r)).
    const int r = lane & 31, h = lane >> 5;
    const int swr = wide_sw(r);
    const int u0 = 4 * r + (h ^ (swr & 1)) + (swr & 2);
    int xrd[4], wrd[2];  // byte offsets in X slot 0 (index 2 b + s) / weight buffer 0
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) xrd[c2] = kWideXBase + 16 * (1024 * wm + 8 * r + ((2 * c2 + h) ^ wide_sw8(r)));
    wrd[0] = kWideWBase + 16 * (512 * wn + u0);
    wrd[1] = kWideWBase + 16 * (512 * wn + (u0 ^ 2));

    f16 acc[4][4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mt][nt][v] = 0.f;

    h8 xa[2][4], bw[2][4];
    // the i-th of the eight operand reads of a half, in the order the MFMAs want them: the
    // first weight operand, the four activation operands, the other three weight operands
    // kblock: the block's number modulo 4 (its pair's X slot is kblock / 2, its half of the pair kblock % 2)
    auto read_operand = [&](int set, int kblock, int wbuf, int s, int i) __attribute__((always_inline)) {
        if (i >= 1 && i <= 4) {
            const int t = i - 1;
            xa[set][t] = *reinterpret_cast<const h8*>(ldsb + xrd[2 * (kblock & 1) + s] + (kblock >> 1) * kWideXBytes + 4096 * t);
        } else {
            const int t = i == 0 ? 0 : i - 4;
            bw[set][t] = *reinterpret_cast<const h8*>(ldsb + wrd[(s ^ t) & 1] + wbuf * kWideWBytes + 2048 * t);
        }
    };

    // ---- prologue: the loads the iterations before the first would have issued, block 0 expanded ---
    int s_issue_bytes = 0;  // scales ring slot (as a byte offset) of the next group to request
    int s_fetch_bytes = 0;  //                                      of the next group to fetch
    auto advance3 = [&](int& slot_bytes) __attribute__((always_inline)) {
        slot_bytes = slot_bytes == 2 * kWideSBytes ? 0 : slot_bytes + kWideSBytes;
    };
    load_c(0);
    c_next += c_block_bytes;
    load_c(1);
    c_next += c_block_bytes;
    // (the kernel runs on at least two groups; s_next never points past the last one)
    load_s(s_issue_bytes);
    s_next += s_group_bytes;
    advance3(s_issue_bytes);
    load_s(s_issue_bytes);
    if (ngroups > 2) s_next += s_group_bytes;
    advance3(s_issue_bytes);
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x(0, i);
    load_c(2);
    c_next += c_block_bytes;
#pragma unroll
    for (int i = 4; i < 8; ++i) load_x(0, i);
    x_next += 128;
    load_c(3);
    c_next += c_block_bytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x(1, i);
    UNIQL_WIDE_WAIT_VMCNT(5);  // all but the last five: codes 0..2, both groups of scales, the first pair of X blocks
    __builtin_amdgcn_s_barrier();
    expand_fetch(0);
    scale_fetch(s_fetch_bytes);
    advance3(s_fetch_bytes);
#pragma unroll
    for (int e = 0; e < 16; ++e) expand_begin(e);
#pragma unroll
    for (int e = 0; e < 16; ++e) expand_end(e);
#pragma unroll
    for (int e = 0; e < 4; ++e) expand_store(0, e >> 1, e & 1);
    expand_fetch(1);
    UNIQL_WIDE_WAIT_LGKM0();  // the words of block 0 are in registers: their slot may take block 4
    load_c(0);
    c_next += c_block_bytes;
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) read_operand(0, 0, 0, 0, i);

    uint32_t c_step = c_block_bytes;  // how far the codes offset moves after an iteration
    // ---- one iteration; J = kb % 4 is a constant --------------------------------------------
    // One MFMA per slot, issued first; what else a slot does (in the matrix pipe's shadow) is
    // fixed by hand and closed by a scheduling barrier.
    // kVm: how many loads may still be outstanding at the barrier, i.e. how many were issued after
    // the youngest one that must have landed.  Behind an odd iteration's barrier the first block
    // of the next pair is read: its upper rows were the last request of the previous iteration's
    // first half, followed only by that iteration's second half (codes, and scales in a group's
    // first iteration).  Behind an even iteration's barrier the codes of block kb+2 are fetched:
    // the last request of iteration kb-3, followed by everything iterations kb-2 and kb-1 issue and
    // this iteration's first half.  The counts below are the SAME constants that the issue sites
    // are written with (loops over kXRowLoads, one load_c per iteration, load_s in iteration 0),
    // so a load added there changes the wait here; the static_assert states the table the
    // pipeline was validated with.
    auto iteration = [&](auto jc, auto tailc) __attribute__((always_inline)) {
        constexpr int J = decltype(jc)::value;
        constexpr bool kTail = decltype(tailc)::value != 0;
        constexpr int kVm = kTail && J != 0 ? 0 : wide_vmcnt_at_barrier(J);
        static_assert(wide_vmcnt_at_barrier(0) == 14 && wide_vmcnt_at_barrier(1) == 2 && wide_vmcnt_at_barrier(2) == 15 &&
                          wide_vmcnt_at_barrier(3) == 1,
                      "the load schedule changed: re-derive and re-validate the waits of the K loop");
        constexpr int wbuf = J & 1, wbuf_next = (J + 1) & 1;
        // first half: K values 0..15 of block kb with operand set 0.  Meanwhile the second
        // half's operands are read and block kb+1 is expanded into the other weight buffer.
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int nt = i >> 2, mt = i & 3;
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bw[0][nt], xa[0][mt], acc[mt][nt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (i < 8) read_operand(1, J, wbuf, 1, i);
            expand_begin(i);
            if (i > 0) expand_end(i - 1);
            if (i == 5) expand_store(wbuf_next, 0, 0);
            if (i == 9) expand_store(wbuf_next, 0, 1);
            if (i == 13) expand_store(wbuf_next, 1, 0);
            // an even iteration requests the upper rows of the pair of X blocks whose lower rows the
            // iteration before has requested (the last group's first iteration included)
            if ((J & 1) == 0 && (!kTail || J == 0)) {
#pragma unroll
                for (int q = 0; q < kWideXRowLoads; ++q)
                    if (i == 8 + 2 * q) load_x(((J + 2) >> 1) & 1, kWideXRowLoads + q);
                if (i == 15) x_next += 128;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // second half: K values 16..31 with operand set 1.  At the barrier the expanded
        // weights of block kb+1 are written and everybody has read what the loads issued behind
        // the barrier will overwrite.  Then: the next block's first operands, the words of block
        // kb+2 (and, where that block starts a group, the group's scales), this iteration's loads.
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int nt = i >> 2, mt = i & 3;
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bw[1][nt], xa[1][mt], acc[mt][nt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (i == 0) expand_end(15);
            if (i == 1) expand_store(wbuf_next, 1, 1);
            if (i == 4) {
                UNIQL_WIDE_WAIT_LGKM0();
                UNIQL_WIDE_WAIT_VMCNT(kVm);
                __builtin_amdgcn_s_barrier();
            }
            if (i >= 5 && i < 13) read_operand(0, (J + 1) & 3, wbuf_next, 0, i - 5);
            if (i == 13) {
                expand_fetch((J + 2) & 3);
                if (J == 2) {
                    scale_fetch(s_fetch_bytes);
                    advance3(s_fetch_bytes);
                }
            }
            if (!kTail) {
                if (J == 0 && i == 5) {
                    load_s(s_issue_bytes);
                    advance3(s_issue_bytes);
                }
                if ((J & 1) == 1) {  // the lower rows of the pair after next, into the slot this barrier has freed
#pragma unroll
                    for (int q = 0; q < kWideXRowLoads; ++q)
                        if (i == 6 + 2 * q) load_x(((J + 3) >> 1) & 1, q);
                }
                if (i == 14) load_c((J + 1) & 3);
                if (i == 15) c_next += c_step;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // groups 0 .. ngroups-2 request what lies four and five blocks ahead (the scales two groups
    // ahead: the last such request asks for the last group again); the last group requests nothing
    for (int g = 0; g < ngroups - 1; ++g) {
        iteration(WideInt<0>{}, WideInt<0>{});
        if (g + 3 < ngroups) s_next += s_group_bytes;
        iteration(WideInt<1>{}, WideInt<0>{});
        // block kb + 5 of the last two iterations before the last group does not exist: they ask
        // for the last block again (into a slot nobody reads any more)
        if (g + 2 == ngroups) c_step = 0;
        iteration(WideInt<2>{}, WideInt<0>{});
        iteration(WideInt<3>{}, WideInt<0>{});
    }
    iteration(WideInt<0>{}, WideInt<1>{});
    iteration(WideInt<1>{}, WideInt<1>{});
    iteration(WideInt<2>{}, WideInt<1>{});
    iteration(WideInt<3>{}, WideInt<1>{});
    UNIQL_WIDE_WAIT_VMCNT(0);

    // ---- store: acc[mt][nt][4 q + i] on lane l is row 128 wm + 32 mt + l % 32, column
    // 128 wn + 32 nt + 8 q + 4 (l / 32) + i of the tile (the weights are the MFMA's first operand).
    // The lane's coordinates are derived again behind the loop (the empty asm keeps the compiler
    // from computing the store addresses in front of it, where they would cost registers the loop needs).
    int lane_s = lane;
    asm volatile("" : "+v"(lane_s));
    const int rs = lane_s & 31, hs = lane_s >> 5;
    // (written with constant indices throughout: a loop the compiler declines to unroll would
    // index the accumulators at run time and so move them from registers to memory, for the whole kernel)
    auto four_times = [&](auto&& f) __attribute__((always_inline)) {
        f(WideInt<0>{});
        f(WideInt<1>{});
        f(WideInt<2>{});
        f(WideInt<3>{});
    };
    // The wave's quarter goes through LDS, 32 rows at a time, and leaves it as (row, 8 consecutive
    // columns) units through the same store code as the 128-column kernel, in a loop: 16 lanes write
    // 256 contiguous bytes of an output row.  (Straight from the registers a store instruction
    // writes 16 bytes to each of 32 rows, 1-2.5 % of a launch slower even for the plain product, and
    // the epilogue's cases would be instantiated once per accumulator quad, 64 times: several
    // hundred KB of code that every compute unit fetches once per launch, 8 to 34 % of a launch
    // at 1024 to 4096 rows.)
    __builtin_amdgcn_s_barrier();  // every wave has read its last operands: their LDS is free
    constexpr int kStride = 132;   // floats per staged row
    float* const stage = reinterpret_cast<float*>(ldsb) + (size_t)w * 32 * kStride;  // this wave's 32 x 128 block
    const bool gated = a.epi.gated != 0;  // uniform: columns c and c + 64 of the wave's strip are a (gate, up) pair
    four_times([&](auto mtc) __attribute__((always_inline)) {
        constexpr int mt = decltype(mtc)::value;
        four_times([&](auto ntc) __attribute__((always_inline)) {
            constexpr int nt = decltype(ntc)::value;
            four_times([&](auto qc) __attribute__((always_inline)) {
                constexpr int q = decltype(qc)::value;
                const f16& t = acc[mt][nt];
                *reinterpret_cast<f4*>(stage + rs * kStride + 32 * nt + 8 * q + 4 * hs) =
                    f4{t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
            });
        });
        // LDS operations of one wave complete in issue order: the reads below see the writes above
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int mrow = m0 + 128 * wm + 32 * mt;
        if (!gated) {
#pragma clang loop unroll(disable)
            for (int u = 0; u < 8; ++u) {
                const int unit = 64 * u + lane_s, row = unit >> 4, c0 = (unit & 15) * 8;
                const float* src = stage + row * kStride + c0;
                const f4 lo = *reinterpret_cast<const f4*>(src), hi = *reinterpret_cast<const f4*>(src + 4);
                if (mrow + row < a.M) store_eight(a.epi, a.D, mrow + row, n0 + 128 * wn + c0, lo, hi);
            }
        } else {
#pragma clang loop unroll(disable)
            for (int u = 0; u < 4; ++u) {
                const int unit = 64 * u + lane_s, row = unit >> 3, c0 = (unit & 7) * 8;
                const float* src = stage + row * kStride + c0;
                const f4 glo = *reinterpret_cast<const f4*>(src), ghi = *reinterpret_cast<const f4*>(src + 4);
                const f4 ulo = *reinterpret_cast<const f4*>(src + 64), uhi = *reinterpret_cast<const f4*>(src + 68);
                if (mrow + row < a.M) store_eight_gated(a.epi, a.D, mrow + row, (n0 + 128 * wn) / 2 + c0, glo, ghi, ulo, uhi);
            }
        }
        // the next 32 rows overwrite the block: not before these reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    });
}

// ---------------------------------------------------------------------------------
// Whether wide_launch can take the call at all: grouped scales, whole 256-column blocks, at
// least two K groups (the pipeline's prologue), 32-bit byte offsets into the X tile (256 rows of
// ldx elements) and into the packed weights.
bool wide_shape_ok(int m, int n, int k, int groups, int64_t ldx) {
    return m > 0 && n % 256 == 0 && k % 128 == 0 && k >= 256 && groups == k / 128 &&
           (255 * ldx + k) * 2 < (1LL << 32) && (int64_t)k * n / 2 < (1LL << 32) &&
           (int64_t)(n / 256) * ((m + 255) / 256) <= 0x7fffffffLL;
}

// Whether the entry point sends a call of the tiled path here.  tune: the tiled kernel's fields;
// 8 in its "row tiles of 32 per workgroup" field (bits 8..11) asks for this kernel, any other
// non-zero value there for the 128 x 128 one.
// Without a forced choice: measured on the Llama and Mamba2 shapes at 256 to 8192 rows, the
// 256 x 256 tiles win (by 5 to 30 %) where their grid keeps the chip busy: the share of real
// output in the tile slots of its rounds of 256 workgroups is at least 0.62.
bool wide_preferred(int m, int n, int k, unsigned tune) {
    if (m <= 0 || n % 256 != 0 || k % 128 != 0 || k < 256) return false;
    const int mt = (int)((tune >> 8) & 0xfu);
    if (mt != 0) return mt == 8;
    if ((tune & 0xffu) != 0 || ((tune >> 12) & 3u) != 0) return false;  // forced K splits or quartets: the 128 x 128 kernel's
    const int64_t tiles = (int64_t)(n / 256) * ((m + 255) / 256);
    const int64_t rounds = (tiles + 255) / 256;
    return (double)m * n / 65536.0 >= 0.62 * 256.0 * (double)rounds;
}

static hipError_t wide_launch_one(const WideArgs& a, int grid, hipStream_t stream) {
    auto kern = &w4a16_wide_kernel;
    static std::atomic<unsigned long long> done{0};  // the attribute is set once per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
    if (dev < 0 || dev >= 64 || !((done.load(std::memory_order_relaxed) >> dev) & 1ull)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kWideLdsBytes);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), kWideLdsBytes, stream, a);
    return hipGetLastError();
}

int wide_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, const Epilogue& epi, int m, int n,
                int k, int groups, hipStream_t stream) {
    if (!wide_shape_ok(m, n, k, groups, lda)) return UNIQL_E_SHAPE;
    WideArgs a;
    a.B = reinterpret_cast<const u32x4*>(B);
    a.S = reinterpret_cast<const half_t*>(S);
    a.X = reinterpret_cast<const half_t*>(A);
    a.D = D;
    a.ldx = lda;
    a.M = m;
    a.N = n;
    a.K = k;
    a.mblocks = (m + 255) / 256;
    a.epi = epi;
    const int grid = (n / 256) * a.mblocks;
    const hipError_t e = wide_launch_one(a, grid, stream);
    return e == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
