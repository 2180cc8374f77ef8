// Tiled W4A16 kernel for M > 16 (prefill): D[M,N] = X[M,K] . dequant(B)[K,N].
//
// A workgroup of four wavefronts owns a (32 MT) x 128 output tile (MT = 1, 2 or 4) and a
// range of 128-wide K groups.  The four waves split K: of the eight packed rows (16 K
// values each) of a group, wave w takes rows w and w + 4 and accumulates the WHOLE tile
// for them with v_mfma_f32_32x32x16_f16, so every weight of the tile is expanded to fp16
// (code-8)*scale exactly once per workgroup.  The partial tiles of the four waves are
// added through LDS at the end.
//
// Operand layout.  A 16-byte piece (c8, kq) of a packed row holds, in 32-bit word j,
// K rows {2kq, 2kq+1, 2kq+8, 2kq+9} of columns 16j + c8 and 16j + 8 + c8.  Lane
//     l = s + 32 h,  s = c8 + 8 ch + 16 jl      (ch: 64-column chunk of the strip)
// reads words 2jl, 2jl+1 of the pieces kq = 2h and 2h+1 and builds four weight operands
// (jo, blk): column 64 ch + 16 (2jl + jo) + 8 blk + c8, K values {4h..4h+3, 4h+8..4h+11}
// (called B operands below).  The activation operand of a 32-row M tile (called A operand) is
// row l % 32 of X with the same eight K values (two 8-byte LDS reads).  The MFMA gets the
// weights as its first source and the activations as its second: the product comes out
// transposed, which gives every lane four consecutive output columns per register quad.
//
// Everything a group needs travels global -> LDS with global_load_lds_dwordx4 (no staging
// registers) into a ring of three stages; the loads of group g+3 are issued during the second
// half of group g, into the slot group g has just left, and the operands of group g+1 are read
// from LDS into a second register set
// during the second half of group g.  A stage holds
//   * the X tile, 256 bytes per row, unpadded: 16-byte segment sg of row r sits at position
//     sg ^ (r % 16);
//   * per wave, its two packed rows of the strip (2 x 1 KiB): piece (c8, ch, kq) at position
//     c8 + 8 ch + 16 kq, so a half-wave's 8-byte reads sweep all 64 banks;
//   * the 256 bytes of scales of the strip (four copies, one per quarter-wave; every wave
//     writes all of them with the same values).
// vmcnt is counted by hand: every stage issues exactly kStageOps LDS-DMA operations per
// wave and nothing else uses the counter inside the loop.
//
// When K is also split over workgroups every workgroup writes its fp32 partial tile to a scratch
// area and the last one to arrive (one arrival count per tile) adds them in split order.
#include <atomic>

#include "common.hpp"

namespace uniql {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kRing = 3;

struct TileArgs {
    const u32x4* B;
    const half_t* S;
    const half_t* X;
    void* D;
    unsigned long long* accum;  // one arrival count per output tile (splits > 1), zero on entry and exit
    float* part;                // [tile][split][32 MT][128] partial tiles (splits > 1), any contents
    int64_t ldx;
    int M, N, K;
    int G;            // K / 128
    int per_column;
    int gps;          // K groups per split
    int splits;
    int mblocks;      // ceil(M / (32 MT))
    Epilogue epi;
};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// 16 bytes per lane from a buffer (descriptor + lane offset + uniform offset) straight into LDS
// (64 lanes fill one contiguous KiB at `dst`)
__device__ __forceinline__ void buffer_to_lds16(__amdgpu_buffer_rsrc_t rsrc, uint32_t* dst, uint32_t lane_bytes, uint32_t uniform_bytes) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lptr_t)dst, 16, lane_bytes, uniform_bytes, 0, 0);
}

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding)
#define UNIQL_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)

// Eight fp32 partial sums to / from a workgroup's slot of the split-K scratch area: relaxed
// device-scope accesses (write-through stores, loads that do not trust a stale cache line), so
// workgroups on different XCDs exchange them without flushing or invalidating a whole L2.  The
// four 8-byte words of a unit lie `stride` words apart: word i of all threads of the workgroup is
// one contiguous run, so every store instruction writes whole cache lines.
__device__ __forceinline__ unsigned long long pack_floats(float a, float b) {
    return (unsigned long long)__float_as_uint(a) | ((unsigned long long)__float_as_uint(b) << 32);
}
__device__ __forceinline__ void store_partial(unsigned long long* d, int stride, f4 lo, f4 hi) {
    __hip_atomic_store(d, pack_floats(lo[0], lo[1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d + stride, pack_floats(lo[2], lo[3]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d + 2 * stride, pack_floats(hi[0], hi[1]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d + 3 * stride, pack_floats(hi[2], hi[3]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void add_partial(const unsigned long long* p, int stride, f4& lo, f4& hi) {
    unsigned long long w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = __hip_atomic_load(p + i * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    lo[0] += __uint_as_float((uint32_t)w[0]);
    lo[1] += __uint_as_float((uint32_t)(w[0] >> 32));
    lo[2] += __uint_as_float((uint32_t)w[1]);
    lo[3] += __uint_as_float((uint32_t)(w[1] >> 32));
    hi[0] += __uint_as_float((uint32_t)w[2]);
    hi[1] += __uint_as_float((uint32_t)(w[2] >> 32));
    hi[2] += __uint_as_float((uint32_t)w[3]);
    hi[3] += __uint_as_float((uint32_t)(w[3] >> 32));
}

template <int MT, int KW = 1>
struct TileLds {
    static constexpr int kRows = 32 * MT;
    static constexpr int kXDwords = kRows * 64;        // X tile
    static constexpr int kBDwords = 4 * 2 * 256;       // 4 waves x 2 packed rows x 1 KiB
    static constexpr int kSDwords = 256;               // 4 copies of the strip's 256 bytes of scales
    static constexpr int kStageDwords = kXDwords + kBDwords + kSDwords;
    static constexpr size_t kRingBytes = (size_t)KW * kRing * kStageDwords * 4;  // one ring per wave quartet
    static constexpr size_t kRedBytes = (size_t)KW * 4 * 32 * 132 * 4;  // every wave's 32-row M tile, fp32, padded rows
    static constexpr size_t kBytes = kRingBytes > kRedBytes ? kRingBytes : kRedBytes;
};

// EXT: the call uses something beyond the plain product (output cut or strided, bias, gated
// pairs); the plain instantiation leaves that code out of the epilogue.
// KW: quartets of waves per workgroup (1 or 2).  With two, the quartets take alternate K groups of
// the same tile (each with its own LDS ring): two waves per SIMD cover each other's LDS and
// expansion latencies, which is what small M tiles (little matrix work per group) lack when the
// grid only gives a compute unit one workgroup.
template <int MT, bool EXT, int KW>
__global__ __launch_bounds__(256 * KW, 1) void w4a16_tile_kernel(const TileArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds_all[];
    using L = TileLds<MT, KW>;
    constexpr int ROWS = L::kRows;
    constexpr int kXOps = ROWS / 16;        // X DMA instructions per wave and stage (4 rows each)
    constexpr int kStageOps = kXOps + 3;    // + two packed rows + scales

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int w = w8 & 3;      // role inside the quartet: packed rows w and w + 4 of a group
    const int par = w8 >> 2;   // quartet: takes K groups par, par + KW, ... of the workgroup's range
    uint32_t* lds = lds_all + par * (kRing * L::kStageDwords);  // this quartet's ring
    // MFMA view of the lane
    const int s = lane & 31;
    const int h = lane >> 5;
    const int c8 = s & 7;
    const int ch = (s >> 3) & 1;
    const int jl = s >> 4;
    // DMA view of the lane (16 lanes per X row; piece gather for the packed rows)
    const int dslot = lane & 15;
    const int dkq = lane >> 4;

    // tile coordinates: strips vary fastest so that neighbouring workgroups share X rows
    const int nstrips = a.N >> 7;
    int id = blockIdx.x;
    const int strip = id % nstrips;
    id /= nstrips;
    const int mblock = id % a.mblocks;
    const int split = id / a.mblocks;
    const int m0 = mblock * ROWS;

    const int N4 = a.N >> 1;
    const int g_first = split * a.gps;
    const int g_end = (g_first + a.gps < a.G) ? (g_first + a.gps) : a.G;
    const int g_begin = g_first + par;
    const int ngroups = (g_end - g_first) / KW;  // per quartet; the plan makes the range a multiple of KW

    // packed rows w and w + 4 of every group; DMA lane (c8', ch', kq') fetches piece 32 ch' + 4 c8' + kq'
    const uint32_t piece_off = (uint32_t)((dslot >> 3) * 32 + 4 * (dslot & 7) + dkq);
    const u32x4* strip_w = a.B + (size_t)strip * 64 + (size_t)w * N4;  // uniform; the lane adds piece_off
    // scales: lanes 0..15 fetch the 16 pieces (8 halves each) of the strip's 128 columns
    const half_t* strip_s = a.S + (size_t)strip * 128;  // uniform; the lane adds 8 * dslot
    const int scale_row_stride = a.per_column ? 0 : a.N;  // per-column mode re-reads row 0 (unused)

    // X tile: wave w brings rows [kXOps 4 w, kXOps 4 (w+1)); one DMA instruction covers 4 rows
    // (64 lanes x 16 bytes, contiguous in LDS).  Lane l lands at row l/16, position l%16, so
    // it must fetch segment (l % 16) ^ (row % 16) of its row.
    // byte offsets from the tile's first row, X + m0 ldx + 128 g (uniform, 64-bit): scalar base +
    // 32-bit lane offset addressing; the host keeps 128 ldx below 2^31 elements
    uint32_t xsrc[kXOps];
    const half_t* x_tile = a.X + (size_t)m0 * a.ldx;
#pragma unroll
    for (int i = 0; i < kXOps; ++i) {
        const int row = kXOps * 4 * w + 4 * i + dkq;
        const int seg = dslot ^ (row & 15);
        const int rc = m0 + row < a.M ? row : a.M - 1 - m0;  // rows past M re-read the last row: never stored
        xsrc[i] = (uint32_t)(((size_t)rc * a.ldx + 8 * seg) * sizeof(half_t));
    }

    NibbleMagic magic;
    magic.init();

    f16 acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int op = 0; op < 4; ++op)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mt][op][v] = 0.f;

    // per-column scales do not depend on the group: fetch them once, into registers
    u32x2 sc_fixed = u32x2{0u, 0u};
    if (a.per_column) {
        uint32_t t[2];
#pragma unroll
        for (int jo = 0; jo < 2; ++jo) {
            const int n0 = strip * 128 + 64 * ch + 16 * (2 * jl + jo) + c8, n1 = n0 + 8;
            const uint16_t lo = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n0));
            const uint16_t hi = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n1));
            t[jo] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        sc_fixed = u32x2{t[0], t[1]};
        UNIQL_WAIT_VMCNT(0);  // keep the hand count below exact: nothing of this stays outstanding
    }

    // One of the kStageOps LDS-DMA operations that bring group g into ring slot `ring`:
    // idx < kXOps: four X rows; kXOps, kXOps + 1: the two packed rows; kXOps + 2: scales.
    // The operations of a stage are spread between the MFMA blocks of the previous stage, so
    // the wave never sits behind a full address queue (the tile needs ~60% of the CU's
    // 64 B/clk vector-memory path).
    // Every load is a buffer load into LDS: a descriptor (uniform base), a 32-bit lane offset that
    // never changes and a uniform 32-bit offset that depends on the group, so that no vector
    // instruction goes into an address (the host keeps the packed weights below 4 GiB).
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x_tile), 0, 0xffffffffu, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4*>(strip_w), 0, 0xffffffffu, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(strip_s), 0, 0xffffffffu, kRsrcFlags);
    const uint32_t piece_bytes = 16u * piece_off, scale_lane_bytes = 16u * (uint32_t)dslot;
    const uint32_t packed_row_bytes = 16u * (uint32_t)N4, scale_row_bytes = 2u * (uint32_t)scale_row_stride;
    auto issue_piece = [&](int g, int ring, int idx) __attribute__((always_inline)) {
        uint32_t* stage = lds + ring * L::kStageDwords;
        if (idx < kXOps) {
            uint32_t* xbuf = stage + (kXOps * 4 * w) * 64;  // this wave's X rows
            buffer_to_lds16(x_rsrc, xbuf + idx * 256, xsrc[idx], 256u * (uint32_t)g);
        } else if (idx < kXOps + 2) {
            uint32_t* bbuf = stage + L::kXDwords + w * 512 + (idx - kXOps) * 256;
            buffer_to_lds16(w_rsrc, bbuf, piece_bytes, (uint32_t)(8 * g + 4 * (idx - kXOps)) * packed_row_bytes);
        } else {
            // scales of the group (row 0 in per-column mode, unused then)
            // all 64 lanes of all four waves take part (a predicated load would split the loop
            // body into several scheduling regions): every quarter-wave fetches the same 256
            // bytes, and the four waves write the same values to the same place
            uint32_t* sbuf = stage + L::kXDwords + L::kBDwords;
            buffer_to_lds16(s_rsrc, sbuf, scale_lane_bytes, (uint32_t)g * scale_row_bytes);
        }
    };
    auto issue_stage = [&](int g, int ring) __attribute__((always_inline)) {
#pragma unroll
        for (int idx = 0; idx < kStageOps; ++idx) issue_piece(g, ring, idx);
    };

    // LDS read offsets (dwords).  X: row s of an M tile, packed row w + 4 t -> segments
    // 2 (w + 4t) and 2 (w + 4t) + 1, K half h = dwords 2h, 2h+1 of the segment.
    int xoff[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int x = 0; x < 2; ++x) xoff[t][x] = s * 64 + (((2 * (w + 4 * t) + x) ^ (s & 15)) << 2) + 2 * h;
    const int boff = (c8 + 8 * ch + 32 * h) * 4 + 2 * jl;  // piece kq = 2h, words 2jl, 2jl+1; kq = 2h+1 is 64 dwords on
    const int soff = (8 * ch + c8) * 4 + 2 * jl;

    // Operands in registers.  pw[set][t][0/1]: the packed words (pieces kq = 2h, 2h+1) of packed
    // row w + 4t; scv[set]: the lane's four scales; two sets because the next stage's words are
    // read while the current ones are still being expanded.  xa0 / xa1: A operands of the two
    // packed rows for every M tile (one set each: xa0 is dead after the first half of a stage
    // and is refilled for the next stage during the second half).
    u32x2 pw[2][2][2];   // set 0: stage being multiplied, set 1: the next one (copied over at the end)
    u32x2 scv[2];
    h8 xa0[MT], xa1[MT];
    auto read_words = [&](int set, int ring) __attribute__((always_inline)) {
        const uint32_t* stage = lds + ring * L::kStageDwords;
        const uint32_t* bbuf = stage + L::kXDwords + w * 512;
        const u32x2 sc_lds = *reinterpret_cast<const u32x2*>(stage + L::kXDwords + L::kBDwords + soff);
        scv[set] = a.per_column ? sc_fixed : sc_lds;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            pw[set][t][0] = *reinterpret_cast<const u32x2*>(bbuf + t * 256 + boff);
            pw[set][t][1] = *reinterpret_cast<const u32x2*>(bbuf + t * 256 + boff + 64);
        }
    };
    auto read_xa = [&](h8 (&xa)[MT], int ring, int t) __attribute__((always_inline)) {
        const uint32_t* stage = lds + ring * L::kStageDwords;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const u32x2 lo = *reinterpret_cast<const u32x2*>(stage + mt * 2048 + xoff[t][0]);
            const u32x2 hi = *reinterpret_cast<const u32x2*>(stage + mt * 2048 + xoff[t][1]);
            const h2 d0 = bits_to_h2(lo.x), d1 = bits_to_h2(lo.y), d2 = bits_to_h2(hi.x), d3 = bits_to_h2(hi.y);
            xa[mt] = h8{d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
        }
    };
    // One quarter (two of the eight values) of B operand `block` = 4 t + 2 jo + blk of a stage.
    // K order of the operand: 4h, 4h+1 | 4h+2, 4h+3 | 4h+8, 4h+9 | 4h+10, 4h+11, i.e. quarter
    // q = 0, 1: low-nibble form of pieces kq = 2h, 2h+1; q = 2, 3: high-nibble form.
    auto expand_quarter = [&](int set, int block, int q) __attribute__((always_inline)) -> h2 {
        const int t = block >> 2, jo = (block >> 1) & 1, blk = block & 1;
        const h2 pr = bits_to_h2(scv[set][jo]);
        const uint32_t word = pw[set][t][q & 1][jo];
        const uint32_t qq = blk ? (word >> 8) : word;
        const h2 sv = blk ? h2{pr.y, pr.y} : h2{pr.x, pr.x};
        return (q < 2 ? magic.pair_low(qq) : magic.pair_high(qq)) * sv;
    };
    auto expand = [&](int set, int block) __attribute__((always_inline)) -> h8 {
        const h2 e0 = expand_quarter(set, block, 0), e1 = expand_quarter(set, block, 1);
        const h2 e2 = expand_quarter(set, block, 2), e3 = expand_quarter(set, block, 3);
        return h8{e0.x, e0.y, e1.x, e1.y, e2.x, e2.y, e3.x, e3.y};
    };
    // Four of the eight blocks of a stage (2 packed rows x 4 B operands, MT MFMAs each), written
    // as 4 MT slots: one MFMA, the share of the NEXT block's expansion that fits its shadow
    // (4 / MT quarters), at most one LDS-DMA load (pieces dma_first.. of group next_g, one every
    // kDmaStride slots: the four waves together must not outrun the compute unit's address
    // path, or they stall at issue and the matrix pipe starves) and the LDS reads the caller
    // assigns to the slot.  A scheduling barrier closes every slot: with one wave
    // per SIMD nothing else fills the matrix pipe's shadow, so the order is fixed by hand.
    auto half_stage = [&](int t, h8 (&xa)[MT], h8& bw, int dma_first, int dma_count, int next_g, int next_ring, auto&& lds_reads) __attribute__((always_inline)) {
        constexpr int kDmaStride = MT == 1 ? 1 : 2;  // slots between two LDS-DMA loads
#pragma unroll
        for (int op = 0; op < 4; ++op) {
            const int block = 4 * t + op;
            const int nset = block < 7 ? 0 : 1, nblock = block < 7 ? block + 1 : 0;
            h2 e[4];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int slot_i = op * MT + mt;
                acc[mt][op] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bw, xa[mt], acc[mt][op], 0, 0, 0);
#pragma unroll
                for (int q = mt * (4 / MT); q < (mt + 1) * (4 / MT); ++q) {
                    // the empty asm pins the quarter to this slot: it cannot sink below the slot's
                    // closing barrier
                    uint32_t bits = h2_to_bits(expand_quarter(nset, nblock, q));
                    asm volatile("" : "+v"(bits));
                    e[q] = bits_to_h2(bits);
                }
                if (slot_i % kDmaStride == 0 && slot_i / kDmaStride < dma_count)
                    issue_piece(next_g, next_ring, dma_first + slot_i / kDmaStride);
                lds_reads(slot_i);
                if (MT == 4) {
                    // inside the slot: the first two operations of the quarter, the MFMA, the rest;
                    // the MFMA between the fp16 add and the dependent multiply fills the wait
                    // state that would otherwise cost an s_nop
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            bw = h8{e[0].x, e[0].y, e[1].x, e[1].y, e[2].x, e[2].y, e[3].x, e[3].y};
        }
    };

    // ---- software pipeline over the K groups ----------------------------------------------
    // Iteration `it` multiplies stage `it`.  First half: packed row w (A operands xa0), while
    // the A operands of packed row w+4 are read from LDS: after that nothing of stage `it` is
    // left in LDS that anybody needs.  Middle: the wave waits for stage it+1 (only the kStageOps
    // loads issued since may remain outstanding) and the workgroup meets at a barrier.  Second
    // half: packed row w+4 (xa1), while the words, scales and first-row A operands of stage it+1
    // are read from LDS.  The LDS-DMA loads of a stage are spread over a whole iteration: the
    // first kDmaA pieces of stage it+3 go out in the second half of iteration it (into the
    // slot stage `it` has just left), the rest in the first half of iteration it+1.  So the
    // address path sees an even load, a piece has more than an iteration to land, and the matrix
    // pipe never waits for the barrier or for LDS.  Past the end the "next" group is the last
    // one again (loaded into a slot nobody reads): no branches in the loop body and constant
    // vmcnt arithmetic.
    constexpr int kDmaA = (kStageOps + 1) / 2, kDmaB = kStageOps - kDmaA;
    // every wait below counts kStageOps loads per stage: that holds only while each half stage has an
    // issue slot for every piece handed to it (4 MT slots, one piece every second slot from MT = 2 on)
    constexpr int kDmaSlots = MT == 1 ? 4 : 2 * MT;
    static_assert(kDmaA <= kDmaSlots && kDmaB <= kDmaSlots,
                  "a half stage has fewer issue slots than LDS-DMA pieces: the vmcnt waits would lose count");
    auto group_or_last = [&](int g) __attribute__((always_inline)) { return g < g_end ? g : g_end - 1; };
    auto read_xa_one = [&](h8 (&xa)[MT], int ring, int t, int mt) __attribute__((always_inline)) {
        const uint32_t* stage = lds + ring * L::kStageDwords;
        const u32x2 lo = *reinterpret_cast<const u32x2*>(stage + mt * 2048 + xoff[t][0]);
        const u32x2 hi = *reinterpret_cast<const u32x2*>(stage + mt * 2048 + xoff[t][1]);
        const h2 d0 = bits_to_h2(lo.x), d1 = bits_to_h2(lo.y), d2 = bits_to_h2(hi.x), d3 = bits_to_h2(hi.y);
        xa[mt] = h8{d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
    };
    const int g_last = g_end - 1;
    h8 bw;
    if (ngroups > 0) {
        issue_stage(g_begin, 0);
        issue_stage(ngroups > 1 ? g_begin + KW : g_last, 1);
#pragma unroll
        for (int idx = 0; idx < kDmaA; ++idx) issue_piece(group_or_last(g_begin + 2 * KW), 2, idx);
        UNIQL_WAIT_VMCNT(kStageOps + kDmaA);
        __builtin_amdgcn_s_barrier();
        read_words(0, 0);
        read_xa(xa0, 0, 0);
        bw = expand(0, 0);
    }
    // one iteration; called with a literal `slot` the ring addresses are constants
    auto iteration = [&](int it, int slot) __attribute__((always_inline)) {
        const int slot_next = slot + 1 == kRing ? 0 : slot + 1;
        const int slot_prev = slot == 0 ? kRing - 1 : slot - 1;   // holds stage it+2
        half_stage(0, xa0, bw, kDmaA, kDmaB, group_or_last(g_begin + KW * (it + 2)), slot_prev, [&](int i) __attribute__((always_inline)) {
            if (i < MT) read_xa_one(xa1, slot, 1, i);
        });
        UNIQL_WAIT_VMCNT(kStageOps);   // stage it+1 has landed; only stage it+2's loads are outstanding
        __builtin_amdgcn_s_barrier();
        half_stage(1, xa1, bw, 0, kDmaA, group_or_last(g_begin + KW * (it + 3)), slot, [&](int i) __attribute__((always_inline)) {
            if (i == 0) read_words(1, slot_next);
            if (i >= 1 && i <= MT) read_xa_one(xa0, slot_next, 0, i - 1);
        });
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            pw[0][t][0] = pw[1][t][0];
            pw[0][t][1] = pw[1][t][1];
        }
        scv[0] = scv[1];
    };
    // three iterations at a time walk the ring once: every LDS address in them is a constant
    int it = 0;
    for (; it + kRing <= ngroups; it += kRing) {
        iteration(it, 0);
        iteration(it + 1, 1);
        iteration(it + 2, 2);
    }
    for (int slot = 0; it < ngroups; ++it, ++slot) iteration(it, slot);
    UNIQL_WAIT_VMCNT(0);
    __syncthreads();

    // ---- add the four waves' partial tiles, one 32-row M tile at a time ---------------------
    // The MFMAs take the weights as their first operand, so the accumulators hold the tile
    // transposed: acc[mt][2 jo + blk][4 j4 + i] on lane l is row 32 mt + l % 32 of the tile and
    // column 64 (j4 % 2) + 16 (2 (j4 / 2) + jo) + 8 blk + 4 h + i of the strip, i.e. four
    // consecutive columns per group of four registers: one 16-byte LDS write each.  Every wave
    // writes its partial tile to LDS (row stride 132 floats); then each thread adds the four
    // partials of two (row, 8 consecutive columns) units and stores each unit with one 16-byte
    // store.
    constexpr int kRedStride = 132;
    float* red = reinterpret_cast<float*>(lds_all);  // [4 KW waves][32 rows][132]
    constexpr int NW = 4 * KW;
    const bool split_k = a.splits > 1;
    const bool gated = EXT && a.epi.gated != 0;  // uniform

    // one finished unit: eight consecutive columns c0.. of output row m
    auto emit = [&](int m, int c0, f4 lo, f4 hi) {
        if constexpr (EXT) {
            store_eight(a.epi, a.D, m, 128 * strip + c0, lo, hi);
        } else {
            const size_t o = (size_t)m * a.N + 128 * strip + c0;
            if (a.epi.out_f32) {
                float* d = reinterpret_cast<float*>(a.D) + o;
                *reinterpret_cast<f4*>(d) = lo;
                *reinterpret_cast<f4*>(d + 4) = hi;
            } else {
                const h2 r0 = h2{(half_t)lo[0], (half_t)lo[1]}, r1 = h2{(half_t)lo[2], (half_t)lo[3]};
                const h2 r2 = h2{(half_t)hi[0], (half_t)hi[1]}, r3 = h2{(half_t)hi[2], (half_t)hi[3]};
                *reinterpret_cast<u32x4*>(reinterpret_cast<half_t*>(a.D) + o) =
                    u32x4{h2_to_bits(r0), h2_to_bits(r1), h2_to_bits(r2), h2_to_bits(r3)};
            }
        }
    };

    // K split over workgroups: every workgroup writes its 32 MT x 128 partial tile (fp32) to its
    // slot of the scratch area, then counts itself in the tile's word; whoever completes the count
    // adds the slots in split order (so the sum does not depend on who came last) and stores.
    // A slot holds the tile as 512 MT units of (row, 8 columns); unit u of M tile mt (row u / 16,
    // columns 8 (u % 16)..) is the four words ((mt UPT + u / T) 4 + i) T + u % T, i = 0..3, with
    // T the workgroup's thread count: the thread that reduces a unit writes it, lane after lane.
    const int tile = mblock * nstrips + strip;
    constexpr int T = 256 * KW, UPT = 512 / T, kSlotWords = ROWS * 64;
    unsigned long long* part_tile =
        split_k ? reinterpret_cast<unsigned long long*>(a.part) + (size_t)tile * a.splits * kSlotWords : nullptr;
    unsigned long long* part_mine = split_k ? part_tile + (size_t)split * kSlotWords : nullptr;
    auto unit_word = [&](int mt, int unit) { return ((mt * UPT + unit / T) * 4) * T + unit % T; };
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (m0 + mt * 32 < a.M) {  // uniform
            if (mt > 0) __syncthreads();
            {
                float* wred = red + w8 * 32 * kRedStride + s * kRedStride + 4 * h;
#pragma unroll
                for (int op = 0; op < 4; ++op)
#pragma unroll
                    for (int j4 = 0; j4 < 4; ++j4)
                        *reinterpret_cast<f4*>(wred + 64 * (j4 & 1) + 32 * (j4 >> 1) + 16 * (op >> 1) + 8 * (op & 1)) =
                            f4{acc[mt][op][4 * j4], acc[mt][op][4 * j4 + 1], acc[mt][op][4 * j4 + 2], acc[mt][op][4 * j4 + 3]};
            }
            __syncthreads();
            // gated and not split: the 32 x 64 output block is 256 units, one per thread (columns
            // c0 and c0 + 64 of the strip); else 512 units, two per thread
            const bool pairs_now = gated && !split_k;
            const int units = pairs_now ? 256 : 512;
            for (int unit = tid; unit < units; unit += 256 * KW) {
                const int row = pairs_now ? unit >> 3 : unit >> 4;
                const int c0 = pairs_now ? (unit & 7) * 8 : (unit & 15) * 8;
                const int m = m0 + mt * 32 + row;
                const float* src = red + row * kRedStride + c0;
                f4 lo = *reinterpret_cast<const f4*>(src), hi = *reinterpret_cast<const f4*>(src + 4);
#pragma unroll
                for (int ww = 1; ww < NW; ++ww) {
                    lo += *reinterpret_cast<const f4*>(src + ww * 32 * kRedStride);
                    hi += *reinterpret_cast<const f4*>(src + ww * 32 * kRedStride + 4);
                }
                if (split_k) {
                    if (m < a.M) store_partial(part_mine + unit_word(mt, unit), T, lo, hi);  // (1) rows that exist only
                } else if (!gated) {
                    if (m < a.M) emit(m, c0, lo, hi);
                } else {
                    f4 ulo = *reinterpret_cast<const f4*>(src + 64), uhi = *reinterpret_cast<const f4*>(src + 68);
#pragma unroll
                    for (int ww = 1; ww < NW; ++ww) {
                        ulo += *reinterpret_cast<const f4*>(src + ww * 32 * kRedStride + 64);
                        uhi += *reinterpret_cast<const f4*>(src + ww * 32 * kRedStride + 68);
                    }
                    if (m < a.M) store_eight_gated(a.epi, a.D, m, 64 * strip + c0, lo, hi, ulo, uhi);
                }
            }
        }
    }
    if (!split_k) return;  // uniform

    // ---- the split-K exchange: message passing with relaxed device-scope operations only -------
    // What it relies on, step by step (the numbers are used again at the lines they govern):
    //  (1) store_partial: relaxed agent-scope stores.  On gfx950 these are write-through (sc1)
    //      stores that bypass the XCD's own L2, so a workgroup on another XCD can see them.
    //  (2) s_waitcnt vmcnt(0): the counter is decremented when such a store has been ACKNOWLEDGED
    //      by the memory side, i.e. is visible to every XCD.  A workgroup barrier alone does not
    //      wait for outstanding stores: without this wait the arrival count below overtook the
    //      partial tile in 8 of 130 000 randomised cases (tests/test_gpu_soak.py replays their seeds).
    //  (3) the workgroup barrier: every thread's (2) is behind it.
    //  (4) thread 0's relaxed agent-scope fetch_add on the tile's arrival count; nothing may move
    //      it in front of (3) (the barrier is a compiler and hardware ordering point for it).
    //  (5) the workgroup that completes the count reads the slots with relaxed agent-scope loads
    //      (add_partial; sc1: they do not hit a stale line of the local L2).
    // The language's memory model would ask for a release at (4) and an acquire before (5); at
    // agent scope those compile to a write-back and an invalidate of the whole L2, measured at two
    // to three times the K loop the split saves.  (2), which the ISA documents for vmcnt, stands in
    // for the release; (5)'s cache-bypassing loads for the acquire.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (2)
    __syncthreads();                                   // (3)
    int* last_flag = reinterpret_cast<int*>(lds_all);
    if (tid == 0) {
        const unsigned long long old =
            __hip_atomic_fetch_add(a.accum + tile, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // (4)
        *last_flag = (int)old == a.splits - 1;
    }
    __syncthreads();
    if (*last_flag == 0) return;  // uniform
    const int units = gated ? 256 : 512;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (m0 + mt * 32 >= a.M) break;  // uniform
        for (int unit = tid; unit < units; unit += 256 * KW) {
            const int row = gated ? unit >> 3 : unit >> 4;
            const int c0 = gated ? (unit & 7) * 8 : (unit & 15) * 8;
            const int m = m0 + mt * 32 + row;
            if (m >= a.M) continue;
            // the unit's number in the writers' enumeration (16 units per row); a gated pair's up
            // half is 8 units on
            const int wunit = row * 16 + (c0 >> 3);
            const unsigned long long* src = part_tile + unit_word(mt, wunit);
            const unsigned long long* usrc = part_tile + unit_word(mt, wunit + 8);
            f4 lo = f4{0.f, 0.f, 0.f, 0.f}, hi = lo, ulo = lo, uhi = lo;
            for (int sp = 0; sp < a.splits; ++sp) {
                add_partial(src + (size_t)sp * kSlotWords, T, lo, hi);  // (5)
                if (gated) add_partial(usrc + (size_t)sp * kSlotWords, T, ulo, uhi);
            }
            if (!gated) emit(m, c0, lo, hi);
            else store_eight_gated(a.epi, a.D, m, 64 * strip + c0, lo, hi, ulo, uhi);
        }
    }
    if (tid == 0) __hip_atomic_store(a.accum + tile, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------
static inline int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

struct TilePlan {
    int mtiles, splits, gps;
    int quartets;  // wave quartets per workgroup (1 or 2)
};
static TilePlan tile_plan(int m, int n, int k, int splits_override, int mt_override = 0, int kw_override = 0);

static TilePlan tile_plan_tuned(int m, int n, int k, unsigned tune) {
    return tile_plan(m, n, k, (int)(tune & 0xffu), (int)((tune >> 8) & 0xfu), (int)((tune >> 12) & 0x3u));
}

// What a plan that splits K over workgroups needs (tune: the same fields as tile_launch takes):
// one arrival count per output tile in `accum` (zero on entry, zero again on exit) and one fp32
// partial tile per (tile, split) in a scratch area whose contents do not matter.
size_t tile_accum_bytes(int m, int n, int k, unsigned tune) {
    const TilePlan plan = tile_plan_tuned(m, n, k, tune);
    if (plan.splits <= 1) return 0;
    return (size_t)(n / 128) * ceil_div_i(m, 32 * plan.mtiles) * sizeof(unsigned long long);
}
size_t tile_part_bytes(int m, int n, int k, unsigned tune) {
    const TilePlan plan = tile_plan_tuned(m, n, k, tune);
    if (plan.splits <= 1) return 0;
    const size_t tiles = (size_t)(n / 128) * ceil_div_i(m, 32 * plan.mtiles);
    return tiles * plan.splits * (32 * plan.mtiles * 128) * sizeof(float);
}

// Measured on MI355X, in units of the time one MT = 4 workgroup takes for its K loop when every
// compute unit has one ("a round"):
//   * MT = 4: one workgroup per compute unit, every started round of 256 costs 1;
//   * MT = 2: two workgroups share a compute unit; a full round of 512 costs 1.08 (every weight
//     is expanded twice per 128 rows), a last round of at most 256 costs 0.85;
//   * MT = 1: up to four share a compute unit: 0.62 for at most 256 workgroups, 0.88 for at most
//     512, 1.62 per started round of 1024;
//   * a grid that gives a compute unit at most one MT = 1 or MT = 2 workgroup runs faster with two
//     wave quartets per workgroup (factors 0.85 and 0.92);
//   * K split over workgroups: every workgroup writes its fp32 partial tile to scratch memory and
//     the last one to arrive adds them (about 1 to 1.5 us per MB of partial tiles).
// So: the MT with the cheapest grid; K splits while the grid stays within one workgroup per compute
// unit and the partial tiles stay small against the weights; two quartets whenever the final
// grid has at most 256 workgroups of MT <= 2 and every workgroup gets an even number of groups.
static TilePlan tile_plan(int m, int n, int k, int splits_override, int mt_override, int kw_override) {
    TilePlan p;
    const int strips = n / 128, G = k / 128;
    const bool even_g = G % 2 == 0;
    const int64_t t4 = (int64_t)strips * ceil_div_i(m, 128), t2 = (int64_t)strips * ceil_div_i(m, 64);
    const int64_t t1 = (int64_t)strips * ceil_div_i(m, 32);
    const double cost4 = (double)((t4 + 255) / 256);
    const int64_t rem2 = t2 % 512;
    double cost2 = 1.08 * (double)(t2 / 512) + (rem2 == 0 ? 0.0 : (rem2 <= 256 ? 0.85 : 1.08));
    double cost1 = t1 <= 256 ? 0.62 : (t1 <= 512 ? 0.88 : 1.62 * (double)((t1 + 1023) / 1024));
    if (even_g && t2 <= 256) cost2 *= 0.92;
    if (even_g && t1 <= 256) cost1 *= 0.85;
    p.mtiles = 4;
    if (cost2 < cost4 && cost2 <= cost1) p.mtiles = 2;
    else if (cost1 < cost4) p.mtiles = 1;
    if (m <= 32) p.mtiles = 1;
    // a long K loop over few 64-row tiles: two K splits of 64-row tiles beat 32-row tiles (every
    // weight is expanded for twice the rows; down_proj at M = 256: 545 -> 650 TFLOP/s)
    if (p.mtiles == 1 && G >= 64 && m >= 64 && t2 <= 128) p.mtiles = 2;
    if (mt_override == 1 || mt_override == 2 || mt_override == 4) p.mtiles = mt_override;
    const int64_t tiles = (int64_t)strips * ceil_div_i(m, 32 * p.mtiles);
    int splits = 1;
    if (splits_override > 0) {
        splits = splits_override;
    } else {
        // K splits while the grid stays within one workgroup per compute unit, every workgroup
        // keeps at least 8 groups, and the partial tiles (m x n x 4 bytes per split, written and
        // read once) stay below a quarter of the packed weights the launch streams
        while (tiles * (2 * splits) <= 256 && G / (2 * splits) >= 8 && (int64_t)(2 * splits) * m * 16 <= k) splits *= 2;
    }
    if (splits > G) splits = G;
    if (splits > 255) splits = 255;
    p.gps = ceil_div_i(G, splits);
    p.splits = ceil_div_i(G, p.gps);
    // two quartets take alternate groups: every workgroup's range must hold an even number
    p.quartets = 1;
    const bool want2 = kw_override == 2 || (kw_override == 0 && tiles * p.splits <= 256);
    if (want2 && p.mtiles <= 2 && even_g) {
        const int gps2 = p.gps + (p.gps & 1);
        if (splits_override == 0 || gps2 == p.gps) {
            p.gps = gps2;
            p.splits = ceil_div_i(G, p.gps);
            p.quartets = 2;
        }
    }
    return p;
}

// Whether tile_launch can take the call: grid size, and the 32-bit offsets of the loads (128 rows of
// ldx elements, 2 bytes each, and the packed weights must stay below 2^32 bytes).  Checked by the entry point
// before anything is enqueued.
bool tile_shape_ok(int m, int n, int k, int64_t ldx, unsigned tune) {
    const TilePlan plan = tile_plan_tuned(m, n, k, tune);
    const int64_t grid = (int64_t)(n / 128) * ceil_div_i(m, 32 * plan.mtiles) * plan.splits;
    return grid <= 0x7fffffffLL && ldx < (1LL << 24) && (int64_t)k * n / 2 < (1LL << 32);
}

template <int MT, bool EXT, int KW>
static hipError_t tile_launch_one(const TileArgs& a, int grid, hipStream_t stream) {
    const size_t shmem = TileLds<MT, KW>::kBytes;
    auto kern = &w4a16_tile_kernel<MT, EXT, KW>;
    if (shmem > 64 * 1024) {
        // the attribute is a property of (instantiation, device): set it on the first launch there
        static std::atomic<unsigned long long> done{0};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return hipErrorInvalidDevice;
        if (dev < 0 || dev >= 64 || !((done.load(std::memory_order_relaxed) >> dev) & 1ull)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
            if (e != hipSuccess) return e;
            if (dev >= 0 && dev < 64) done.fetch_or(1ull << dev, std::memory_order_relaxed);
        }
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256 * KW), shmem, stream, a);
    return hipGetLastError();
}

template <int MT, int KW>
static hipError_t tile_launch_ext(const TileArgs& a, bool ext, int grid, hipStream_t stream) {
    return ext ? tile_launch_one<MT, true, KW>(a, grid, stream) : tile_launch_one<MT, false, KW>(a, grid, stream);
}

// tune: bits 0..7 force the number of K splits, bits 8..11 the number of 32-row M tiles per
// workgroup, bits 12..13 the number of wave quartets (0 = choose)
int tile_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, const Epilogue& epi, void* accum,
                size_t accum_bytes, void* part, size_t part_bytes, int m, int n, int k, int groups, unsigned tune,
                hipStream_t stream) {
    const TilePlan plan = tile_plan_tuned(m, n, k, tune);
    if (plan.splits > 1 && (!accum || accum_bytes < tile_accum_bytes(m, n, k, tune) || !part ||
                            part_bytes < tile_part_bytes(m, n, k, tune)))
        return UNIQL_E_WORKSPACE;
    TileArgs a;
    a.part = reinterpret_cast<float*>(part);
    a.B = reinterpret_cast<const u32x4*>(B);
    a.S = reinterpret_cast<const half_t*>(S);
    a.X = reinterpret_cast<const half_t*>(A);
    a.D = D;
    a.accum = reinterpret_cast<unsigned long long*>(accum);
    a.ldx = lda;
    a.M = m;
    a.N = n;
    a.K = k;
    a.G = k / 128;
    a.per_column = (groups == 1) ? 1 : 0;
    a.gps = plan.gps;
    a.splits = plan.splits;
    a.mblocks = ceil_div_i(m, 32 * plan.mtiles);
    a.epi = epi;
    const int64_t grid = (int64_t)(n / 128) * a.mblocks * a.splits;
    if (grid > 0x7fffffffLL) return UNIQL_E_SHAPE;
    hipError_t e;
    const bool ext = epi.gated || epi.bias || epi.residual || epi.relu2 || epi.transpose || epi.n_store != n ||
                     epi.ldd != n || !epi.vec_ok;
    if (plan.mtiles == 1)
        e = plan.quartets == 2 ? tile_launch_ext<1, 2>(a, ext, (int)grid, stream) : tile_launch_ext<1, 1>(a, ext, (int)grid, stream);
    else if (plan.mtiles == 2)
        e = plan.quartets == 2 ? tile_launch_ext<2, 2>(a, ext, (int)grid, stream) : tile_launch_ext<2, 1>(a, ext, (int)grid, stream);
    else
        e = tile_launch_ext<4, 1>(a, ext, (int)grid, stream);
    return e == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
