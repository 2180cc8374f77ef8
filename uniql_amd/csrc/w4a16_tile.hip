// Tiled W4A16 kernel for M > 16 (prefill): D[M,N] = X[M,K] . dequant(B)[K,N].
//
// A workgroup of four wavefronts owns a (16 MTILES) x 128 output tile and a range of
// 128-wide K groups.  The packed weights never touch LDS: as in the streaming kernel,
// each wave fetches 16-byte pieces in the lane order that makes the registers the B
// operand of v_mfma_f32_16x16x32_f16 (lane = column slot + 16 * K quarter), expands them
// to fp16 (code-8)*scale in registers and feeds MFMA directly.  The four waves split
// every K group between them (wave w takes the two packed rows 2w, 2w+1 = 32 K values),
// so every weight of the tile is expanded exactly once per workgroup.
//
// The activations are the A operand.  The X tile of a K group (rows x 128 halves) is
// loaded by the whole workgroup with coalesced 16-byte loads into LDS (double buffered,
// row stride 68 dwords so that the 64 lanes of an operand read hit 64 distinct banks);
// each wave reads the 32-K slice it needs for all its 16-row M tiles.  Global loads
// for group g+1 (X tile, packed rows, scales) are issued before the MFMAs of group g.
//
// At the end the four waves' accumulators meet in LDS.  When K is also split over
// workgroups (grid.z > 1) the tile goes through the same 64-bit fixed-point
// sum|count words as the streaming kernel.
#include "common.hpp"

namespace uniql {

constexpr int kTileXsStride = 68;            // dwords per staged X row (64 + 4)
constexpr float kTileAccumScale = 16777216.0f;  // 2^24
constexpr float kTileAccumClamp = 4194304.0f;   // 2^22

struct TileArgs {
    const u32x4* B;
    const half_t* S;
    const half_t* X;
    void* D;
    unsigned long long* accum;  // [M][N] sum|count words (splits > 1), zero on entry and exit
    int64_t ldx;
    int M, N, K;
    int G;            // K / 128
    int per_column;
    int gps;          // K groups per split
    int splits;
    int mblocks;      // ceil(M / (16 MTILES))
    int out_f32;
};

template <int MTILES>
__global__ __launch_bounds__(256, 1) void w4a16_tile_kernel(const TileArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[];
    constexpr int ROWS = 16 * MTILES;
    constexpr int BUF_DWORDS = ROWS * kTileXsStride;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot = lane & 15;
    const int kq = lane >> 4;
    const int c8 = slot & 7;

    // tile coordinates: strips vary fastest so that neighbouring workgroups share X rows
    const int nstrips = a.N >> 7;
    int id = blockIdx.x;
    const int strip = id % nstrips;
    id /= nstrips;
    const int mblock = id % a.mblocks;
    const int split = id / a.mblocks;
    const int m0 = mblock * ROWS;

    const int N4 = a.N >> 1;
    const int g_begin = split * a.gps;
    const int g_end = (g_begin + a.gps < a.G) ? (g_begin + a.gps) : a.G;

    const uint32_t piece_off = (uint32_t)((slot >> 3) * 32 + 4 * c8 + kq);
    const uint32_t scale_off = (uint32_t)((slot >> 3) * 64 + 8 * c8);
    const u32x4* strip_w = a.B + (size_t)strip * 64 + (size_t)(2 * w) * N4;  // this wave's two rows of a group
    const half_t* strip_s = a.S + (size_t)strip * 128;

    // cooperative X tile load: thread t covers row (t / 16) + 16 p, 16-byte segment t % 16
    const int xr_row = tid >> 4;
    const int xr_seg = tid & 15;

    NibbleMagic magic;
    magic.init();

    f4 acc[MTILES][8];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt)
#pragma unroll
        for (int jb = 0; jb < 8; ++jb) acc[mt][jb] = f4{0.f, 0.f, 0.f, 0.f};

    u32x4 xv[MTILES];
    u32x4 wq[2];
    u32x4 sc;
    auto issue_loads = [&](int g) {
#pragma unroll
        for (int p = 0; p < MTILES; ++p) {
            const int m = m0 + xr_row + 16 * p;
            xv[p] = u32x4{0u, 0u, 0u, 0u};
            if (m < a.M) xv[p] = *reinterpret_cast<const u32x4*>(a.X + (size_t)m * a.ldx + 128 * g + 8 * xr_seg);
        }
        if (!a.per_column) {
            sc = *reinterpret_cast<const u32x4*>(strip_s + (size_t)g * a.N + scale_off);
        } else {
            uint32_t t[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int n0 = strip * 128 + (slot >> 3) * 64 + c8 + 8 * (2 * p), n1 = n0 + 8;
                const uint16_t lo = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n0));
                const uint16_t hi = *reinterpret_cast<const uint16_t*>(a.S + single_scale_pos(n1));
                t[p] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            sc = u32x4{t[0], t[1], t[2], t[3]};
        }
        const u32x4* rowp = strip_w + (size_t)(8 * g) * N4;
        wq[0] = rowp[piece_off];
        wq[1] = rowp[(size_t)N4 + piece_off];
    };
    auto stage_x = [&](int buf) {
        uint32_t* dst = lds + buf * BUF_DWORDS;
#pragma unroll
        for (int p = 0; p < MTILES; ++p)
            *reinterpret_cast<u32x4*>(dst + (xr_row + 16 * p) * kTileXsStride + 4 * xr_seg) = xv[p];
    };

    if (g_begin < g_end) {
        issue_loads(g_begin);
        stage_x(0);
    }
    __syncthreads();

    for (int g = g_begin; g < g_end; ++g) {
        const int buf = (g - g_begin) & 1;
        const u32x4 cur0 = wq[0], cur1 = wq[1];
        const u32x4 sc_cur = sc;
        if (g + 1 < g_end) issue_loads(g + 1);

        // A operands of this wave's 32-K slice, all M tiles
        const uint32_t* xs = lds + buf * BUF_DWORDS + 16 * w + kq;
        h8 xa[MTILES];
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const uint32_t* xr = xs + (mt * 16 + slot) * kTileXsStride;
            const h2 d0 = bits_to_h2(xr[0]), d1 = bits_to_h2(xr[4]);
            const h2 d2 = bits_to_h2(xr[8]), d3 = bits_to_h2(xr[12]);
            xa[mt] = h8{d0.x, d0.y, d1.x, d1.y, d2.x, d2.y, d3.x, d3.y};
        }

#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t q0 = cur0[j], q1 = cur1[j];
            const h2 pr = bits_to_h2(sc_cur[j]);
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const uint32_t p0 = blk ? (q0 >> 8) : q0;
                const uint32_t p1 = blk ? (q1 >> 8) : q1;
                const h2 sv = blk ? h2{pr.y, pr.y} : h2{pr.x, pr.x};
                const h2 e0 = magic.pair_low(p0) * sv, e1 = magic.pair_high(p0) * sv;
                const h2 e2 = magic.pair_low(p1) * sv, e3 = magic.pair_high(p1) * sv;
                const h8 bw = h8{e0.x, e0.y, e1.x, e1.y, e2.x, e2.y, e3.x, e3.y};
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt)
                    acc[mt][2 * j + blk] =
                        __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], bw, acc[mt][2 * j + blk], 0, 0, 0);
            }
        }

        if (g + 1 < g_end) stage_x(buf ^ 1);
        __syncthreads();
    }

    // ---- combine the four waves, one 16-row M tile at a time -------------------------------
    float* red = reinterpret_cast<float*>(lds);  // [4 waves][16 rows][128 columns]
    const int ncol_lane = 64 * (slot >> 3) + c8;
    const int col_out = tid & 127;
    const int n_out = 128 * strip + col_out;
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
        if (m0 + mt * 16 < a.M) {  // uniform
            if (mt > 0) __syncthreads();
#pragma unroll
            for (int jb = 0; jb < 8; ++jb)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    red[(w * 16 + 4 * kq + v) * 128 + ncol_lane + 16 * (jb >> 1) + 8 * (jb & 1)] = acc[mt][jb][v];
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int ml = (tid >> 7) + 2 * i;
                const int m = m0 + mt * 16 + ml;
                if (m < a.M) {
                    const float sum = (red[(0 * 16 + ml) * 128 + col_out] + red[(1 * 16 + ml) * 128 + col_out]) +
                                      (red[(2 * 16 + ml) * 128 + col_out] + red[(3 * 16 + ml) * 128 + col_out]);
                    float outv = sum;
                    bool emit = true;
                    unsigned long long* slot_ptr = nullptr;
                    if (a.splits > 1) {
                        const float v = fminf(fmaxf(sum, -kTileAccumClamp), kTileAccumClamp);
                        const long long fixed = __float2ll_rn(v * kTileAccumScale);
                        const unsigned long long word = ((unsigned long long)fixed << 8) + 1ull;
                        slot_ptr = a.accum + (size_t)m * a.N + n_out;
                        const unsigned long long old =
                            __hip_atomic_fetch_add(slot_ptr, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        emit = ((int)(old & 0xffull) == a.splits - 1);
                        outv = (float)((long long)(old + word) >> 8) * (1.0f / kTileAccumScale);
                    }
                    if (emit) {
                        if (a.out_f32)
                            reinterpret_cast<float*>(a.D)[(size_t)m * a.N + n_out] = outv;
                        else
                            reinterpret_cast<half_t*>(a.D)[(size_t)m * a.N + n_out] = (half_t)outv;
                        if (slot_ptr) __hip_atomic_store(slot_ptr, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------
static inline int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

struct TilePlan {
    int mtiles, splits, gps;
};
static TilePlan tile_plan(int m, int n, int k, int splits_override);

size_t tile_accum_bytes(int m, int n, int k) {
    // one word per output element, only when the plan splits K over workgroups
    return tile_plan(m, n, k, 0).splits > 1 ? (size_t)m * n * sizeof(unsigned long long) : 0;
}

static TilePlan tile_plan(int m, int n, int k, int splits_override) {
    TilePlan p;
    p.mtiles = m <= 32 ? 2 : (m <= 64 ? 4 : 8);
    const int G = k / 128;
    const int tiles = (n / 128) * ceil_div_i(m, 16 * p.mtiles);
    int splits = 1;
    if (splits_override > 0) {
        splits = splits_override;
    } else {
        // fill the 256 compute units, keep at least 4 K groups per workgroup
        while (tiles * splits < 256 && G / (splits * 2) >= 4 && splits < 64) splits *= 2;
    }
    if (splits > G) splits = G;
    if (splits > 255) splits = 255;
    p.gps = ceil_div_i(G, splits);
    p.splits = ceil_div_i(G, p.gps);
    return p;
}

template <int MTILES>
static hipError_t tile_launch_one(const TileArgs& a, int grid, hipStream_t stream) {
    const size_t stage = (size_t)2 * 16 * MTILES * kTileXsStride * 4;
    const size_t red = (size_t)4 * 16 * 128 * 4;
    const size_t shmem = stage > red ? stage : red;
    auto kern = &w4a16_tile_kernel<MTILES>;
    if (shmem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), shmem, stream, a);
    return hipGetLastError();
}

// tune: bits 0..7 force the number of K splits (0 = choose)
int tile_launch(const void* A, int64_t lda, const void* B, const void* S, void* D, void* accum, size_t accum_bytes,
                int m, int n, int k, int groups, bool out_f32, unsigned tune, hipStream_t stream) {
    const TilePlan plan = tile_plan(m, n, k, (int)(tune & 0xffu));
    if (plan.splits > 1 && (!accum || accum_bytes < (size_t)m * n * sizeof(unsigned long long)))
        return UNIQL_E_WORKSPACE;
    TileArgs a;
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
    a.mblocks = ceil_div_i(m, 16 * plan.mtiles);
    a.out_f32 = out_f32 ? 1 : 0;
    const int64_t grid = (int64_t)(n / 128) * a.mblocks * a.splits;
    if (grid > 0x7fffffffLL) return UNIQL_E_SHAPE;
    hipError_t e;
    if (plan.mtiles == 2) e = tile_launch_one<2>(a, (int)grid, stream);
    else if (plan.mtiles == 4) e = tile_launch_one<4>(a, (int)grid, stream);
    else e = tile_launch_one<8>(a, (int)grid, stream);
    return e == hipSuccess ? UNIQL_OK : UNIQL_E_LAUNCH;
}

}  // namespace uniql
